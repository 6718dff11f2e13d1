"""Operator-level mirror of the reference's GPU tensor engine for the hot path.

``Mi355Engine`` keeps the operator names and shape rules of ``IEngine`` /
``DirectGpuTensorEngine`` for the members on the path
(src/AiDotNet.Tensors/Engines/IEngine.cs:3186 TensorMatMul, :4133-4140 ScaledDotProductAttention,
:4587-4594 FlashAttention; routing src/AiDotNet.Tensors/Engines/DirectGpuTensorEngine.cs:19660-19857,
19987-20019, 10966-11089, 11436-11548) on device-resident ``torch`` tensors, and calls the backend
members of :class:`Mi355Backend`.  Unlike the reference there is no CPU fallback: a failure raises
(the behaviour of ``ThrowOnGpuKernelFallback = true``, DirectGpuTensorEngine.cs:19850-19856).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import weakref

import torch

from .backend import (ArgumentException, ArgumentNullException, ArgumentOutOfRangeException, Mi355Backend,
                      NotSupportedException)
from .precision import GpuPrecisionDiagnostics, GpuPrecisionOperation, GpuPrecisionPlanner, GpuScalarType, scalar_type_for

_KIND = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16"}


class Mi355Engine:
    def __init__(self, backend: Optional[Mi355Backend] = None):
        self.backend = backend or Mi355Backend()

    # ------------------------------------------------------------------ MatMul
    def _storage_as(self, t: torch.Tensor, storage: GpuScalarType) -> torch.Tensor:
        """``t`` in the storage type a plan asks for, converted on the device by the backend's converters when it differs
        (AllocateReducedPrecisionInput, DirectGpuTensorEngine.cs:19520-19545; the reference's upload widens 16-bit tensors)."""
        want = {GpuScalarType.Float32: torch.float32, GpuScalarType.Float16: torch.float16, GpuScalarType.BFloat16: torch.bfloat16}[storage]
        if t.dtype == want:
            return t
        be = self.backend
        if t.dtype != torch.float32 and want != torch.float32:                   # 16-bit -> the other 16-bit type: through fp32
            t = self._storage_as(t, GpuScalarType.Float32)
        out = torch.empty(t.shape, dtype=want, device=t.device)
        convert = {(torch.float32, torch.float16): be.ConvertToFp16, (torch.float32, torch.bfloat16): be.ConvertToBf16,
                   (torch.float16, torch.float32): be.ConvertToFp32, (torch.bfloat16, torch.float32): be.ConvertBf16ToFp32}[(t.dtype, want)]
        convert(be.WrapTensor(t), be.WrapTensor(out), t.numel())
        return out

    def TensorMatMul(self, a: torch.Tensor, b: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """rank-2 x rank-2, ND x 2D (leading dims collapse into M) and ND x ND of equal rank
        (batched), as CpuEngine.TensorMatMul (CpuEngine.cs:12458-12575).  The compute format comes from the precision
        planner under the current ``GpuExecutionPolicyScope`` (DirectGpuTensorEngine.cs:19660-19857 with ExecutePlannedGemm
        :19547-19590): by default 16-bit tensors multiply in their own type and fp32 tensors in fp32; an explicit Float16 /
        BFloat16 preference converts fp32 operands on the device and runs the fp32-output half GEMM.  Accumulation is always
        fp32.  The result has the operands' dtype (``out_dtype`` float32 keeps the fp32 accumulator of a 16-bit product)."""
        if a is None or b is None:
            raise ArgumentNullException("a" if a is None else "b")
        if a.dim() < 2 or b.dim() < 2:
            raise ArgumentException("TensorMatMul requires tensors of rank >= 2")
        if a.dtype != b.dtype or a.dtype not in _KIND:
            raise NotSupportedException("TensorMatMul: unsupported dtype combination %s x %s" % (a.dtype, b.dtype))
        if a.shape[-1] != b.shape[-2]:
            raise ArgumentException("inner dimensions do not match: %s x %s" % (tuple(a.shape), tuple(b.shape)))
        be = self.backend
        a = a.contiguous(); b = b.contiguous()
        K, N = b.shape[-2], b.shape[-1]
        out_dtype = out_dtype or a.dtype
        if b.dim() == 2:
            plan = GpuPrecisionPlanner.CreatePlan(a.dtype, GpuPrecisionOperation.MatMul, "TensorMatMul" if a.dim() == 2 else "TensorMatMul.NDx2D")
            M = a.numel() // K
            sa = self._storage_as(a, plan.InputStorage); sb = self._storage_as(b, plan.InputStorage)
            # a 16-bit result of a 16-bit product is the fp32 accumulator rounded once: the 16-bit-output kernels do that in their epilogue
            direct16 = sa.dtype != torch.float32 and out_dtype == sa.dtype
            out = torch.empty(*a.shape[:-1], N, dtype=out_dtype if (direct16 or out_dtype == torch.float32) else torch.float32, device=a.device)
            A, B, C = be.WrapTensor(sa), be.WrapTensor(sb), be.WrapTensor(out)
            if sa.dtype == torch.float32:
                be.Gemm(A, B, C, M, N, K)
            elif sa.dtype == torch.float16:
                (be.Hgemm if direct16 else be.GemmFp16In32fOut)(A, B, C, M, N, K)
            else:
                (be.Bf16Gemm if direct16 else be.GemmBf16In32fOut)(A, B, C, M, N, K)
            GpuPrecisionDiagnostics.Publish(plan)
            return out if out.dtype == out_dtype else self._storage_as(out, scalar_type_for(out_dtype))
        if a.dim() != b.dim() or a.shape[:-2] != b.shape[:-2]:
            raise ArgumentException("batched TensorMatMul needs equal leading dimensions")
        return self.BatchMatMul(a, b)

    def TensorMatMulCachedB(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """a [..., K] times a rank-2 weight b [K, N] that is expected again: b is packed once (backend.PackB) and the packed form
        is kept, keyed the way SimdGemm.SgemmWithCachedB keys its PrePackedB entries (SimdGemm.cs:292, 327-684: a
        ConditionalWeakTable on the identity of the weight array, collected with the array, plus the array's version; a changed
        weight is packed again) -- here the identity of the caller's tensor object, held through a weak reference that is
        compared on every hit and that drops the entry when the tensor dies, plus torch's in-place version counter.  A device
        address is never the key: the allocator hands a freed block to the next tensor of the same size.  A weight that is not
        contiguous (a transposed view) is packed from a temporary copy on every call and not cached.  Values are those of
        TensorMatMul.  At most ``CACHED_B_CAPACITY`` weights are kept, the least recently used one leaves first (the reference
        bounds its cache the same way, SimdGemm.cs:1030-1159)."""
        if a is None or b is None:
            raise ArgumentNullException("a" if a is None else "b")
        if b.dim() != 2 or a.dim() < 1:
            raise ArgumentException("TensorMatMulCachedB needs a rank-2 weight")
        if a.dtype != b.dtype or a.dtype not in _KIND:
            raise NotSupportedException("TensorMatMulCachedB: unsupported dtype combination %s x %s" % (a.dtype, b.dtype))
        if a.shape[-1] != b.shape[0]:
            raise ArgumentException("inner dimensions do not match: %s x %s" % (tuple(a.shape), tuple(b.shape)))
        be = self.backend
        a = a.contiguous()
        K, N = b.shape
        kind = _KIND[a.dtype]
        if not b.is_contiguous():
            packed = be.PackB(kind, be.WrapTensor(b.contiguous()), K, N)      # a temporary copy has no identity to key on
        else:
            cache = self.__dict__.setdefault("_packed_b", {})
            key = id(b)
            hit = cache.pop(key, None)
            if hit is None or hit[0]() is not b or hit[1] != b._version or hit[2] != (b.data_ptr(), K, N, b.dtype):
                owner = weakref.ref(b, lambda _r, c=cache, k=key: c.pop(k, None) if (k in c and c[k][0] is _r) else None)
                hit = (owner, b._version, (b.data_ptr(), K, N, b.dtype), be.PackB(kind, be.WrapTensor(b), K, N))
            cache[key] = hit                                                    # most recently used last
            while len(cache) > self.CACHED_B_CAPACITY:
                cache.pop(next(iter(cache)))
            packed = hit[3]
        M = a.numel() // K
        out = torch.empty(*a.shape[:-1], N, dtype=a.dtype, device=a.device)
        be.GemmPackedB(kind, be.WrapTensor(a), packed, None, be.WrapTensor(out), M, N, K, outputIsFp32=(a.dtype == torch.float32))
        return out

    CACHED_B_CAPACITY = 64

    def TensorMatMulTransposed(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """a [..., M, K] times the transpose of b stored [..., N, K] -> [..., M, N] (CpuEngine.cs:12337-12452 for the argument rules;
        DirectGpuTensorEngine.cs:19860-19905: rank 2 runs the backend's MatMulTransposed, which reads B in place with no transposed
        copy; other ranks materialise the transpose and take TensorMatMul).  The backend route is fp32: 16-bit tensors are widened
        on the device, as the reference's upload does, and the result returns in the operands' dtype."""
        if a is None or b is None:
            raise ArgumentNullException("a" if a is None else "b")
        if a.dim() < 2 or b.dim() < 2:
            raise ArgumentException("TensorMatMulTransposed requires rank >= 2 for both operands.")
        if a.dtype != b.dtype or a.dtype not in _KIND:
            raise NotSupportedException("TensorMatMulTransposed: unsupported dtype combination %s x %s" % (a.dtype, b.dtype))
        M, K, N, Kb = a.shape[-2], a.shape[-1], b.shape[-2], b.shape[-1]
        if K != Kb:
            raise ArgumentException("TensorMatMulTransposed K mismatch: a's trailing dim %d != b's trailing dim %d." % (K, Kb))
        if a.dim() != 2 or b.dim() != 2:
            return self.TensorMatMul(a, b.transpose(-1, -2).contiguous())
        plan = GpuPrecisionPlanner.CreatePlan(a.dtype, GpuPrecisionOperation.MatMulTransposed, "TensorMatMulTransposed")
        if plan.InputStorage != GpuScalarType.Float32:
            raise NotSupportedException("The selected %s transposed GEMM route has no backend dispatch implementation." % plan.InputStorage.name)
        be = self.backend
        sa = self._storage_as(a.contiguous(), GpuScalarType.Float32); sb = self._storage_as(b.contiguous(), GpuScalarType.Float32)
        out = torch.empty(M, N, dtype=torch.float32, device=a.device)
        be.MatMulTransposed(be.WrapTensor(sa), be.WrapTensor(sb), be.WrapTensor(out), M, N, K)
        GpuPrecisionDiagnostics.Publish(plan)
        return out if a.dtype == torch.float32 else self._storage_as(out, scalar_type_for(a.dtype))

    _ACTIVATIONS = {"None": 0, "ReLU": 1, "GELU": 2, "Sigmoid": 3, "Tanh": 4, "LeakyReLU": 5, "Swish": 6}

    def FusedLinear(self, input: torch.Tensor, weights: torch.Tensor, bias: Optional[torch.Tensor] = None,
                    activation="None", alpha: float = 0.01, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """activation(input @ weights + bias): input [..., K] (leading dims collapse), weights [K, N], bias [N] or
        None (IEngine.cs:5166; CpuEngine FusedLinear: GEMM, then the bias + activation epilogue of
        Helpers/CpuFusedOperations.cs:590-700).  activation is a FusedActivationType name or number 0..6; alpha is
        the LeakyReLU slope.  fp16 / bf16 inputs take an fp32 bias and accumulate in fp32."""
        if input is None or weights is None:
            raise ArgumentNullException("input" if input is None else "weights")
        if weights.dim() != 2 or input.dim() < 2:
            raise ArgumentException("FusedLinear needs input of rank >= 2 and weights of rank 2")
        if input.dtype != weights.dtype or input.dtype not in _KIND:
            raise NotSupportedException("FusedLinear: unsupported dtype combination %s x %s" % (input.dtype, weights.dtype))
        K, N = weights.shape
        if input.shape[-1] != K:
            raise ArgumentException("Weight matrix shape mismatch: expected [%d, N], got %s" % (input.shape[-1], tuple(weights.shape)))
        act = self._ACTIVATIONS.get(activation, activation) if isinstance(activation, str) else int(activation)
        if not isinstance(act, int) or not 0 <= act <= 6:
            raise NotSupportedException("FusedLinear: activation %r has no fused epilogue" % (activation,))
        if bias is not None and (bias.dim() != 1 or bias.shape[0] != N):
            raise ArgumentException("bias must have N = %d elements" % N)
        be = self.backend
        a = input.contiguous(); w = weights.contiguous()
        M = a.numel() // K
        bb = be.WrapTensor(bias.to(torch.float32).contiguous()) if bias is not None else None
        if a.dtype == torch.float32:
            out = torch.empty(*a.shape[:-1], N, dtype=torch.float32, device=a.device)
            be.GemmBiasActivationInto(be.WrapTensor(a), be.WrapTensor(w), bb, be.WrapTensor(out), M, N, K, act, alpha)
            return out
        out_dtype = out_dtype or a.dtype
        out = torch.empty(*a.shape[:-1], N, dtype=out_dtype, device=a.device)
        be.GemmBiasActivationHalf(_KIND[a.dtype], be.WrapTensor(a), be.WrapTensor(w), bb, be.WrapTensor(out), M, N, K, act, alpha,
                                  outputIsFp32=out_dtype == torch.float32)
        return out

    def TensorMatMulFp16WeightB(self, a: torch.Tensor, bFp16: torch.Tensor) -> torch.Tensor:
        """fp32 activations [..., K] x fp16 weights [K, N] -> fp32 [..., N] (CpuEngine.TensorMatMulFp16WeightB ->
        SimdGemm.SgemmFp16WeightB, Engines/Simd/SimdGemm.Fp16Weight.cs:22-91)."""
        return self.FusedLinearFp16WeightB(a, bFp16, None, "None")

    def FusedLinearFp16WeightB(self, input: torch.Tensor, weightsFp16: torch.Tensor, bias: Optional[torch.Tensor] = None,
                               activation="None", alpha: float = 0.01) -> torch.Tensor:
        """activation(input @ widen(weightsFp16) + bias) in fp32 with fp16-stored weights (CpuEngine.FusedLinearFp16WeightB)."""
        if input is None or weightsFp16 is None:
            raise ArgumentNullException("input" if input is None else "weightsFp16")
        if input.dtype != torch.float32 or weightsFp16.dtype != torch.float16:
            raise NotSupportedException("Fp16WeightB: fp32 activations and fp16 weights are required")
        if weightsFp16.dim() != 2 or input.dim() < 1 or input.shape[-1] != weightsFp16.shape[0]:
            raise ArgumentException("Fp16WeightB: input [..., K] (or [K]) and weights [K, N] are required")
        act = self._ACTIVATIONS.get(activation, activation) if isinstance(activation, str) else int(activation)
        if not isinstance(act, int) or not 0 <= act <= 6:
            raise NotSupportedException("Fp16WeightB: activation %r has no fused epilogue" % (activation,))
        K, N = weightsFp16.shape
        if bias is not None and (bias.dim() != 1 or bias.shape[0] != N):
            raise ArgumentException("bias must have N = %d elements" % N)
        be = self.backend
        a = input.contiguous(); w = weightsFp16.contiguous()
        M = a.numel() // K
        out = torch.empty(*a.shape[:-1], N, dtype=torch.float32, device=a.device)
        bb = be.WrapTensor(bias.to(torch.float32).contiguous()) if bias is not None else None
        be.GemmFp16WeightB(be.WrapTensor(a), be.WrapTensor(w), bb, be.WrapTensor(out), M, N, K, act, alpha)
        return out

    def BatchMatMul(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """[..., M, K] x [..., K, N], fp32 (DirectGpuTensorEngine.cs:19987-20019 -> BatchedGemm)."""
        if a.dtype != torch.float32 or b.dtype != torch.float32:
            raise NotSupportedException("BatchMatMul is fp32 only (as the reference's batched route)")
        # the batched backend contract is fp32: a reduced-precision preference resolves to Float32 here or is refused
        # (ExecutePlannedBatchedGemm, DirectGpuTensorEngine.cs:19592-19624)
        plan = GpuPrecisionPlanner.CreatePlan(a.dtype, GpuPrecisionOperation.BatchMatMul, "BatchMatMul")
        if plan.InputStorage != GpuScalarType.Float32:
            raise NotSupportedException("No batched GEMM dispatch exists for %s storage." % plan.InputStorage.name)
        a = a.contiguous(); b = b.contiguous()
        M, K, N = a.shape[-2], a.shape[-1], b.shape[-1]
        batch = a.numel() // (M * K)
        out = torch.empty(*a.shape[:-2], M, N, dtype=torch.float32, device=a.device)
        be = self.backend
        be.BatchedGemm(be.WrapTensor(a), be.WrapTensor(b), be.WrapTensor(out), M, N, K, batch)
        GpuPrecisionDiagnostics.Publish(plan)
        return out

    # ------------------------------------------------------------------ attention
    def FlashAttention(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, scale: Optional[float] = None,
                       isCausal: bool = False, attentionBias: Optional[torch.Tensor] = None,
                       queryOffset: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
        """[B,H,Sq,d] x [B,H,Sk,d] -> (O [B,H,Sq,d], LSE [B,H,Sq]); top-left causal rule shifted by
        queryOffset (IEngine.cs:4587-4594; CpuEngine.cs:28748, 29146-29288).  16-bit inputs give an
        fp32 O and LSE."""
        for t, n in ((query, "query"), (key, "key"), (value, "value")):
            if t is None:
                raise ArgumentNullException(n)
            if t.dim() != 4:
                raise ArgumentException("%s must be rank 4 [B,H,S,d]" % n)
        B, H, Sq, D = query.shape
        Sk = key.shape[2]
        if key.shape != value.shape or key.shape[0] != B or key.shape[3] != D:
            raise ArgumentException("key/value shapes do not match the query")
        if isCausal and queryOffset != 0 and queryOffset + Sq > Sk:
            # the offset form is rejected when it runs past the keys (FusedAttentionAuditTests.cs:81-92);
            # plain top-left causal with Sq > Sk is legal for IEngine.FlashAttention (CpuEngine.cs:29235)
            raise ArgumentException("queryOffset + Sq exceeds Sk")
        if scale is None:
            scale = 1.0 / math.sqrt(D)
        be = self.backend
        q = query.contiguous(); k = key.contiguous(); v = value.contiguous()
        out = torch.empty(B, H, Sq, D, dtype=torch.float32, device=q.device)
        lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device)
        kind = _KIND.get(q.dtype)
        if kind is None:
            raise NotSupportedException("unsupported dtype %s" % q.dtype)
        if kind == "f32" and queryOffset == 0 and key.shape[1] == H:
            bias = None
            bstride = 0
            if attentionBias is not None:
                bias = be.WrapTensor(attentionBias.contiguous().float())
                bstride = H * Sq * Sk if attentionBias.dim() == 4 else 0
            be.FlashAttentionV2(be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out), be.WrapTensor(lse),
                                B, H, Sq, Sk, D, scale, isCausal, bias, bstride)
        else:
            if attentionBias is not None:
                raise NotSupportedException("attention bias is available on the fp32 route only")
            if kind == "f32":
                from ._lib import AttnDesc
                d = AttnDesc(B=B, H=H, Hkv=key.shape[1], Sq=Sq, Sk=Sk, D=D, scale=scale, causal=int(isCausal),
                             causal_query_offset=queryOffset)
                be._attn("f32", be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out), be.WrapTensor(lse),
                         None, None, None, d)
            else:
                be.FlashAttentionHalf(kind, be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out),
                                      be.WrapTensor(lse), B, H, Sq, Sk, D, scale, isCausal, queryOffset, key.shape[1])
        return out, lse

    def MultiHeadAttentionForward(self, input: torch.Tensor, qWeight: torch.Tensor, kWeight: torch.Tensor, vWeight: torch.Tensor,
                                  outWeight: torch.Tensor, numHeads: int, mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """input [B, seq, dModel], four [dModel, dModel] projections, optional boolean keep-mask broadcastable to
        [B, H, seq, seq] -> [B, seq, dModel]; inference only (CpuEngine.MultiHeadAttention.cs:68-143 for the argument rules).
        fp32, fp16 and bf16 tensors are accepted; the output has the input's dtype."""
        for t, n in ((input, "input"), (qWeight, "qWeight"), (kWeight, "kWeight"), (vWeight, "vWeight"), (outWeight, "outWeight")):
            if t is None:
                raise ArgumentNullException(n)
        if input.dim() != 3:
            raise ArgumentException("MultiHeadAttentionForward expects rank-3 input [B, seq, dModel]; got rank %d." % input.dim())
        if numHeads <= 0:
            raise ArgumentOutOfRangeException("numHeads must be positive.")
        B, S, dM = input.shape
        if dM % numHeads != 0:
            raise ArgumentException("dModel (%d) must be divisible by numHeads (%d)." % (dM, numHeads))
        for w, n in ((qWeight, "qWeight"), (kWeight, "kWeight"), (vWeight, "vWeight"), (outWeight, "outWeight")):
            if w.dim() != 2 or w.shape[0] != dM or w.shape[1] != dM:
                raise ArgumentException("%s must be [%d, %d]." % (n, dM, dM))
            if w.dtype != input.dtype:
                raise NotSupportedException("MultiHeadAttentionForward: %s dtype differs from the input's" % n)
        if input.dtype not in _KIND:
            raise NotSupportedException("MultiHeadAttentionForward: unsupported dtype %s" % input.dtype)
        be = self.backend
        m = None
        if mask is not None:
            if mask.dim() != 4:
                raise ArgumentException("mask must be rank 4, broadcastable to [B,H,seq,seq]")
            shared = mask.shape[0] == 1 and mask.shape[1] == 1
            full = mask.expand(1 if shared else B, 1 if shared else numHeads, S, S)
            m = be.WrapTensor(full.to(torch.float32).contiguous().reshape(-1))
        out = torch.empty(B, S, dM, dtype=input.dtype, device=input.device)
        W = be.WrapTensor
        be.MultiHeadAttentionForward(_KIND[input.dtype], W(input.contiguous()), W(qWeight.contiguous()), W(kWeight.contiguous()),
                                     W(vWeight.contiguous()), W(outWeight.contiguous()), m, W(out), B, S, dM, numHeads)
        return out

    def ScaledDotProductAttention(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                  mask: Optional[torch.Tensor] = None, scale: Optional[float] = None,
                                  softcap: float = 0.0, isCausal: bool = False,
                                  returnWeights: bool = True) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        """fp32 SDPA with an optional boolean keep-mask broadcastable to [B,H,Sq,Sk] (true = keep) and
        soft-cap; returns (O, weights) (IEngine.cs:4133-4140; CpuEngine.cs:27376, 27695-27881; GPU
        route DirectGpuTensorEngine.MissingKernels.cs:6085-6140).  GQA is inferred from key.shape[1];
        the causal rule is bottom-right (DirectGpuTensorEngine.cs:11501)."""
        if query is None or key is None or value is None:
            raise ArgumentNullException("query/key/value")
        if query.dim() != 4 or query.dtype != torch.float32:
            raise NotSupportedException("ScaledDotProductAttention GPU route is float + rank 4 only")
        B, H, Sq, D = query.shape
        Hkv, Sk = key.shape[1], key.shape[2]
        if scale is None:
            scale = 1.0 / math.sqrt(D)
        be = self.backend
        q = query.contiguous(); k = key.contiguous(); v = value.contiguous()
        out = torch.empty(B, H, Sq, D, dtype=torch.float32, device=q.device)
        w = torch.empty(B, H, Sq, Sk, dtype=torch.float32, device=q.device) if returnWeights else None
        m = None
        if mask is not None:
            if mask.dim() != 4:
                raise ArgumentException("mask must be rank 4, broadcastable to [B,H,Sq,Sk]")
            shared = mask.shape[0] == 1 and mask.shape[1] == 1
            full = mask.expand(1 if shared else B, 1 if shared else H, Sq, Sk)
            m = be.WrapTensor(full.to(torch.float32).contiguous().reshape(-1))
        be.ScaledDotProductAttention(be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out),
                                     be.WrapTensor(w) if w is not None else None, m, B, H, Sq, Sk, D, scale,
                                     isCausal, softcap, Hkv)
        return out, w
