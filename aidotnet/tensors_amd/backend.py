"""Host-side mirror of the reference's GPU-backend slot for the GEMM / attention hot path.

``Mi355Backend`` keeps the member names, argument order, defaults and error behaviour of
``IDirectGpuBackend`` (src/AiDotNet.Tensors/Engines/DirectGpu/IDirectGpuBackend.cs:160-222,
1395-1471, 1876-1911) and ``IGpuHalfPrecisionBackend``
(src/AiDotNet.Tensors/Engines/Gpu/IGpuHalfPrecisionBackend.cs:21-114) for the members on the
path, and forwards each to one C-ABI call of ``libaidotnet_mi355.so`` -- exactly what a C#
``DelegatingGpuBackend`` subclass would do by P/Invoke.  The reference is C# and cannot be
built where this runs, so this module is its stand-in above the C ABI; PyTorch is used only to
own device memory and the stream.

Exceptions mirror the managed ones by name (``ArgumentNullException`` ...), raised before the
native call for the same conditions the managed backend checks
(HipBackend.HalfPrecision.cs:167-177, HipBackend.cs:6123-6141, GpuKernelGuards.cs:12-68).
Every op synchronises before returning unless ``synchronous=False`` (the reference's
contract: HipBackend.cs:1444-1446).
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import AttnDesc


class ArgumentException(ValueError):
    pass


class ArgumentNullException(ArgumentException):
    pass


class ArgumentOutOfRangeException(ArgumentException):
    pass


class InvalidOperationException(RuntimeError):
    pass


class NotSupportedException(RuntimeError):
    pass


class HipException(RuntimeError):
    """A non-zero status from the native library (HipNativeBindings.CheckError, :646-654)."""

    def __init__(self, status: int, message: str):
        super().__init__("native status %d: %s" % (status, message))
        self.status = status


MAX_HEAD_DIM = 256   # GpuKernelGuards.MaxHeadDim (GpuKernelGuards.cs:12)


class GpuBuffer:
    """``IGpuBuffer`` (IDirectGpuBackend.cs:3776-3803): ``Size`` in elements for float buffers and
    in bytes for byte buffers, ``SizeInBytes``, ``Handle`` = raw device pointer."""

    def __init__(self, tensor: torch.Tensor, is_bytes: bool = False):
        if not tensor.is_contiguous():
            raise ArgumentException("buffer storage must be contiguous")
        self.tensor = tensor
        self._is_bytes = is_bytes

    @property
    def Size(self) -> int:
        return self.tensor.numel() * self.tensor.element_size() if self._is_bytes else self.tensor.numel()

    @property
    def SizeInBytes(self) -> int:
        return self.tensor.numel() * self.tensor.element_size()

    @property
    def Handle(self) -> int:
        return self.tensor.data_ptr()

    def Dispose(self) -> None:
        self.tensor = None


class Mi355Backend:
    """The GEMM / attention members of the backend slot, backed by hand-written gfx950 kernels."""

    BackendName = "HIP-MI355X"

    def __init__(self, device: int = 0, synchronous: bool = True, validate_block_tables: Optional[bool] = None):
        # validate_block_tables: read every block table back to the host and check its ids against the pool before a paged
        # call (a device-to-host copy and a stream synchronisation per call; the reference's guard checks capacities only,
        # GpuKernelGuards.cs:83-100).  The kernels index the pools with the ids unchecked, so a bad id is an out-of-bounds
        # device read: None (the default) checks whenever the current stream is not being captured into a graph, True always
        # (a capture then fails on the copy), False never (launch-only calls; the caller vouches for the table).
        self.ValidateBlockTables = validate_block_tables
        self._lib = _lib.load()
        if not torch.cuda.is_available():
            raise InvalidOperationException("no HIP device visible")
        self.device = torch.device("cuda", device)
        torch.cuda.set_device(self.device)
        ctx = ctypes.c_void_p()
        st = self._lib.aidn_mi355_create(device, ctypes.byref(ctx))
        if st != 0:
            raise InvalidOperationException("aidn_mi355_create failed with status %d (a gfx950 device is required)" % st)
        self._ctx = ctx
        self.synchronous = synchronous
        self.IsAvailable = True

    # ------------------------------------------------------------------ plumbing
    def Dispose(self) -> None:
        if getattr(self, "_ctx", None):
            self._lib.aidn_mi355_destroy(self._ctx)
            self._ctx = None
            self.IsAvailable = False

    def __del__(self):
        try:
            self.Dispose()
        except Exception:
            pass

    def _stream(self) -> ctypes.c_void_p:
        return ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    def _check(self, status: int) -> None:
        if status != 0:
            msg = self._lib.aidn_mi355_last_error(self._ctx).decode("utf-8", "replace")
            if status == _lib.AIDN_ERR_INVALID_ARGUMENT:
                raise ArgumentException(msg)
            if status == _lib.AIDN_ERR_UNSUPPORTED:
                raise NotSupportedException(msg)
            if status == _lib.AIDN_ERR_WORKSPACE:
                raise InvalidOperationException(msg)
            raise HipException(status, msg)

    def _done(self) -> None:
        if self.synchronous:
            self.Synchronize()

    def Synchronize(self) -> None:
        self._check(self._lib.aidn_mi355_sync(self._ctx, self._stream()))

    def SetGemmTile(self, tile: int) -> None:
        """Test hook: force the GEMM tile edge (0 = automatic)."""
        self._check(self._lib.aidn_mi355_set_gemm_tile(self._ctx, tile))

    def SetAttentionFastPath(self, enabled) -> None:
        """Test hook: False routes every attention shape through the general kernel; 2 / 3 keep the fast paths and pin unsplit
        head-dimension-128 prefill to the phase-structured / the software-pipelined kernel (True: chosen by pass length); at head
        dimension 256, 2 pins the older 32-key-tile form in place of the 64-key-tile kernel."""
        self._check(self._lib.aidn_mi355_set_attention_fast_path(self._ctx, int(enabled) if enabled in (2, 3) and enabled is not True else (1 if enabled else 0)))

    def ReserveWorkspace(self, size_in_bytes: int) -> None:
        """Grow the library workspace of the current stream now, so that later calls on it allocate nothing (needed before a
        call sequence is captured into a HIP graph).  No counterpart in the reference."""
        if size_in_bytes < 0:
            raise ArgumentOutOfRangeException("size must not be negative")
        self._check(self._lib.aidn_mi355_reserve_workspace(self._ctx, self._stream(), int(size_in_bytes)))

    def WorkspaceBytes(self) -> int:
        """Current size of the library workspace of the current stream."""
        return int(self._lib.aidn_mi355_workspace_bytes(self._ctx, self._stream()))

    def ReleaseStreamWorkspace(self) -> None:
        """Waits for the current stream and frees the workspace the library holds for it (for callers that create and destroy
        streams; graphs captured from the stream must not be replayed afterwards).  No counterpart in the reference."""
        self._check(self._lib.aidn_mi355_release_stream_workspace(self._ctx, self._stream()))

    # buffers -- AllocateBuffer zero-fills (HipBackend.cs:1251-1273)
    def AllocateBuffer(self, data_or_size) -> GpuBuffer:
        if isinstance(data_or_size, int):
            if data_or_size <= 0:
                raise ArgumentOutOfRangeException("size must be positive")
            return GpuBuffer(torch.zeros(data_or_size, dtype=torch.float32, device=self.device))
        t = torch.as_tensor(data_or_size, dtype=torch.float32).reshape(-1).contiguous()
        return GpuBuffer(t.to(self.device))

    def AllocateByteBuffer(self, size_in_bytes: int) -> GpuBuffer:
        if size_in_bytes <= 0:
            raise ArgumentOutOfRangeException("size must be positive")
        return GpuBuffer(torch.zeros(size_in_bytes, dtype=torch.uint8, device=self.device), is_bytes=True)

    def WrapTensor(self, t: torch.Tensor) -> GpuBuffer:
        """View an existing device tensor as a buffer (no copy); 16-bit tensors count as byte buffers."""
        return GpuBuffer(t, is_bytes=t.element_size() != 4)

    def DownloadBuffer(self, buf: GpuBuffer) -> torch.Tensor:
        self.Synchronize()
        return buf.tensor.detach().cpu()

    # ------------------------------------------------------------------ checks
    @staticmethod
    def _need(buf: Optional[GpuBuffer], name: str) -> GpuBuffer:
        if buf is None:
            raise ArgumentNullException(name)
        return buf

    @staticmethod
    def _positive(**dims) -> None:
        for k, v in dims.items():
            if v <= 0:
                raise ArgumentOutOfRangeException("%s: Dimensions must be positive." % k)

    @staticmethod
    def _capacity(buf: GpuBuffer, required_bytes: int, name: str, op: str) -> None:
        # GpuKernelGuards.Capacity (GpuKernelGuards.cs:61-68), in bytes so 16-bit buffers work too
        if buf.SizeInBytes < required_bytes:
            raise ArgumentException("%s: %s holds %d bytes but the kernel needs %d." % (op, name, buf.SizeInBytes, required_bytes))

    # ------------------------------------------------------------------ GEMM (fp32)
    def Gemm(self, A: GpuBuffer, B: GpuBuffer, C: GpuBuffer, M: int, N: int, K: int,
             alpha: float = 1.0, beta: float = 0.0) -> None:
        """C = alpha * A * B + beta * C, row-major fp32 (IDirectGpuBackend.cs:160-172)."""
        self._gemm(A, B, C, M, N, K, alpha, beta, 0, "Gemm")

    def MatMulTransposed(self, A: GpuBuffer, B: GpuBuffer, C: GpuBuffer, M: int, N: int, K: int,
                         alpha: float = 1.0, beta: float = 0.0) -> None:
        """C = A * B^T with B stored [N, K] (IDirectGpuBackend.cs:184-203)."""
        self._gemm(A, B, C, M, N, K, alpha, beta, 1, "MatMulTransposed")

    def _gemm(self, A, B, C, M, N, K, alpha, beta, transB, op):
        self._need(A, "A"); self._need(B, "B"); self._need(C, "C")
        self._positive(M=M, N=N, K=K)
        self._capacity(A, M * K * 4, "A", op); self._capacity(B, K * N * 4, "B", op); self._capacity(C, M * N * 4, "C", op)
        self._check(self._lib.aidn_mi355_sgemm(self._ctx, self._stream(), A.Handle, B.Handle, C.Handle,
                                               M, N, K, alpha, beta, transB))
        self._done()

    def MatMul(self, A: GpuBuffer, B: GpuBuffer, M: int, N: int, K: int) -> GpuBuffer:
        """Allocates C and returns it (IDirectGpuBackend.cs:174-183; HipBackend.cs:1592-1597)."""
        self._positive(M=M, N=N, K=K)
        C = self.AllocateBuffer(M * N)
        self.Gemm(A, B, C, M, N, K, 1.0, 0.0)
        return C

    def BatchedGemm(self, A: GpuBuffer, B: GpuBuffer, C: GpuBuffer, M: int, N: int, K: int, batchCount: int,
                    alpha: float = 1.0, beta: float = 0.0) -> None:
        """C[i] = alpha * A[i] * B[i] + beta * C[i] on concatenated matrices (IDirectGpuBackend.cs:205-222)."""
        if batchCount <= 0:
            raise ArgumentException("Batch count must be positive")      # HipBackend.cs:1601-1602
        self._need(A, "A"); self._need(B, "B"); self._need(C, "C")
        self._positive(M=M, N=N, K=K)
        self._capacity(A, batchCount * M * K * 4, "A", "BatchedGemm")
        self._capacity(B, batchCount * K * N * 4, "B", "BatchedGemm")
        self._capacity(C, batchCount * M * N * 4, "C", "BatchedGemm")
        self._check(self._lib.aidn_mi355_sgemm_batched(self._ctx, self._stream(), A.Handle, B.Handle, C.Handle,
                                                       M, N, K, batchCount, alpha, beta))
        self._done()

    # ------------------------------------------------------------------ fused projection epilogues
    # FusedActivationType numbering (src/AiDotNet.Tensors/Engines/FusedActivationType.cs:23-70)
    ACT_NONE, ACT_RELU, ACT_GELU, ACT_SIGMOID, ACT_TANH, ACT_LEAKY_RELU, ACT_SWISH = range(7)

    def GemmBiasActivationInto(self, A: GpuBuffer, B: GpuBuffer, bias: Optional[GpuBuffer], C: GpuBuffer,
                               M: int, N: int, K: int, activation: int = 0, alpha: float = 0.0) -> None:
        """C = act(A * B + bias) in one kernel, fp32 (the work of GemmBias + an activation kernel,
        HipBackend.cs:1637-1785, without the intermediate buffers)."""
        op = "GemmBiasActivation"
        self._need(A, "A"); self._need(B, "B"); self._need(C, "C")
        self._positive(M=M, N=N, K=K)
        self._capacity(A, M * K * 4, "A", op); self._capacity(B, K * N * 4, "B", op); self._capacity(C, M * N * 4, "C", op)
        if bias is not None:
            self._capacity(bias, N * 4, "bias", op)
        self._check(self._lib.aidn_mi355_sgemm_bias_act(self._ctx, self._stream(), A.Handle, B.Handle,
                                                        bias.Handle if bias is not None else None, C.Handle,
                                                        M, N, K, int(activation), float(alpha)))
        self._done()

    def _gemm_bias(self, A, B, bias, M, N, K, activation, alpha=0.0) -> GpuBuffer:
        self._need(bias, "bias")
        self._positive(M=M, N=N, K=K)
        C = self.AllocateBuffer(M * N)
        self.GemmBiasActivationInto(A, B, bias, C, M, N, K, activation, alpha)
        return C

    def GemmBias(self, A: GpuBuffer, B: GpuBuffer, bias: GpuBuffer, M: int, N: int, K: int) -> GpuBuffer:
        """output = A * B + bias, bias broadcast across the M rows (IDirectGpuBackend.cs:254-265)."""
        return self._gemm_bias(A, B, bias, M, N, K, self.ACT_NONE)

    def GemmBiasRelu(self, A: GpuBuffer, B: GpuBuffer, bias: GpuBuffer, M: int, N: int, K: int) -> GpuBuffer:
        """ReLU(A * B + bias) (IDirectGpuBackend.cs:227-237)."""
        return self._gemm_bias(A, B, bias, M, N, K, self.ACT_RELU)

    def GemmBiasGelu(self, A: GpuBuffer, B: GpuBuffer, bias: GpuBuffer, M: int, N: int, K: int) -> GpuBuffer:
        """GELU(A * B + bias), tanh form (IDirectGpuBackend.cs:239-242; HipActivationKernels.cs:44-54)."""
        return self._gemm_bias(A, B, bias, M, N, K, self.ACT_GELU)

    def GemmBiasSigmoid(self, A: GpuBuffer, B: GpuBuffer, bias: GpuBuffer, M: int, N: int, K: int) -> GpuBuffer:
        return self._gemm_bias(A, B, bias, M, N, K, self.ACT_SIGMOID)

    def GemmBiasTanh(self, A: GpuBuffer, B: GpuBuffer, bias: GpuBuffer, M: int, N: int, K: int) -> GpuBuffer:
        return self._gemm_bias(A, B, bias, M, N, K, self.ACT_TANH)

    def GemmBiasSwish(self, A: GpuBuffer, B: GpuBuffer, bias: GpuBuffer, M: int, N: int, K: int) -> GpuBuffer:
        """x * sigmoid(x) of A * B + bias (IDirectGpuBackend.cs:267-270)."""
        return self._gemm_bias(A, B, bias, M, N, K, self.ACT_SWISH)

    def GemmBiasLeakyRelu(self, A: GpuBuffer, B: GpuBuffer, bias: GpuBuffer, M: int, N: int, K: int,
                          alpha: float = 0.01) -> GpuBuffer:
        """LeakyReLU(A * B + bias, alpha) (IDirectGpuBackend.cs:272-275)."""
        return self._gemm_bias(A, B, bias, M, N, K, self.ACT_LEAKY_RELU, alpha)

    def GemmFp16WeightB(self, A: GpuBuffer, bFp16: GpuBuffer, bias: Optional[GpuBuffer], C: GpuBuffer,
                        M: int, N: int, K: int, activation: int = 0, alpha: float = 0.0) -> None:
        """C = act(A * widen(B) + bias) with fp32 A, fp16 weights B [K,N] and fp32 C: the weight-only fp16 GEMM of
        SimdGemm.SgemmFp16WeightB (Engines/Simd/SimdGemm.Fp16Weight.cs:22-91).  No member of this name exists in the
        reference's GPU interface."""
        op = "GemmFp16WeightB"
        self._need(A, "A"); self._need(bFp16, "bFp16"); self._need(C, "C")
        self._positive(M=M, N=N, K=K)
        self._capacity(A, M * K * 4, "A", op); self._capacity(bFp16, K * N * 2, "bFp16", op); self._capacity(C, M * N * 4, "C", op)
        if bias is not None:
            self._capacity(bias, N * 4, "bias", op)
        self._check(self._lib.aidn_mi355_sgemm_f16weight(self._ctx, self._stream(), A.Handle, bFp16.Handle,
                                                         bias.Handle if bias is not None else None, C.Handle,
                                                         M, N, K, int(activation), float(alpha)))
        self._done()

    def GemmBiasActivationHalf(self, kind: str, a: GpuBuffer, b: GpuBuffer, bias: Optional[GpuBuffer], c: GpuBuffer,
                               m: int, n: int, k: int, activation: int = 0, alpha: float = 0.0,
                               outputIsFp32: bool = False) -> None:
        """16-bit A and B ("f16" / "bf16"), fp32 bias, fp32 accumulation and epilogue, output fp32 or the input
        type.  No member of this name exists in the reference interface (its fused epilogues are fp32 only)."""
        fn = {"f16": self._lib.aidn_mi355_hgemm_bias_act, "bf16": self._lib.aidn_mi355_bf16gemm_bias_act}.get(kind)
        if fn is None:
            raise NotSupportedException("GemmBiasActivationHalf: kind must be 'f16' or 'bf16'")
        op = "GemmBiasActivationHalf"
        self._need(a, "a"); self._need(b, "b"); self._need(c, "c")
        self._positive(m=m, n=n, k=k)
        self._capacity(a, m * k * 2, "a", op); self._capacity(b, k * n * 2, "b", op)
        self._capacity(c, m * n * (4 if outputIsFp32 else 2), "c", op)
        if bias is not None:
            self._capacity(bias, n * 4, "bias", op)
        self._check(fn(self._ctx, self._stream(), a.Handle, b.Handle, bias.Handle if bias is not None else None, c.Handle,
                       1 if outputIsFp32 else 0, m, n, k, int(activation), float(alpha)))
        self._done()

    # ------------------------------------------------------------------ pre-packed weight operand
    _PACK_KIND = {"f32": 0, "f16": 1, "bf16": 2}

    def PackB(self, kind: str, B: GpuBuffer, K: int, N: int, transB: bool = False) -> GpuBuffer:
        """Packs a weight matrix once for GemmPackedB -- the GPU form of the reference's cached packed B
        (``SimdGemm.SgemmWithCachedB`` / ``PrePackedB``, src/AiDotNet.Tensors/Engines/Simd/SimdGemm.cs:327-684, 1030-1159).
        Returns a byte buffer the caller owns; repack when the weight changes."""
        if kind not in self._PACK_KIND:
            raise NotSupportedException("PackB: kind must be 'f32', 'f16' or 'bf16'")
        self._need(B, "B"); self._positive(K=K, N=N)
        es = 4 if kind == "f32" else 2
        self._capacity(B, K * N * es, "B", "PackB")
        nbytes = int(self._lib.aidn_mi355_packed_b_bytes(self._PACK_KIND[kind], K, N, 1 if transB else 0))
        if nbytes <= 0:
            raise NotSupportedException("PackB: no packed layout for this kind / shape")
        packed = self.AllocateByteBuffer(nbytes)
        self._check(self._lib.aidn_mi355_pack_b(self._ctx, self._stream(), self._PACK_KIND[kind], B.Handle, K, N,
                                                1 if transB else 0, packed.Handle))
        self._done()
        return packed

    def GemmPackedB(self, kind: str, A: GpuBuffer, packedB: GpuBuffer, bias: Optional[GpuBuffer], C: GpuBuffer,
                    M: int, N: int, K: int, transB: bool = False, activation: int = 0, alpha: float = 0.0,
                    outputIsFp32: bool = True) -> None:
        """C = act(A * B + bias) with B given as PackB's result; the values are those of the plain GEMM entry points."""
        if kind not in self._PACK_KIND:
            raise NotSupportedException("GemmPackedB: kind must be 'f32', 'f16' or 'bf16'")
        op = "GemmPackedB"
        self._need(A, "A"); self._need(packedB, "packedB"); self._need(C, "C")
        self._positive(M=M, N=N, K=K)
        es = 4 if kind == "f32" else 2
        out32 = True if kind == "f32" else bool(outputIsFp32)
        self._capacity(A, M * K * es, "A", op); self._capacity(C, M * N * (4 if out32 else 2), "C", op)
        nbytes = int(self._lib.aidn_mi355_packed_b_bytes(self._PACK_KIND[kind], K, N, 1 if transB else 0))
        if nbytes <= 0:
            raise NotSupportedException("GemmPackedB: no packed layout for this kind / shape")
        self._capacity(packedB, nbytes, "packedB", op)
        if bias is not None:
            self._capacity(bias, N * 4, "bias", op)
        self._check(self._lib.aidn_mi355_gemm_packed_b(self._ctx, self._stream(), self._PACK_KIND[kind], A.Handle, packedB.Handle,
                                                       bias.Handle if bias is not None else None, C.Handle, 1 if out32 else 0,
                                                       M, N, K, 1 if transB else 0, int(activation), float(alpha)))
        self._done()

    # ------------------------------------------------------------------ rotary position embedding
    def RopeInterleaved(self, input: GpuBuffer, cos: GpuBuffer, sin: GpuBuffer, output: GpuBuffer,
                        rows: int, headDim: int, seqLen: int, startPosition: int, kind: str = "f32") -> None:
        """Rotates every adjacent pair (2i, 2i+1) of a [rows, headDim] view by the angle of position
        startPosition + row % seqLen; caches [maxSeq, headDim/2] fp32; output may alias input
        (IDirectGpuBackend.cs:1427-1446; HipBackend.cs:6177-6210).  kind "f16" / "bf16" is an addition."""
        fn = {"f32": self._lib.aidn_mi355_rope_interleaved_f32, "f16": self._lib.aidn_mi355_rope_interleaved_f16,
              "bf16": self._lib.aidn_mi355_rope_interleaved_bf16}.get(kind)
        if fn is None:
            raise NotSupportedException("RopeInterleaved: kind must be 'f32', 'f16' or 'bf16'")
        if rows <= 0 or headDim <= 0 or seqLen <= 0:
            raise ArgumentOutOfRangeException("RoPE dimensions must be positive.")
        if headDim & 1:
            raise ArgumentException("RoPE requires an even head dimension.")
        if startPosition < 0:
            raise ArgumentOutOfRangeException("startPosition")
        for b, n in ((input, "input"), (cos, "cos"), (sin, "sin"), (output, "output")):
            self._need(b, n)
        es = 4 if kind == "f32" else 2
        if input.SizeInBytes < rows * headDim * es or output.SizeInBytes < rows * headDim * es:
            raise ArgumentException("RoPE input/output buffers are smaller than rows * headDim.")
        need = (startPosition + min(seqLen, rows)) * (headDim // 2) * 4
        if cos.SizeInBytes < need or sin.SizeInBytes < need:
            raise ArgumentException("RoPE cos/sin caches are shorter than startPosition + seqLen positions.")
        self._check(fn(self._ctx, self._stream(), input.Handle, cos.Handle, sin.Handle, output.Handle, rows, headDim, seqLen,
                       startPosition))
        self._done()

    # ------------------------------------------------------------------ paged K/V cache attention
    def _paged(self, op, kind, q, kcache, vcache, blockTable, heads, kvHeads, headDim, blockSize, numQueries, keyLen, startPos,
               scale, splits, decode) -> GpuBuffer:
        # GpuKernelGuards.Attention / Gqa / PagedAttentionBuffers (GpuKernelGuards.cs:14-30, 87-108)
        if heads <= 0:
            raise ArgumentOutOfRangeException("%s: heads must be > 0 (got %d)." % (op, heads))
        if headDim <= 0 or headDim > 256:
            raise ArgumentOutOfRangeException("%s: headDim must be in [1, 256] (got %d)." % (op, headDim))
        if blockSize <= 0:
            raise ArgumentOutOfRangeException("%s: blockSize must be > 0 (got %d)." % (op, blockSize))
        if numQueries <= 0 or keyLen <= 0:
            raise ArgumentOutOfRangeException("%s: sequence/query count must be > 0." % op)
        if kvHeads <= 0 or kvHeads > heads or heads % kvHeads != 0:
            raise ArgumentOutOfRangeException("%s: kvHeads must satisfy 1 <= kvHeads <= heads and heads %% kvHeads == 0." % op)
        if startPos < 0:
            raise ArgumentOutOfRangeException("startPos")
        for b, n in ((q, "q"), (kcache, "kcache"), (vcache, "vcache"), (blockTable, "blockTable")):
            self._need(b, n)
        es = 4 if kind == "f32" else 2
        self._capacity(q, numQueries * heads * headDim * es, "q", op)
        blocks = (keyLen + blockSize - 1) // blockSize
        self._capacity(blockTable, blocks * 4, "blockTable", op)
        per_block = blockSize * kvHeads * headDim * es
        if kcache.SizeInBytes <= 0 or kcache.SizeInBytes != vcache.SizeInBytes:
            raise ArgumentException("%s: kcache/vcache must be equal-sized, non-empty K/V pools." % op)
        if kcache.SizeInBytes % per_block != 0:
            raise ArgumentException("%s: K/V pool size is not a whole number of blocks." % op)
        bt = blockTable.tensor.reshape(-1)[:blocks]
        if bt.dtype != torch.int32:
            raise ArgumentException("%s: blockTable must hold 32-bit block ids." % op)
        validate = self.ValidateBlockTables
        if validate is None:
            validate = not torch.cuda.is_current_stream_capturing()
        if validate and (int(bt.min()) < 0 or int(bt.max()) >= kcache.SizeInBytes // per_block):
            raise ArgumentException("%s: blockTable names a block outside the pool." % op)
        out = self.AllocateBuffer(numQueries * heads * headDim)
        if decode:
            fn = getattr(self._lib, "aidn_mi355_paged_attn_decode_" + kind)
            self._check(fn(self._ctx, self._stream(), q.Handle, kcache.Handle, vcache.Handle, blockTable.Handle, out.Handle,
                           heads, kvHeads, headDim, blockSize, keyLen, float(scale), int(splits)))
        else:
            fn = getattr(self._lib, "aidn_mi355_paged_attn_prefill_" + kind)
            self._check(fn(self._ctx, self._stream(), q.Handle, kcache.Handle, vcache.Handle, blockTable.Handle, out.Handle,
                           heads, kvHeads, headDim, blockSize, numQueries, startPos, float(scale)))
        self._done()
        return out

    def PagedAttentionDecode(self, q: GpuBuffer, kcache: GpuBuffer, vcache: GpuBuffer, blockTable: GpuBuffer,
                             heads: int, headDim: int, blockSize: int, seqLen: int, scale: float) -> GpuBuffer:
        """out[heads*headDim] = softmax(scale q K) V over a paged cache [numBlocks, blockSize, heads, headDim] gathered through
        blockTable (IDirectGpuBackend.cs:3614-3618; HipBackend.cs:831-852)."""
        return self._paged("PagedAttentionDecode", "f32", q, kcache, vcache, blockTable, heads, heads, headDim, blockSize, 1, seqLen, 0,
                           scale, 0, True)

    def PagedAttentionDecodeGqa(self, q: GpuBuffer, kcache: GpuBuffer, vcache: GpuBuffer, blockTable: GpuBuffer,
                                heads: int, kvHeads: int, headDim: int, blockSize: int, seqLen: int, scale: float) -> GpuBuffer:
        """Query head h reads KV head h / (heads / kvHeads) (IDirectGpuBackend.cs:3625-3627)."""
        return self._paged("PagedAttentionDecodeGqa", "f32", q, kcache, vcache, blockTable, heads, kvHeads, headDim, blockSize, 1, seqLen,
                           0, scale, 0, True)

    def PagedAttentionPrefill(self, q: GpuBuffer, kcache: GpuBuffer, vcache: GpuBuffer, blockTable: GpuBuffer,
                              heads: int, headDim: int, blockSize: int, numQueries: int, startPos: int, scale: float) -> GpuBuffer:
        """Causal multi-query form: query i attends to keys 0 .. startPos + i; out [numQueries, heads, headDim]
        (IDirectGpuBackend.cs:3620-3623; HipBackend.cs:854-876)."""
        return self._paged("PagedAttentionPrefill", "f32", q, kcache, vcache, blockTable, heads, heads, headDim, blockSize, numQueries,
                           startPos + numQueries, startPos, scale, 0, False)

    def PagedAttentionPrefillGqa(self, q: GpuBuffer, kcache: GpuBuffer, vcache: GpuBuffer, blockTable: GpuBuffer,
                                 heads: int, kvHeads: int, headDim: int, blockSize: int, numQueries: int, startPos: int,
                                 scale: float) -> GpuBuffer:
        return self._paged("PagedAttentionPrefillGqa", "f32", q, kcache, vcache, blockTable, heads, kvHeads, headDim, blockSize,
                           numQueries, startPos + numQueries, startPos, scale, 0, False)

    def PagedAttentionHalf(self, kind: str, q: GpuBuffer, kcache: GpuBuffer, vcache: GpuBuffer, blockTable: GpuBuffer,
                           heads: int, kvHeads: int, headDim: int, blockSize: int, numQueries: int, startPos: int, scale: float,
                           splits: int = 0) -> GpuBuffer:
        """fp16 / bf16 pools and queries, fp32 output; numQueries == 1 and startPos = seqLen - 1 is decode.  No member of this
        name exists in the reference interface (its paged attention is fp32 only)."""
        if kind not in ("f16", "bf16"):
            raise NotSupportedException("PagedAttentionHalf: kind must be 'f16' or 'bf16'")
        decode = numQueries == 1
        return self._paged("PagedAttentionHalf", kind, q, kcache, vcache, blockTable, heads, kvHeads, headDim, blockSize, numQueries,
                           startPos + numQueries, 0 if decode else startPos, scale, splits, decode)

    # ------------------------------------------------------------------ multi-head attention forward
    def MultiHeadAttentionForward(self, kind: str, input: GpuBuffer, qWeight: GpuBuffer, kWeight: GpuBuffer, vWeight: GpuBuffer,
                                  outWeight: GpuBuffer, mask: Optional[GpuBuffer], output: GpuBuffer,
                                  batch: int, seqLen: int, dModel: int, numHeads: int) -> None:
        """output[B,S,dModel] = MHA(input) with [dModel,dModel] weights and no biases, as three launches over a packed
        QKV activation (CpuEngine.MultiHeadAttention.cs:155-285 restated for the device; the reference has no GPU route).
        kind "f32" / "f16" / "bf16"; mask: fp32 keep-mask of seqLen*seqLen (shared) or batch*numHeads*seqLen*seqLen elements."""
        fn = {"f32": self._lib.aidn_mi355_mha_fwd_f32, "f16": self._lib.aidn_mi355_mha_fwd_f16,
              "bf16": self._lib.aidn_mi355_mha_fwd_bf16}.get(kind)
        if fn is None:
            raise NotSupportedException("MultiHeadAttentionForward: kind must be 'f32', 'f16' or 'bf16'")
        op = "MultiHeadAttentionForward"
        for b, n in ((input, "input"), (qWeight, "qWeight"), (kWeight, "kWeight"), (vWeight, "vWeight"), (outWeight, "outWeight"),
                     (output, "output")):
            self._need(b, n)
        self._positive(batch=batch, seqLen=seqLen, dModel=dModel, numHeads=numHeads)
        if dModel % numHeads != 0:
            raise ArgumentException("dModel (%d) must be divisible by numHeads (%d)." % (dModel, numHeads))
        if dModel // numHeads > 256:
            raise ArgumentException("head dimension %d exceeds 256" % (dModel // numHeads))          # GpuKernelGuards.cs:12
        es = 4 if kind == "f32" else 2
        self._capacity(input, batch * seqLen * dModel * es, "input", op)
        self._capacity(output, batch * seqLen * dModel * es, "output", op)
        for b, n in ((qWeight, "qWeight"), (kWeight, "kWeight"), (vWeight, "vWeight"), (outWeight, "outWeight")):
            self._capacity(b, dModel * dModel * es, n, op)
        mode = 0
        if mask is not None:
            plane = seqLen * seqLen
            if mask.SizeInBytes == plane * 4:
                mode = 1
            elif mask.SizeInBytes == batch * numHeads * plane * 4:
                mode = 2
            else:
                raise ArgumentException("mask must hold seqLen*seqLen or batch*numHeads*seqLen*seqLen floats")
        self._check(fn(self._ctx, self._stream(), input.Handle, qWeight.Handle, kWeight.Handle, vWeight.Handle, outWeight.Handle,
                       mask.Handle if mask is not None else None, mode, output.Handle, batch, seqLen, dModel, numHeads))
        self._done()

    def PackQkvWeights(self, kind: str, qWeight: GpuBuffer, kWeight: GpuBuffer, vWeight: GpuBuffer, dModel: int) -> GpuBuffer:
        """[Wq|Wk|Wv] side by side in one new [dModel, 3 dModel] buffer: the constant operand of the fused QKV projection,
        packed once instead of on every forward call."""
        if kind not in ("f32", "f16", "bf16"):
            raise NotSupportedException("PackQkvWeights: kind must be 'f32', 'f16' or 'bf16'")
        self._positive(dModel=dModel)
        es = 4 if kind == "f32" else 2
        for b, n in ((qWeight, "qWeight"), (kWeight, "kWeight"), (vWeight, "vWeight")):
            self._capacity(self._need(b, n), dModel * dModel * es, n, "PackQkvWeights")
        packed = self.AllocateByteBuffer(3 * dModel * dModel * es)
        self._check(self._lib.aidn_mi355_mha_pack_qkv(self._ctx, self._stream(), qWeight.Handle, kWeight.Handle, vWeight.Handle,
                                                       packed.Handle, dModel, es))
        self._done()
        return packed

    def MultiHeadAttentionForwardPacked(self, kind: str, input: GpuBuffer, qkvWeight: GpuBuffer, outWeight: GpuBuffer,
                                        mask: Optional[GpuBuffer], output: GpuBuffer,
                                        batch: int, seqLen: int, dModel: int, numHeads: int) -> None:
        """MultiHeadAttentionForward on a weight packed by PackQkvWeights (no per-call weight gather)."""
        fn = {"f32": self._lib.aidn_mi355_mha_fwd_packed_f32, "f16": self._lib.aidn_mi355_mha_fwd_packed_f16,
              "bf16": self._lib.aidn_mi355_mha_fwd_packed_bf16}.get(kind)
        if fn is None:
            raise NotSupportedException("MultiHeadAttentionForwardPacked: kind must be 'f32', 'f16' or 'bf16'")
        op = "MultiHeadAttentionForwardPacked"
        for b, n in ((input, "input"), (qkvWeight, "qkvWeight"), (outWeight, "outWeight"), (output, "output")):
            self._need(b, n)
        self._positive(batch=batch, seqLen=seqLen, dModel=dModel, numHeads=numHeads)
        if dModel % numHeads != 0:
            raise ArgumentException("dModel (%d) must be divisible by numHeads (%d)." % (dModel, numHeads))
        if dModel // numHeads > 256:
            raise ArgumentException("head dimension %d exceeds 256" % (dModel // numHeads))
        es = 4 if kind == "f32" else 2
        self._capacity(input, batch * seqLen * dModel * es, "input", op)
        self._capacity(output, batch * seqLen * dModel * es, "output", op)
        self._capacity(qkvWeight, 3 * dModel * dModel * es, "qkvWeight", op)
        self._capacity(outWeight, dModel * dModel * es, "outWeight", op)
        mode = 0
        if mask is not None:
            plane = seqLen * seqLen
            if mask.SizeInBytes == plane * 4:
                mode = 1
            elif mask.SizeInBytes == batch * numHeads * plane * 4:
                mode = 2
            else:
                raise ArgumentException("mask must hold seqLen*seqLen or batch*numHeads*seqLen*seqLen floats")
        self._check(fn(self._ctx, self._stream(), input.Handle, qkvWeight.Handle, outWeight.Handle,
                       mask.Handle if mask is not None else None, mode, output.Handle, batch, seqLen, dModel, numHeads))
        self._done()

    # ------------------------------------------------------------------ GEMM (16-bit)
    SupportsHgemm = True
    SupportsBf16Gemm = True   # no member of this name exists in the reference interface

    def _gemm16(self, fn, a, b, c, m, n, k, out_bytes, op):
        self._need(a, "a"); self._need(b, "b"); self._need(c, "c")
        if m <= 0: raise ArgumentOutOfRangeException("m: Dimensions must be positive.")
        if n <= 0: raise ArgumentOutOfRangeException("n: Dimensions must be positive.")
        if k <= 0: raise ArgumentOutOfRangeException("k: Dimensions must be positive.")
        self._capacity(a, m * k * 2, "a", op); self._capacity(b, k * n * 2, "b", op); self._capacity(c, m * n * out_bytes, "c", op)
        self._check(fn(self._ctx, self._stream(), a.Handle, b.Handle, c.Handle, m, n, k))
        self._done()

    def Hgemm(self, aFp16: GpuBuffer, bFp16: GpuBuffer, cFp16: GpuBuffer, m: int, n: int, k: int) -> None:
        """fp16 in, fp16 out, fp32 accumulation (IGpuHalfPrecisionBackend.cs:27-37)."""
        self._gemm16(self._lib.aidn_mi355_hgemm_f16out, aFp16, bFp16, cFp16, m, n, k, 2, "Hgemm")

    def GemmFp16In32fOut(self, aFp16: GpuBuffer, bFp16: GpuBuffer, cFp32: GpuBuffer, m: int, n: int, k: int) -> None:
        """fp16 in, fp32 out (IGpuHalfPrecisionBackend.cs:39-48)."""
        self._gemm16(self._lib.aidn_mi355_hgemm_f32out, aFp16, bFp16, cFp32, m, n, k, 4, "GemmFp16In32fOut")

    def Bf16Gemm(self, aBf16: GpuBuffer, bBf16: GpuBuffer, cBf16: GpuBuffer, m: int, n: int, k: int) -> None:
        """bf16 in, bf16 out, fp32 accumulation: the CPU kernel BFloat16Kernels.Matmul on the GPU."""
        self._gemm16(self._lib.aidn_mi355_bf16gemm_bf16out, aBf16, bBf16, cBf16, m, n, k, 2, "Bf16Gemm")

    def GemmBf16In32fOut(self, aBf16: GpuBuffer, bBf16: GpuBuffer, cFp32: GpuBuffer, m: int, n: int, k: int) -> None:
        self._gemm16(self._lib.aidn_mi355_bf16gemm_f32out, aBf16, bBf16, cFp32, m, n, k, 4, "GemmBf16In32fOut")

    def GemmRope(self, kind: str, a: GpuBuffer, b: GpuBuffer, c: GpuBuffer, m: int, n: int, k: int, cos: GpuBuffer, sin: GpuBuffer,
                 headDim: int, ropeCols: int, seqLen: int, startPosition: int) -> None:
        """C[m,n] = A * B in fp16 / bf16 (fp32 accumulation), then RopeInterleaved over the first ropeCols columns of C (heads of
        headDim side by side; row r at position startPosition + r % seqLen) in the same call: a projection of a decode step
        (SimdGemm.NParallelSmallM.cs:95-109) and its rotation (IDirectGpuBackend.cs:1427-1446) with one launch fewer.  Same values
        as Hgemm / Bf16Gemm followed by RopeInterleaved.  No single member of the reference does both."""
        fn = {"f16": self._lib.aidn_mi355_hgemm_rope, "bf16": self._lib.aidn_mi355_bf16gemm_rope}.get(kind)
        if fn is None:
            raise NotSupportedException("GemmRope: kind must be 'f16' or 'bf16'")
        if m <= 0 or n <= 0 or k <= 0:
            raise ArgumentOutOfRangeException("GemmRope: M, N, K must all be > 0 (got M=%d, N=%d, K=%d)." % (m, n, k))
        if headDim <= 0 or seqLen <= 0:
            raise ArgumentOutOfRangeException("RoPE dimensions must be positive.")
        if headDim & 1:
            raise ArgumentException("RoPE requires an even head dimension.")
        if startPosition < 0:
            raise ArgumentOutOfRangeException("startPosition")
        if ropeCols < 0 or ropeCols > n or ropeCols % headDim != 0 or n & 1:
            raise ArgumentException("GemmRope: ropeCols must be a multiple of headDim within n, and n even.")
        for buf, nm in ((a, "a"), (b, "b"), (c, "c"), (cos, "cos"), (sin, "sin")):
            self._need(buf, nm)
        self._capacity(a, m * k * 2, "a", "GemmRope"); self._capacity(b, k * n * 2, "b", "GemmRope"); self._capacity(c, m * n * 2, "c", "GemmRope")
        need = (startPosition + min(seqLen, m)) * (headDim // 2) * 4
        if cos.SizeInBytes < need or sin.SizeInBytes < need:
            raise ArgumentException("RoPE cos/sin caches are shorter than startPosition + seqLen positions.")
        self._check(fn(self._ctx, self._stream(), a.Handle, b.Handle, c.Handle, m, n, k, cos.Handle, sin.Handle, headDim, ropeCols, seqLen,
                       startPosition))
        self._done()

    # ------------------------------------------------------------------ conversions
    def _convert(self, fn, inp, out, size, in_bytes, out_bytes, op):
        self._need(inp, "input"); self._need(out, "output")
        if size <= 0:
            raise ArgumentOutOfRangeException("size must be positive")
        self._capacity(inp, size * in_bytes, "input", op); self._capacity(out, size * out_bytes, "output", op)
        self._check(fn(self._ctx, self._stream(), inp.Handle, out.Handle, size))
        self._done()

    def ConvertToFp16(self, input: GpuBuffer, output: GpuBuffer, size: int) -> None:
        """fp32 -> fp16, RNE (IDirectGpuBackend.cs:1876-1890)."""
        self._convert(self._lib.aidn_mi355_convert_f32_to_f16, input, output, size, 4, 2, "ConvertToFp16")

    def ConvertToFp32(self, input: GpuBuffer, output: GpuBuffer, size: int) -> None:
        """fp16 -> fp32 (IDirectGpuBackend.cs:1892-1911)."""
        self._convert(self._lib.aidn_mi355_convert_f16_to_f32, input, output, size, 2, 4, "ConvertToFp32")

    def ConvertToBf16(self, input: GpuBuffer, output: GpuBuffer, size: int) -> None:
        self._convert(self._lib.aidn_mi355_convert_f32_to_bf16, input, output, size, 4, 2, "ConvertToBf16")

    def ConvertBf16ToFp32(self, input: GpuBuffer, output: GpuBuffer, size: int) -> None:
        self._convert(self._lib.aidn_mi355_convert_bf16_to_f32, input, output, size, 2, 4, "ConvertBf16ToFp32")

    # ------------------------------------------------------------------ attention
    def _attn(self, kind: str, q, k, v, o, lse, bias, mask, weights, desc: AttnDesc) -> None:
        fn = {"f32": self._lib.aidn_mi355_attn_fwd_f32, "f16": self._lib.aidn_mi355_attn_fwd_f16,
              "bf16": self._lib.aidn_mi355_attn_fwd_bf16}[kind]
        h = lambda b: b.Handle if b is not None else None
        self._check(fn(self._ctx, self._stream(), ctypes.byref(desc), q.Handle, k.Handle, v.Handle, o.Handle,
                       h(lse), h(bias), h(mask), h(weights)))
        self._done()

    def ScaledDotProductAttention(self, query: GpuBuffer, key: GpuBuffer, value: GpuBuffer, output: GpuBuffer,
                                  attentionWeights: Optional[GpuBuffer], mask: Optional[GpuBuffer],
                                  batch: int, numHeads: int, seqQ: int, seqK: int, headDim: int, scale: float,
                                  isCausal: bool, softcap: float = 0.0, numKVHeads: int = 0) -> None:
        """IDirectGpuBackend.cs:1395-1424 / HipBackend.cs:6118-6175: fp32, optional weights output,
        float mask (0 = masked; shared [seqQ*seqK] plane or full), bottom-right causal alignment,
        grouped-query heads."""
        if batch <= 0 or numHeads <= 0 or seqQ <= 0 or seqK <= 0 or headDim <= 0:
            raise ArgumentOutOfRangeException("batch: Attention dimensions must be positive.")
        kvHeads = numKVHeads if numKVHeads > 0 else numHeads
        if numHeads % kvHeads != 0:
            raise ArgumentException("numHeads must be an integer multiple of numKVHeads.")
        if headDim > MAX_HEAD_DIM:
            raise ArgumentOutOfRangeException("headDim must be in [1, %d]" % MAX_HEAD_DIM)
        qsz = batch * numHeads * seqQ * headDim
        kvsz = batch * kvHeads * seqK * headDim
        wsz = batch * numHeads * seqQ * seqK
        for b, nm in ((query, "query"), (key, "key"), (value, "value"), (output, "output")):
            self._need(b, nm)
        if query.Size < qsz or key.Size < kvsz or value.Size < kvsz or output.Size < qsz:
            raise ArgumentException("Attention tensor buffers are smaller than the requested dimensions.")
        if attentionWeights is not None and attentionWeights.Size < wsz:
            raise ArgumentException("The attention-weights buffer is too small.")
        if mask is not None and mask.Size < seqQ * seqK:
            raise ArgumentException("The attention mask must contain at least seqQ * seqK elements.")
        d = AttnDesc(B=batch, H=numHeads, Hkv=kvHeads, Sq=seqQ, Sk=seqK, D=headDim, scale=scale,
                     causal=1 if isCausal else 0, causal_query_offset=seqK - seqQ, softcap=softcap,
                     mask_mode=0 if mask is None else (2 if mask.Size >= wsz else 1))
        self._attn("f32", query, key, value, output, None, None, mask, attentionWeights, d)

    def FlashAttentionV2(self, query: GpuBuffer, key: GpuBuffer, value: GpuBuffer, output: GpuBuffer,
                         softmaxStats: GpuBuffer, batch: int, numHeads: int, seqQ: int, seqK: int, headDim: int,
                         scale: float, isCausal: bool, attentionBias: Optional[GpuBuffer] = None,
                         biasBatchStride: int = 0) -> None:
        """IDirectGpuBackend.cs:1451-1471 / HipBackend.cs:6261-6302: fp32, LSE output, additive bias,
        top-left causal alignment (key j masked iff j > i)."""
        if batch <= 0 or numHeads <= 0 or seqQ <= 0 or seqK <= 0 or headDim <= 0:
            raise ArgumentOutOfRangeException("batch: Attention dimensions must be positive.")
        if headDim > MAX_HEAD_DIM:
            raise ArgumentOutOfRangeException("headDim must be in [1, %d]" % MAX_HEAD_DIM)
        for b, nm in ((query, "query"), (key, "key"), (value, "value"), (output, "output"), (softmaxStats, "softmaxStats")):
            self._need(b, nm)
        qsz = batch * numHeads * seqQ * headDim
        kvsz = batch * numHeads * seqK * headDim
        if query.Size < qsz or key.Size < kvsz or value.Size < kvsz or output.Size < qsz:
            raise ArgumentException("Attention tensor buffers are smaller than the requested dimensions.")
        if softmaxStats.Size < batch * numHeads * seqQ:
            raise ArgumentException("The softmax-statistics buffer is too small.")
        d = AttnDesc(B=batch, H=numHeads, Hkv=numHeads, Sq=seqQ, Sk=seqK, D=headDim, scale=scale,
                     causal=1 if isCausal else 0, causal_query_offset=0, bias_batch_stride=biasBatchStride)
        self._attn("f32", query, key, value, output, softmaxStats, attentionBias, None, None, d)

    def FlashAttention(self, query: GpuBuffer, key: GpuBuffer, value: GpuBuffer, output: GpuBuffer,
                       mask: Optional[GpuBuffer], batch: int, numHeads: int, seqLen: int, headDim: int,
                       scale: float, isCausal: bool) -> None:
        """IDirectGpuBackend.cs:1448-1449; the reference forwards to FlashAttentionV2 with a scratch
        statistics buffer and ignores `mask` (HipBackend.cs:6250-6259)."""
        stats = self.AllocateBuffer(batch * numHeads * seqLen)
        self.FlashAttentionV2(query, key, value, output, stats, batch, numHeads, seqLen, seqLen, headDim, scale, isCausal)

    def FlashAttentionHalf(self, kind: str, query: GpuBuffer, key: GpuBuffer, value: GpuBuffer, output: GpuBuffer,
                           softmaxStats: Optional[GpuBuffer], batch: int, numHeads: int, seqQ: int, seqK: int,
                           headDim: int, scale: float, isCausal: bool, causalQueryOffset: int = 0,
                           numKVHeads: int = 0, outputIs16Bit: bool = False) -> None:
        """fp16 / bf16 Q, K, V with fp32 softmax and accumulation; fp32 O + fp32 LSE by default -- the
        contract of the reference's only reduced-precision attention route
        (src/AiDotNet.Tensors/Engines/DirectGpuTensorEngine.cs:11143-11167).  No member of this
        name exists in the reference interface."""
        if kind not in ("f16", "bf16"):
            raise ArgumentException("kind must be 'f16' or 'bf16'")
        if batch <= 0 or numHeads <= 0 or seqQ <= 0 or seqK <= 0 or headDim <= 0:
            raise ArgumentOutOfRangeException("batch: Attention dimensions must be positive.")
        kvHeads = numKVHeads if numKVHeads > 0 else numHeads
        if numHeads % kvHeads != 0:
            raise ArgumentException("numHeads must be an integer multiple of numKVHeads.")
        if headDim > MAX_HEAD_DIM:
            raise ArgumentOutOfRangeException("headDim must be in [1, %d]" % MAX_HEAD_DIM)
        qsz = batch * numHeads * seqQ * headDim
        kvsz = batch * kvHeads * seqK * headDim
        self._capacity(self._need(query, "query"), qsz * 2, "query", "FlashAttentionHalf")
        self._capacity(self._need(key, "key"), kvsz * 2, "key", "FlashAttentionHalf")
        self._capacity(self._need(value, "value"), kvsz * 2, "value", "FlashAttentionHalf")
        self._capacity(self._need(output, "output"), qsz * (2 if outputIs16Bit else 4), "output", "FlashAttentionHalf")
        if softmaxStats is not None:
            self._capacity(softmaxStats, batch * numHeads * seqQ * 4, "softmaxStats", "FlashAttentionHalf")
        d = AttnDesc(B=batch, H=numHeads, Hkv=kvHeads, Sq=seqQ, Sk=seqK, D=headDim, scale=scale,
                     causal=1 if isCausal else 0, causal_query_offset=causalQueryOffset,
                     out_is_16bit=1 if outputIs16Bit else 0)
        self._attn(kind, query, key, value, output, softmaxStats, None, None, None, d)

    # ------------------------------------------------------------------ decode
    def _decode(self, kind, q, k, v, o, lse, desc, splits, no_alloc=False):
        if no_alloc:
            if kind != "bf16":
                raise NotSupportedException("the allocation-free decode entry point exists for bf16 only")
            fn = self._lib.aidn_mi355_attn_decode_bf16_noalloc
        else:
            fn = {"f32": self._lib.aidn_mi355_attn_decode_f32, "f16": self._lib.aidn_mi355_attn_decode_f16,
                  "bf16": self._lib.aidn_mi355_attn_decode_bf16}[kind]
        self._check(fn(self._ctx, self._stream(), ctypes.byref(desc), q.Handle, k.Handle, v.Handle, o.Handle,
                       lse.Handle if lse is not None else None, splits))
        self._done()

    def FlashDecode(self, q: GpuBuffer, k: GpuBuffer, v: GpuBuffer, heads: int, kvHeads: int, headDim: int,
                    seqLen: int, scale: float, splits: int = 0) -> GpuBuffer:
        """Single-sequence decode over K/V laid out [seqLen, kvHeads, headDim], fp32; returns a new
        [heads * headDim] buffer (HipBackend.cs:919-965; guards GpuKernelGuards.cs:41-52)."""
        if heads <= 0:
            raise ArgumentOutOfRangeException("FlashDecode: heads must be > 0 (got %d)." % heads)
        if headDim <= 0 or headDim > MAX_HEAD_DIM:
            raise ArgumentOutOfRangeException("FlashDecode: headDim must be in [1, %d] (got %d)." % (MAX_HEAD_DIM, headDim))
        if seqLen <= 0:
            raise ArgumentOutOfRangeException("FlashDecode: seqLen must be > 0 (got %d)." % seqLen)
        if kvHeads <= 0 or kvHeads > heads or heads % kvHeads != 0:
            raise ArgumentOutOfRangeException("FlashDecode: kvHeads must satisfy 1 <= kvHeads <= heads and heads %% kvHeads == 0 (heads=%d, kvHeads=%d)." % (heads, kvHeads))
        self._need(q, "q"); self._need(k, "k"); self._need(v, "v")
        self._capacity(q, heads * headDim * 4, "q", "FlashDecode")
        self._capacity(k, seqLen * kvHeads * headDim * 4, "k", "FlashDecode")
        self._capacity(v, seqLen * kvHeads * headDim * 4, "v", "FlashDecode")
        out = self.AllocateBuffer(heads * headDim)
        d = AttnDesc(B=1, H=heads, Hkv=kvHeads, Sq=1, Sk=seqLen, D=headDim, scale=scale)
        # [seqLen, kvHeads, d]: batch stride unused (B = 1), head stride d, row stride kvHeads * d
        d.q_strides[:] = [heads * headDim, headDim, headDim]
        d.k_strides[:] = [seqLen * kvHeads * headDim, headDim, kvHeads * headDim]
        d.v_strides[:] = [seqLen * kvHeads * headDim, headDim, kvHeads * headDim]
        d.o_strides[:] = [heads * headDim, headDim, headDim]
        self._decode("f32", q, k, v, out, None, d, splits)
        return out

    def DecodeAttention(self, kind: str, q: GpuBuffer, k: GpuBuffer, v: GpuBuffer, output: GpuBuffer,
                        batch: int, numHeads: int, seqK: int, headDim: int, scale: float,
                        numKVHeads: int = 0, splits: int = 0, outputIs16Bit: bool = False,
                        softmaxStats: Optional[GpuBuffer] = None, kvLayout: str = "bhsd", noAlloc: bool = False) -> None:
        """Batched decode: q [B,H,1,d]; the KV cache [B,Hkv,S,d] ("bhsd") or the reference's dense
        KVCache layout [B,S,Hkv,d] ("bshd", src/AiDotNet.Tensors/Engines/Autodiff/KVCache.cs:5-8).
        What ScaledDotProductAttention with seqQ = 1 computes (bottom-right causal = all keys);
        no member of this name exists in the reference interface."""
        if kind not in ("f32", "f16", "bf16"):
            raise ArgumentException("kind must be 'f32', 'f16' or 'bf16'")
        if batch <= 0 or numHeads <= 0 or seqK <= 0 or headDim <= 0:
            raise ArgumentOutOfRangeException("batch: Attention dimensions must be positive.")
        kvHeads = numKVHeads if numKVHeads > 0 else numHeads
        if kvHeads > numHeads or numHeads % kvHeads != 0:
            raise ArgumentOutOfRangeException("kvHeads must divide numHeads")
        if headDim > MAX_HEAD_DIM:
            raise ArgumentOutOfRangeException("headDim must be in [1, %d]" % MAX_HEAD_DIM)
        eb = 4 if kind == "f32" else 2
        self._capacity(self._need(q, "q"), batch * numHeads * headDim * eb, "q", "DecodeAttention")
        self._capacity(self._need(k, "k"), batch * kvHeads * seqK * headDim * eb, "k", "DecodeAttention")
        self._capacity(self._need(v, "v"), batch * kvHeads * seqK * headDim * eb, "v", "DecodeAttention")
        self._capacity(self._need(output, "output"), batch * numHeads * headDim * (2 if outputIs16Bit else 4), "output", "DecodeAttention")
        d = AttnDesc(B=batch, H=numHeads, Hkv=kvHeads, Sq=1, Sk=seqK, D=headDim, scale=scale,
                     out_is_16bit=1 if outputIs16Bit else 0)
        if kvLayout == "bshd":
            d.q_strides[:] = [numHeads * headDim, headDim, headDim]
            d.o_strides[:] = [numHeads * headDim, headDim, headDim]
            d.k_strides[:] = [seqK * kvHeads * headDim, headDim, kvHeads * headDim]
            d.v_strides[:] = [seqK * kvHeads * headDim, headDim, kvHeads * headDim]
        elif kvLayout != "bhsd":
            raise ArgumentException("kvLayout must be 'bhsd' or 'bshd'")
        # noAlloc: the bf16 entry point whose split partials live in the library's static device array (never allocates)
        self._decode(kind, q, k, v, output, softmaxStats, d, splits, no_alloc=noAlloc)
