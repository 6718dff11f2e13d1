"""GPU parity of fused attention (prefill) through the C ABI against the CPU oracle.

Bars: |a - e| <= 1e-4 * (1 + |e|) for fp32, 2e-2 for fp16 / bf16 inputs, against the fp64 truth of the
same (already rounded) inputs; the fp32 kernel is also held to the CPU restatement itself.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import TORCH16, dev, from_bits16, mixed_err, round_to

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-4
HALF_TOL = 2e-2


@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    b = Mi355Backend()
    yield b
    b.Dispose()


@pytest.fixture(scope="module")
def eng(be):
    from aidotnet.tensors_amd import Mi355Engine
    return Mi355Engine(be)


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


# B, H, Hkv, Sq, Sk, D, causal, offset
CASES = [
    (1, 2, 2, 4, 4, 8, True, 0),            # OpParityRegistry.cs:1896-1899
    (2, 3, 3, 33, 65, 20, False, 0),        # FusedAttentionFp32PrecisionTests.cs:30-58 (Sq != Sk, d = 20)
    (1, 4, 4, 70, 70, 64, True, 0),         # non block-aligned S
    (1, 2, 2, 100, 100, 32, True, 0),
    (2, 4, 2, 17, 40, 32, True, 23),        # GQA + bottom-right causal
    (1, 2, 1, 1, 77, 48, True, 76),         # decode shape through the prefill kernel
    (1, 1, 1, 129, 257, 128, False, 0),
    (2, 2, 2, 256, 256, 128, True, 0),
    (1, 2, 2, 130, 200, 72, True, 70),      # DiT head dim 72
    (1, 1, 1, 64, 64, 256, True, 0),
    (1, 2, 2, 300, 300, 256, True, 0),      # head dim 256 over several key tiles: Q fragments are re-fetched per tile
    (1, 2, 1, 130, 200, 200, False, 0),     # head dim between 128 and 256, GQA
    (1, 3, 3, 200, 50, 16, True, 0),        # Sq > Sk top-left: late rows see every key
    (1, 2, 2, 5, 9, 7, False, 0),           # odd head dim: element-wise loads
    (8, 49, 49, 200, 200, 32, True, 0),     # 784 workgroups, whole heads per XCD: causal tiles handed out by head group
    (7, 37, 37, 300, 300, 16, True, 0),     # 777 workgroups, heads straddle the XCDs: head groups over the whole grid
]


@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,D,causal,offset", CASES)
def test_fp32_attention_matches_oracle(eng, B, H, Hkv, Sq, Sk, D, causal, offset):
    rng = np.random.default_rng(B + 3 * H + 7 * Sq + 11 * Sk + D)
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    scale = 1.0 / math.sqrt(D)
    o_cpu, lse_cpu, _ = oracle.attention_f32(q, k, v, scale, causal, offset)
    o64, lse64 = oracle.attention_f64(q, k, v, scale, causal, offset)
    o, lse = eng.FlashAttention(dev(q), dev(k), dev(v), scale, causal, queryOffset=offset)
    o = o.cpu().numpy(); lse = lse.cpu().numpy()
    assert mixed_err(o, o64) <= FP32_TOL and mixed_err(lse, lse64) <= FP32_TOL
    assert mixed_err(o, o_cpu) <= FP32_TOL and mixed_err(lse, lse_cpu) <= FP32_TOL
    # FusedAttentionFp32PrecisionTests.cs:30-58: fp32 vs fp64 max-abs < 2e-3
    assert np.max(np.abs(o - o64)) < 2e-3


def test_fp32_invariants(eng):
    rng = np.random.default_rng(2)
    B, H, S, D = 1, 2, 9, 8
    q, k, v = _rand(rng, B, H, S, D), _rand(rng, B, H, S, D), _rand(rng, B, H, S, D)
    o, _ = eng.FlashAttention(dev(q), dev(k), dev(v), 0.3, True)
    assert np.allclose(o.cpu().numpy()[:, :, 0], v[:, :, 0], atol=1e-6)               # causal row 0 = V[0]
    o0, lse0 = eng.FlashAttention(dev(np.zeros_like(q)), dev(k), dev(v), 0.3, True)
    means = np.cumsum(v.astype(np.float64), axis=2) / np.arange(1, S + 1)[None, None, :, None]
    assert np.allclose(o0.cpu().numpy(), means, atol=1e-6)                             # Q = 0 -> running mean
    assert np.allclose(lse0.cpu().numpy(), np.log(np.arange(1, S + 1))[None, None], atol=1e-6)
    perm = rng.permutation(S)
    o1, l1 = eng.FlashAttention(dev(q), dev(k), dev(v), 0.3, False)
    o2, l2 = eng.FlashAttention(dev(q), dev(k[:, :, perm]), dev(v[:, :, perm]), 0.3, False)
    assert np.allclose(o1.cpu().numpy(), o2.cpu().numpy(), atol=2e-6)                  # key permutation invariance


def test_decode_row_equals_last_row_of_causal_prefill(eng):
    # FusedAttentionAuditTests.cs:47-79
    rng = np.random.default_rng(6)
    B, H, S, D = 1, 4, 150, 64
    q, k, v = _rand(rng, B, H, S, D), _rand(rng, B, H, S, D), _rand(rng, B, H, S, D)
    full, lse_full = eng.FlashAttention(dev(q), dev(k), dev(v), 0.125, True)
    for t in (0, 5, 149):
        o, lse = eng.FlashAttention(dev(q[:, :, t:t + 1]), dev(k[:, :, :t + 1]), dev(v[:, :, :t + 1]), 0.125, True, queryOffset=t)
        assert np.allclose(o.cpu().numpy()[:, :, 0], full.cpu().numpy()[:, :, t], atol=2e-6)
        assert np.allclose(lse.cpu().numpy()[:, :, 0], lse_full.cpu().numpy()[:, :, t], atol=2e-6)
    from aidotnet.tensors_amd import ArgumentException
    with pytest.raises(ArgumentException):                                             # offset + Sq > Sk (:81-92)
        eng.FlashAttention(dev(q[:, :, :4]), dev(k[:, :, :5]), dev(v[:, :, :5]), 0.125, True, queryOffset=3)


@pytest.mark.parametrize("rank", [3, 4])
def test_bias_after_scale(eng, rank):
    # FlashAttentionBiasTests.cs:89-115 (identity Q/K/V) + a random case; 3-D bias broadcasts over batch
    S = 4
    eye = np.eye(S, dtype=np.float32)[None, None]
    bias = np.zeros((1, 1, S, S), np.float32); bias[0, 0, :, 2] = 5.0
    o, _ = eng.FlashAttention(dev(eye), dev(eye), dev(eye), 0.5, False, attentionBias=dev(bias if rank == 4 else bias[0]))
    logits = 0.5 * np.eye(S) + bias[0, 0]
    p = np.exp(logits) / np.exp(logits).sum(-1, keepdims=True)
    assert np.allclose(o.cpu().numpy()[0, 0], p, atol=1e-6)
    rng = np.random.default_rng(9)
    B, H, Sq, Sk, D = 2, 3, 37, 53, 32
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, H, Sk, D), _rand(rng, B, H, Sk, D)
    bb = _rand(rng, B, H, Sq, Sk) if rank == 4 else _rand(rng, H, Sq, Sk)
    want, lse_w, _ = oracle.attention_f32(q, k, v, 0.2, True, 0, bias=bb)
    got, lse = eng.FlashAttention(dev(q), dev(k), dev(v), 0.2, True, attentionBias=dev(bb))
    assert mixed_err(got.cpu().numpy(), want) <= FP32_TOL and mixed_err(lse.cpu().numpy(), lse_w) <= FP32_TOL


def test_sdpa_mask_softcap_weights_gqa(eng):
    rng = np.random.default_rng(5)
    B, H, Hkv, Sq, Sk, D = 2, 4, 2, 21, 35, 16
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    # shared [1,1,Sq,Sk] mask with an all-masked row (SdpaMaskBroadcastTests.cs:73-125; CpuEngine.cs:27817-27822)
    keep = rng.random((1, 1, Sq, Sk)) > 0.4
    keep[0, 0, 3, :] = False
    want, _, w_want = oracle.attention_f32(q, k, v, 0.3, keep=keep, want_weights=True)
    o, w = eng.ScaledDotProductAttention(dev(q), dev(k), dev(v), torch.from_numpy(keep).cuda(), 0.3)
    o = o.cpu().numpy(); w = w.cpu().numpy()
    assert mixed_err(o, want) <= FP32_TOL and np.max(np.abs(w - w_want)) <= 1e-5
    assert np.all(o[:, :, 3] == 0) and np.all(w[:, :, 3] == 0)
    assert np.allclose(np.delete(w, 3, axis=2).sum(-1), 1.0, atol=1e-5)                # rows of P sum to 1
    # full [B,H,Sq,Sk] mask equals the materialised broadcast
    full = np.broadcast_to(rng.random((B, 1, 1, Sk)) > 0.3, (B, H, Sq, Sk)).copy()
    full[..., 0] = True
    want2, _, _ = oracle.attention_f32(q, k, v, 0.3, keep=full)
    o2, _ = eng.ScaledDotProductAttention(dev(q), dev(k), dev(v), torch.from_numpy(full).cuda(), 0.3, returnWeights=False)
    assert mixed_err(o2.cpu().numpy(), want2) <= FP32_TOL
    # soft-cap closed form (BatchMatMulAndAttentionTests.cs:288-317)
    want3, _, w3 = oracle.attention_f32(3 * q, 3 * k, v, 1.0, softcap=2.0, want_weights=True)
    o3, w3g = eng.ScaledDotProductAttention(dev(3 * q), dev(3 * k), dev(v), None, 1.0, softcap=2.0)
    assert mixed_err(o3.cpu().numpy(), want3) <= FP32_TOL and np.max(np.abs(w3g.cpu().numpy() - w3)) <= 1e-5
    nocap, _ = eng.ScaledDotProductAttention(dev(3 * q), dev(3 * k), dev(v), None, 1.0, returnWeights=False)
    assert np.max(np.abs(nocap.cpu().numpy() - o3.cpu().numpy())) > 1e-3
    # bottom-right causal rule of the backend's SDPA member (HipAttentionKernels.cs:69-71)
    want4, _, _ = oracle.attention_f32(q, k, v, 0.3, causal=True, query_offset=Sk - Sq)
    o4, _ = eng.ScaledDotProductAttention(dev(q), dev(k), dev(v), None, 0.3, isCausal=True, returnWeights=False)
    assert mixed_err(o4.cpu().numpy(), want4) <= FP32_TOL


def test_strided_qkv_from_packed_projection(be):
    # Q, K, V read in place from a packed [B*S, 3*dModel] activation and O written as [B,S,H,d]: the layout of
    # the fused MHA forward (CpuEngine.MultiHeadAttention.cs:409-420, 501-514), no permute kernels.
    from aidotnet.tensors_amd import AttnDesc
    rng = np.random.default_rng(12)
    B, S, H, D = 2, 75, 3, 32
    dm = H * D
    qkv = _rand(rng, B * S, 3 * dm)
    t = dev(qkv)
    out = torch.full((B, S, H, D), float("nan"), device="cuda")
    d = AttnDesc(B=B, H=H, Hkv=H, Sq=S, Sk=S, D=D, scale=1 / math.sqrt(D), causal=1)
    for name in ("q_strides", "k_strides", "v_strides"):
        getattr(d, name)[:] = [S * 3 * dm, D, 3 * dm]
    d.o_strides[:] = [S * dm, D, dm]
    lse = torch.empty(B, H, S, device="cuda")
    be._attn("f32", be.WrapTensor(t), _Off(t, dm), _Off(t, 2 * dm), be.WrapTensor(out), be.WrapTensor(lse),
             None, None, None, d)
    x = qkv.reshape(B, S, 3, H, D)
    q, k, v = (np.ascontiguousarray(x[:, :, i].transpose(0, 2, 1, 3)) for i in range(3))
    want, lse_w, _ = oracle.attention_f32(q, k, v, 1 / math.sqrt(D), True)
    assert mixed_err(out.cpu().numpy().transpose(0, 2, 1, 3), want) <= FP32_TOL
    assert mixed_err(lse.cpu().numpy(), lse_w) <= FP32_TOL


@pytest.mark.parametrize("kind,D", [("bf16", 128), ("f16", 128), ("bf16", 256), ("f16", 256), ("bf16", 64)])
def test_strided_16bit_qkv_from_packed_projection(be, kind, D):
    # the same packed [B*S, 3*dModel] activation in the 16-bit types: K and V rows 3*dModel elements apart go through the
    # direct-to-LDS tile loads of the head-dimension-128 / 256 kernels (row stride as a run-time value), O is written [B,S,H,d]
    from aidotnet.tensors_amd import AttnDesc
    rng = np.random.default_rng(D + len(kind))
    B, S, H = 2, 203, 3
    dm = H * D
    qkv = _rand(rng, B * S, 3 * dm)
    bits, wide = round_to(qkv, kind)
    dt = TORCH16[kind]
    t = from_bits16(bits, dt)
    out = torch.full((B, S, H, D), float("nan"), device="cuda")
    d = AttnDesc(B=B, H=H, Hkv=H, Sq=S, Sk=S, D=D, scale=1 / math.sqrt(D), causal=1)
    for name in ("q_strides", "k_strides", "v_strides"):
        getattr(d, name)[:] = [S * 3 * dm, D, 3 * dm]
    d.o_strides[:] = [S * dm, D, dm]
    lse = torch.empty(B, H, S, device="cuda")
    be._attn(kind, be.WrapTensor(t), _Off(t, dm), _Off(t, 2 * dm), be.WrapTensor(out), be.WrapTensor(lse), None, None, None, d)
    x = wide.reshape(B, S, 3, H, D)
    q, k, v = (np.ascontiguousarray(x[:, :, i].transpose(0, 2, 1, 3)) for i in range(3))
    o64, lse64 = oracle.attention_f64(q, k, v, 1 / math.sqrt(D), True, 0)
    assert mixed_err(out.cpu().numpy().transpose(0, 2, 1, 3), o64) <= HALF_TOL
    assert mixed_err(lse.cpu().numpy(), lse64) <= 1e-3


@pytest.mark.parametrize("kind,D", [("bf16", 128), ("f16", 128), ("f32", 64), ("bf16", 64), ("bf16", 256), ("f16", 256)])
def test_output_layouts_of_the_direct_to_lds_kernels(be, kind, D):
    # The kernels that stage O through LDS write whole rows; the same call with O laid out [B,S,H,D] (row stride H*D), with a
    # dense O, and with an O that starts 4 bytes off a 16-byte boundary (element-wise stores) must give the same numbers.
    from aidotnet.tensors_amd import AttnDesc
    B, H, S = 2, 3, 333
    g = torch.Generator(device="cuda"); g.manual_seed(D + len(kind))
    dt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[kind]
    q, k, v = (torch.randn(B, H, S, D, device="cuda", generator=g).to(dt) for _ in range(3))
    sc = 1 / math.sqrt(D)

    def run(o_view, o_strides):
        d = AttnDesc(B=B, H=H, Hkv=H, Sq=S, Sk=S, D=D, scale=sc, causal=1)
        d.o_strides[:] = o_strides
        lse = torch.full((B, H, S), float("nan"), device="cuda")
        be._attn(kind, be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), o_view, be.WrapTensor(lse), None, None, None, d)
        return lse

    dense = torch.full((B, H, S, D), float("nan"), device="cuda")
    lse0 = run(be.WrapTensor(dense), [H * S * D, S * D, D])
    bshd = torch.full((B, S, H, D), float("nan"), device="cuda")
    lse1 = run(be.WrapTensor(bshd), [S * H * D, D, H * D])
    raw = torch.full((B * H * S * D + 1,), float("nan"), device="cuda")
    lse2 = run(_Off(raw, 1), [H * S * D, S * D, D])
    torch.cuda.synchronize()
    assert torch.isfinite(dense).all()
    assert torch.equal(bshd.permute(0, 2, 1, 3), dense) and torch.equal(lse1, lse0)
    assert torch.equal(raw[1:].view(B, H, S, D), dense) and torch.equal(lse2, lse0)
    assert torch.isnan(raw[0])
    ref = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=True)
    assert float((dense.double() - ref).abs().max()) <= (1e-4 if kind == "f32" else 2e-2)


class _Off:
    """A buffer view starting `off` elements into a tensor (raw device pointer arithmetic)."""

    def __init__(self, t, off):
        self.Handle = t.data_ptr() + off * t.element_size()


def test_argument_errors(be):
    from aidotnet.tensors_amd import ArgumentException, ArgumentOutOfRangeException
    b = be.AllocateBuffer(4096)
    with pytest.raises(ArgumentOutOfRangeException):
        be.ScaledDotProductAttention(b, b, b, b, None, None, 0, 1, 4, 4, 8, 1.0, False)     # HipBackend.cs:6123-6124
    with pytest.raises(ArgumentException):
        be.ScaledDotProductAttention(b, b, b, b, None, None, 1, 3, 4, 4, 8, 1.0, False, 0.0, 2)   # heads % kvHeads
    with pytest.raises(ArgumentException):
        be.ScaledDotProductAttention(b, b, b, b, None, None, 8, 8, 64, 64, 64, 1.0, False)  # undersized buffers
    with pytest.raises(ArgumentOutOfRangeException):
        be.FlashAttentionV2(b, b, b, b, b, 1, 1, 2, 2, 512, 1.0, False)                    # headDim > 256


# ------------------------------------------------------------------------------------------- 16-bit
HALF_CASES = [
    (1, 2, 2, 4, 4, 16, True, 0),
    (2, 3, 3, 33, 65, 32, False, 0),
    (1, 4, 4, 70, 70, 64, True, 0),
    (2, 4, 2, 17, 40, 32, True, 23),
    (1, 2, 2, 256, 256, 128, True, 0),
    (2, 3, 3, 512, 512, 128, True, 0),      # four query tiles: the fast kernel pairs tile 3 with 0 and 2 with 1 in one workgroup
    (1, 2, 2, 384, 384, 128, True, 0),      # three query tiles: no pairing
    (1, 3, 3, 700, 700, 128, True, 0),      # six tiles, the last one partial
    (1, 2, 2, 130, 200, 72, True, 70),
    (1, 1, 1, 64, 96, 256, False, 0),
    (1, 2, 2, 300, 300, 256, True, 0),
    (1, 2, 1, 130, 200, 200, False, 0),
    (1, 2, 2, 5, 9, 7, False, 0),
    (8, 49, 7, 200, 200, 64, True, 0),      # 784 workgroups (GQA): the head-group order of a causal grid of several rounds
    (33, 16, 16, 100, 150, 256, False, 0),  # head dim 256 on more than 512 workgroups: 32-key tiles, two workgroups per CU
    (33, 16, 8, 130, 130, 200, True, 0),
    (7, 37, 37, 300, 300, 48, True, 0),     # 777 workgroups, heads straddle the XCDs
]


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,D,causal,offset", HALF_CASES)
def test_half_attention_within_tolerance(be, kind, B, H, Hkv, Sq, Sk, D, causal, offset):
    rng = np.random.default_rng(B + 3 * H + 7 * Sq + 11 * Sk + D + len(kind))
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    (qb, qw), (kb, kw), (vb, vw) = round_to(q, kind), round_to(k, kind), round_to(v, kind)
    scale = 1.0 / math.sqrt(D)
    o64, lse64 = oracle.attention_f64(qw, kw, vw, scale, causal, offset)     # truth over the rounded inputs
    dt = TORCH16[kind]
    out = torch.full((B, H, Sq, D), float("nan"), device="cuda")
    lse = torch.empty(B, H, Sq, device="cuda")
    args = (be.WrapTensor(from_bits16(qb, dt)), be.WrapTensor(from_bits16(kb, dt)), be.WrapTensor(from_bits16(vb, dt)))
    be.FlashAttentionHalf(kind, *args, be.WrapTensor(out), be.WrapTensor(lse), B, H, Sq, Sk, D, scale, causal, offset, Hkv)
    assert mixed_err(out.cpu().numpy(), o64) <= HALF_TOL
    assert mixed_err(lse.cpu().numpy(), lse64) <= 1e-3                        # the logits are fp32-accumulated
    out16 = torch.zeros((B, H, Sq, D), dtype=dt, device="cuda")
    be.FlashAttentionHalf(kind, *args, be.WrapTensor(out16), None, B, H, Sq, Sk, D, scale, causal, offset, Hkv, True)
    assert mixed_err(out16.float().cpu().numpy(), o64) <= HALF_TOL
    if Sk >= 64:
        # differs from the fp32 result on unrounded inputs: the reduced-precision kernel really ran
        o32, _ = oracle.attention_f64(q, k, v, scale, causal, offset)
        assert np.max(np.abs(out.cpu().numpy() - o32)) > 1e-5


# ------------------------------------------------------------------------------------ full-size configs
def test_config3_fp32_causal_b8_h12_s512_d64(eng):
    rng = np.random.default_rng(512)
    B, H, S, D = 8, 12, 512, 64
    q, k, v = _rand(rng, B, H, S, D), _rand(rng, B, H, S, D), _rand(rng, B, H, S, D)
    o_cpu, lse_cpu, _ = oracle.attention_f32(q, k, v, 0.125, True)
    o, lse = eng.FlashAttention(dev(q), dev(k), dev(v), 0.125, True)
    o = o.cpu().numpy(); lse = lse.cpu().numpy()
    assert mixed_err(o, o_cpu) <= FP32_TOL and mixed_err(lse, lse_cpu) <= FP32_TOL
    o64, lse64 = oracle.attention_f64(q[:1, :3], k[:1, :3], v[:1, :3], 0.125, True)
    assert mixed_err(o[:1, :3], o64) <= FP32_TOL and mixed_err(lse[:1, :3], lse64) <= FP32_TOL


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_config4_half_causal_b4_h32_s2048_d128(be, kind):
    # B=4, H=32, S=2048, d=128: the oracle checks sampled (batch, head) slices at full sequence length;
    # every slice is additionally held to the size-independent properties (row 0 = V[0], finite LSE).
    B, H, S, D = 4, 32, 2048, 128
    dt = TORCH16[kind]
    g = torch.Generator(device="cuda"); g.manual_seed(2048)
    q = torch.randn(B, H, S, D, device="cuda", generator=g).to(dt)
    k = torch.randn(B, H, S, D, device="cuda", generator=g).to(dt)
    v = torch.randn(B, H, S, D, device="cuda", generator=g).to(dt)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((B, H, S, D), float("nan"), device="cuda")
    lse = torch.empty(B, H, S, device="cuda")
    be.FlashAttentionHalf(kind, be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out), be.WrapTensor(lse),
                          B, H, S, S, D, scale, True)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert torch.allclose(out[:, :, 0], v[:, :, 0].float(), atol=1e-6)
    for (b, h) in [(0, 0), (1, 17), (3, 31)]:
        qs, ks, vs = (t[b:b + 1, h:h + 1].float().cpu().numpy() for t in (q, k, v))
        o64, lse64 = oracle.attention_f64(qs, ks, vs, scale, True)
        assert mixed_err(out[b, h].cpu().numpy(), o64[0, 0]) <= HALF_TOL
        assert mixed_err(lse[b, h].cpu().numpy(), lse64[0, 0]) <= 1e-3
    # every (batch, head) slice, so that a wrong head / workgroup remap cannot hide: the whole LSE column and eight sampled query
    # rows per slice against a float64 softmax of the same rounded inputs (computed on the device; the arithmetic of
    # oracle.attention_f64, which the three slices above tie it to)
    rng = np.random.default_rng(5)
    causal_mask = torch.ones(S, S, device="cuda", dtype=torch.bool).tril()
    for b in range(B):
        for h in range(H):
            q64, k64, v64 = q[b, h].double(), k[b, h].double(), v[b, h].double()
            logits = (q64 @ k64.T) * scale
            logits = logits.masked_fill(~causal_mask, float("-inf"))
            lse_ref = torch.logsumexp(logits, dim=1)
            # the row sum adds the probabilities as rounded to the storage type (the numbers the P V product uses): relative
            # error up to 2^-12 per term in fp16, 2^-9 in bf16, hence the wider bound for bf16
            assert float((lse[b, h].double() - lse_ref).abs().max()) <= (1e-3 if kind == "f16" else 4e-3), (b, h)
            rows = torch.from_numpy(rng.choice(S, 8, replace=False)).cuda()
            o_ref = torch.softmax(logits[rows], dim=1) @ v64
            err = ((out[b, h][rows].double() - o_ref).abs() / (1 + o_ref.abs())).max()
            assert float(err) <= HALF_TOL, (b, h)


# --------------------------------------------------------------- head-dim-128 fast path (direct-to-LDS kernel)
FAST_CASES = [
    (1, 1, 1, 1, 1, False, 0),
    (1, 2, 2, 5, 9, False, 0),
    (2, 3, 3, 128, 128, True, 0),
    (1, 2, 1, 130, 200, True, 70),        # GQA, bottom-right causal, ragged tiles
    (1, 4, 4, 257, 63, True, 0),          # Sq > Sk top-left causal: one partial K/V tile
    (2, 2, 2, 64, 1000, False, 0),
    (1, 2, 2, 1, 4097, True, 4096),       # decode shape through the prefill kernel
    (1, 1, 1, 300, 300, True, 0),
    # few query tiles over a long key sequence: the keys of every tile are cut into ranges that run side by side (merge pass)
    (1, 4, 2, 16, 2100, True, 2084),      # a few new tokens against a long cache, GQA
    (1, 2, 2, 300, 1100, True, 800),      # chunked prefill, three query tiles, ragged ranges
    (2, 2, 2, 200, 3000, False, 0),
    (1, 2, 2, 1024, 1024, True, 0),       # causal self-attention: late ranges are empty for early query tiles
    (1, 3, 3, 130, 1500, True, 100),      # small offset: most ranges are empty for every row
]


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,causal,offset", FAST_CASES)
def test_fast_path_d128_matches_oracle_and_general_kernel(be, kind, B, H, Hkv, Sq, Sk, causal, offset):
    D = 128
    rng = np.random.default_rng(B + 3 * H + 7 * Sq + 11 * Sk + len(kind))
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    (qb, qw), (kb, kw), (vb, vw) = round_to(q, kind), round_to(k, kind), round_to(v, kind)
    scale = 1.0 / math.sqrt(D)
    o64, lse64 = oracle.attention_f64(qw, kw, vw, scale, causal, offset)
    dt = TORCH16[kind]
    args = (be.WrapTensor(from_bits16(qb, dt)), be.WrapTensor(from_bits16(kb, dt)), be.WrapTensor(from_bits16(vb, dt)))
    outs = {}
    try:
        # 2 / 3: the phase-structured / the software-pipelined prefill kernel (key ranges side by side where the shape asks for
        # them in both); False: the general kernel
        for fast in (2, 3, False):
            be.SetAttentionFastPath(fast)
            out = torch.full((B, H, Sq, D), float("nan"), device="cuda")
            lse = torch.full((B, H, Sq), float("nan"), device="cuda")
            be.FlashAttentionHalf(kind, *args, be.WrapTensor(out), be.WrapTensor(lse), B, H, Sq, Sk, D, scale, causal, offset, Hkv)
            outs[fast] = (out.cpu().numpy(), lse.cpu().numpy())
            assert mixed_err(outs[fast][0], o64) <= HALF_TOL
            assert mixed_err(outs[fast][1], lse64) <= 1e-3
        # the kernels agree far inside the 16-bit tolerance (all round P to 16 bits, at different scalings)
        assert mixed_err(outs[2][0], outs[False][0]) <= 1e-2 and mixed_err(outs[3][0], outs[False][0]) <= 1e-2
        for fast in (2, 3):
            be.SetAttentionFastPath(fast)
            out16 = torch.zeros((B, H, Sq, D), dtype=dt, device="cuda")
            be.FlashAttentionHalf(kind, *args, be.WrapTensor(out16), None, B, H, Sq, Sk, D, scale, causal, offset, Hkv, True)
            assert mixed_err(out16.float().cpu().numpy(), o64) <= HALF_TOL
    finally:
        be.SetAttentionFastPath(True)


def test_fast_path_all_masked_rows_and_large_logits(be):
    # rows above the diagonal with a negative offset see no key: O = 0, LSE = -inf (CpuEngine.cs:29243-29249);
    # logits of magnitude ~60 exercise the lazily raised exponent reference
    # (the second size runs with its keys cut into ranges: rows without keys must stay O = 0, LSE = -inf through the merge)
    for S in (200, 1100):
        B, H, D = 1, 2, 128
        rng = np.random.default_rng(77)
        q, k, v = 3 * _rand(rng, B, H, S, D), 3 * _rand(rng, B, H, S, D), _rand(rng, B, H, S, D)
        (qb, qw), (kb, kw), (vb, vw) = round_to(q, "bf16"), round_to(k, "bf16"), round_to(v, "bf16")
        o64, lse64 = oracle.attention_f64(qw, kw, vw, 0.5, True, -3)
        dt = torch.bfloat16
        try:
            for fast in (2, 3):         # (the pipelined kernel meets logits it cannot hold against a standing reference: its safe form)
                be.SetAttentionFastPath(fast)
                out = torch.full((B, H, S, D), float("nan"), device="cuda"); lse = torch.full((B, H, S), float("nan"), device="cuda")
                be.FlashAttentionHalf("bf16", be.WrapTensor(from_bits16(qb, dt)), be.WrapTensor(from_bits16(kb, dt)), be.WrapTensor(from_bits16(vb, dt)),
                                      be.WrapTensor(out), be.WrapTensor(lse), B, H, S, S, D, 0.5, True, -3)
                o = out.cpu().numpy(); l = lse.cpu().numpy()
                assert np.all(o[:, :, :3] == 0) and np.all(np.isneginf(l[:, :, :3]))
                assert mixed_err(o, o64) <= HALF_TOL
                assert mixed_err(l[:, :, 3:], lse64[:, :, 3:]) <= 1e-3
        finally:
            be.SetAttentionFastPath(True)


LONG_PASS_CASES = [
    # B, H, Hkv, Sq, Sk, causal, offset, q scale: passes long enough that every part of the pipelined kernel runs (the assembly loop
    # through several rounds of both LDS stages, tile loads that end before the pass does, paired causal query tiles)
    (1, 4, 4, 2048, 2048, True, 0, 1.0),
    (1, 2, 1, 1024, 2048 + 37, False, 0, 1.0),      # partial last tile behind a long run
    (1, 4, 2, 512, 4096, True, 3584, 1.0),          # chunked prefill against a long cache, GQA
    (2, 2, 2, 1280, 1280, True, 0, 1.0),            # ten query tiles: paired
    (1, 3, 3, 1152, 1152, True, 0, 1.0),            # nine query tiles: not paired
    (1, 2, 2, 1024, 1024, True, 0, 40.0),           # logits far beyond what a standing reference holds: the safe form
    (1, 2, 2, 700, 1900, False, 0, 25.0),
]


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,causal,offset,qscale", LONG_PASS_CASES)
def test_pipelined_prefill_long_passes(be, kind, B, H, Hkv, Sq, Sk, causal, offset, qscale):
    D = 128
    rng = np.random.default_rng(5 * B + 3 * H + 7 * Sq + 11 * Sk + len(kind))
    q, k, v = qscale * _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    (qb, qw), (kb, kw), (vb, vw) = round_to(q, kind), round_to(k, kind), round_to(v, kind)
    scale = 1.0 / math.sqrt(D)
    o64, lse64 = oracle.attention_f64(qw, kw, vw, scale, causal, offset)
    dt = TORCH16[kind]
    args = (be.WrapTensor(from_bits16(qb, dt)), be.WrapTensor(from_bits16(kb, dt)), be.WrapTensor(from_bits16(vb, dt)))
    outs = {}
    try:
        for fast in (3, 2):
            be.SetAttentionFastPath(fast)
            out = torch.full((B, H, Sq, D), float("nan"), device="cuda")
            lse = torch.full((B, H, Sq), float("nan"), device="cuda")
            be.FlashAttentionHalf(kind, *args, be.WrapTensor(out), be.WrapTensor(lse), B, H, Sq, Sk, D, scale, causal, offset, Hkv)
            outs[fast] = (out.cpu().numpy(), lse.cpu().numpy())
            assert mixed_err(outs[fast][0], o64) <= HALF_TOL
            assert mixed_err(outs[fast][1], lse64) <= 1e-3
            out16 = torch.zeros((B, H, Sq, D), dtype=dt, device="cuda")
            be.FlashAttentionHalf(kind, *args, be.WrapTensor(out16), None, B, H, Sq, Sk, D, scale, causal, offset, Hkv, True)
            assert mixed_err(out16.float().cpu().numpy(), o64) <= HALF_TOL
        assert mixed_err(outs[3][0], outs[2][0]) <= 1e-2
    finally:
        be.SetAttentionFastPath(True)


# --------------------------------------------------------------- fp32 head-dim-64 direct-to-LDS form of the general kernel
@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,causal,offset", FAST_CASES + [(2, 4, 2, 17, 40, True, 23), (1, 4, 4, 70, 70, True, 0),
                                                                   (1, 2, 2, 512, 512, True, 0), (1, 3, 3, 200, 50, True, 0),
                                                                   (8, 49, 7, 200, 200, True, 0)])
@pytest.mark.parametrize("D", [64, 128])
def test_fp32_d64_direct_load_form_matches_oracle_and_general_form(be, eng, D, B, H, Hkv, Sq, Sk, causal, offset):
    rng = np.random.default_rng(B + 3 * H + 7 * Sq + 11 * Sk + 64)
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    scale = 1.0 / math.sqrt(D)
    o64, lse64 = oracle.attention_f64(q, k, v, scale, causal, offset)
    outs = {}
    try:
        for direct in (True, False):
            be.SetAttentionFastPath(direct)
            o, lse = eng.FlashAttention(dev(q), dev(k), dev(v), scale, causal, queryOffset=offset)
            outs[direct] = (o.cpu().numpy(), lse.cpu().numpy())
            assert mixed_err(outs[direct][0], o64) <= FP32_TOL and mixed_err(outs[direct][1], lse64) <= FP32_TOL
    finally:
        be.SetAttentionFastPath(True)
    # the two forms multiply and sum the same values in the same order: identical results
    assert np.array_equal(outs[True][0], outs[False][0]) and np.array_equal(outs[True][1], outs[False][1])


# --------------------------------------------------------------- head dimension 256, 16-bit: the phase-structured kernel at that width
D256_CASES = [
    (1, 1, 1, 1, 1, False, 0),
    (1, 2, 2, 5, 9, False, 0),
    (2, 3, 3, 128, 128, True, 0),
    (1, 2, 1, 130, 200, True, 70),        # GQA, bottom-right causal, ragged tiles
    (1, 4, 4, 257, 63, True, 0),          # Sq > Sk top-left causal: one partial K/V tile
    (2, 2, 2, 64, 1000, False, 0),
    (1, 2, 2, 1, 1025, True, 1024),       # decode shape through the prefill kernel
    (1, 1, 1, 300, 300, True, 0),
    (1, 2, 2, 512, 512, True, 0),         # paired causal query tiles (two passes per workgroup)
    (1, 2, 2, 1024, 1024, True, 0),
    (3, 4, 2, 200, 456, False, 0),
]


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,causal,offset", D256_CASES)
def test_half_d256_kernel_matches_oracle_and_the_other_forms(be, kind, B, H, Hkv, Sq, Sk, causal, offset):
    D = 256
    rng = np.random.default_rng(B + 3 * H + 7 * Sq + 11 * Sk + len(kind) + 256)
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    (qb, qw), (kb, kw), (vb, vw) = round_to(q, kind), round_to(k, kind), round_to(v, kind)
    scale = 1.0 / math.sqrt(D)
    o64, lse64 = oracle.attention_f64(qw, kw, vw, scale, causal, offset)
    dt = TORCH16[kind]
    args = (be.WrapTensor(from_bits16(qb, dt)), be.WrapTensor(from_bits16(kb, dt)), be.WrapTensor(from_bits16(vb, dt)))
    outs = {}
    try:
        # True: the 64-key-tile kernel of 512-byte rows; 2: the 32-key-tile direct-to-LDS form; False: the general kernel
        for fast in (True, 2, False):
            be.SetAttentionFastPath(fast)
            out = torch.full((B, H, Sq, D), float("nan"), device="cuda")
            lse = torch.full((B, H, Sq), float("nan"), device="cuda")
            be.FlashAttentionHalf(kind, *args, be.WrapTensor(out), be.WrapTensor(lse), B, H, Sq, Sk, D, scale, causal, offset, Hkv)
            outs[fast] = (out.cpu().numpy(), lse.cpu().numpy())
            assert mixed_err(outs[fast][0], o64) <= HALF_TOL
            assert mixed_err(outs[fast][1], lse64) <= 1e-3
            out16 = torch.zeros((B, H, Sq, D), dtype=dt, device="cuda")
            be.FlashAttentionHalf(kind, *args, be.WrapTensor(out16), None, B, H, Sq, Sk, D, scale, causal, offset, Hkv, True)
            assert mixed_err(out16.float().cpu().numpy(), o64) <= HALF_TOL
        assert mixed_err(outs[True][0], outs[False][0]) <= 1e-2 and mixed_err(outs[2][0], outs[False][0]) <= 1e-2
    finally:
        be.SetAttentionFastPath(True)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_half_d256_causal_b2_h32_s2048_every_slice(be, kind):
    # the full grid of the head-dimension-256 kernel (1024 query tiles in pairs, one workgroup per CU, two rounds): one slice against
    # the oracle, every (batch, head) slice against a float64 softmax of the same rounded inputs computed on the device (whole LSE
    # column, eight sampled rows of O), so that a wrong head / tile / pass remap cannot hide
    B, H, S, D = 2, 32, 2048, 256
    dt = TORCH16[kind]
    g = torch.Generator(device="cuda"); g.manual_seed(256)
    q = torch.randn(B, H, S, D, device="cuda", generator=g).to(dt)
    k = torch.randn(B, H, S, D, device="cuda", generator=g).to(dt)
    v = torch.randn(B, H, S, D, device="cuda", generator=g).to(dt)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((B, H, S, D), float("nan"), device="cuda")
    lse = torch.empty(B, H, S, device="cuda")
    be.FlashAttentionHalf(kind, be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out), be.WrapTensor(lse),
                          B, H, S, S, D, scale, True)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert torch.allclose(out[:, :, 0], v[:, :, 0].float(), atol=1e-6)
    qs, ks, vs = (t[1:2, 17:18].float().cpu().numpy() for t in (q, k, v))
    o64, lse64 = oracle.attention_f64(qs, ks, vs, scale, True)
    assert mixed_err(out[1, 17].cpu().numpy(), o64[0, 0]) <= HALF_TOL
    assert mixed_err(lse[1, 17].cpu().numpy(), lse64[0, 0]) <= 1e-3
    rng = np.random.default_rng(6)
    causal_mask = torch.ones(S, S, device="cuda", dtype=torch.bool).tril()
    for b in range(B):
        for h in range(H):
            q64, k64, v64 = q[b, h].double(), k[b, h].double(), v[b, h].double()
            logits = ((q64 @ k64.T) * scale).masked_fill(~causal_mask, float("-inf"))
            lse_ref = torch.logsumexp(logits, dim=1)
            assert float((lse[b, h].double() - lse_ref).abs().max()) <= (1e-3 if kind == "f16" else 4e-3), (b, h)
            rows = torch.from_numpy(rng.choice(S, 8, replace=False)).cuda()
            o_ref = torch.softmax(logits[rows], dim=1) @ v64
            err = ((out[b, h][rows].double() - o_ref).abs() / (1 + o_ref.abs())).max()
            assert float(err) <= HALF_TOL, (b, h)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,causal,offset", FAST_CASES + [(2, 4, 2, 17, 40, True, 23), (1, 4, 4, 70, 70, True, 0),
                                                                   (1, 2, 2, 512, 512, True, 0), (1, 3, 3, 200, 50, True, 0)])
def test_half_d64_direct_load_form_matches_oracle_and_general_form(be, kind, B, H, Hkv, Sq, Sk, causal, offset):
    D = 64
    rng = np.random.default_rng(B + 3 * H + 7 * Sq + 11 * Sk + len(kind) + 64)
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    (qb, qw), (kb, kw), (vb, vw) = round_to(q, kind), round_to(k, kind), round_to(v, kind)
    scale = 1.0 / math.sqrt(D)
    o64, lse64 = oracle.attention_f64(qw, kw, vw, scale, causal, offset)
    dt = TORCH16[kind]
    args = (be.WrapTensor(from_bits16(qb, dt)), be.WrapTensor(from_bits16(kb, dt)), be.WrapTensor(from_bits16(vb, dt)))
    outs = {}
    try:
        for direct in (True, False):
            be.SetAttentionFastPath(direct)
            out = torch.full((B, H, Sq, D), float("nan"), device="cuda")
            lse = torch.full((B, H, Sq), float("nan"), device="cuda")
            be.FlashAttentionHalf(kind, *args, be.WrapTensor(out), be.WrapTensor(lse), B, H, Sq, Sk, D, scale, causal, offset, Hkv)
            outs[direct] = (out.cpu().numpy(), lse.cpu().numpy())
            assert mixed_err(outs[direct][0], o64) <= HALF_TOL
            assert mixed_err(outs[direct][1], lse64) <= 1e-3
        be.SetAttentionFastPath(True)
        out16 = torch.zeros((B, H, Sq, D), dtype=dt, device="cuda")
        be.FlashAttentionHalf(kind, *args, be.WrapTensor(out16), None, B, H, Sq, Sk, D, scale, causal, offset, Hkv, True)
        assert mixed_err(out16.float().cpu().numpy(), o64) <= HALF_TOL
    finally:
        be.SetAttentionFastPath(True)
    # same values multiplied and summed in the same order by both forms
    assert np.array_equal(outs[True][0], outs[False][0]) and np.array_equal(outs[True][1], outs[False][1])
