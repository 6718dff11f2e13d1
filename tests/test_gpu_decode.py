"""GPU parity of decode attention (one query row per head) through the C ABI against the CPU oracle.

Reference precedent: FlashDecodeHipTests.cs:43-130 (tests/AiDotNet.Tensors.Tests/Engines/DirectGpu): in-test
DecodeOracle, tolerance 2e-3 + 2e-3 * |e|, split-count independence, grouped-query heads.  The task's bar
is tighter and is what is asserted: 1e-4 (fp32), 2e-2 (bf16 / fp16) in the mixed metric.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import TORCH16, dev, from_bits16, mixed_err, round_to

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    b = Mi355Backend()
    yield b
    b.Dispose()


def _run_flash_decode(be, heads, kv, d, seq, splits, seed):
    rng = np.random.default_rng(seed)
    k = rng.uniform(-1, 1, (seq, kv, d)).astype(np.float32)
    v = rng.uniform(-1, 1, (seq, kv, d)).astype(np.float32)
    q = rng.uniform(-1, 1, (heads, d)).astype(np.float32)
    scale = 1.0 / math.sqrt(d)
    out = be.FlashDecode(be.AllocateBuffer(q), be.AllocateBuffer(k), be.AllocateBuffer(v), heads, kv, d, seq, scale, splits)
    got = be.DownloadBuffer(out).numpy().reshape(heads, d)
    want = oracle.decode_f32(q, k, v, heads, kv, d, seq, scale)
    return got, want


@pytest.mark.parametrize("heads,d,seq,splits", [(4, 64, 40, 8), (8, 32, 100, 8), (4, 64, 7, 8), (4, 64, 64, 1), (6, 48, 77, 0),
                                                (2, 128, 3000, 0), (2, 128, 3000, 5), (3, 20, 513, 2), (1, 256, 700, 3)])
def test_mha_decode_matches_oracle(be, heads, d, seq, splits):
    got, want = _run_flash_decode(be, heads, heads, d, seq, splits, 0xFDE + heads + seq + splits)
    assert np.all(np.abs(got - want) <= 2e-3 + 2e-3 * np.abs(want))        # the reference's tolerance
    assert mixed_err(got, want) <= 1e-4                                     # the task's


# query heads per K/V head 4, 8 (two workgroups of four), 3 (one head per workgroup), 6 and 2 (pairs): the heads that share a workgroup
# share its K/V loads
@pytest.mark.parametrize("heads,kv,d,seq,splits", [(8, 2, 64, 50, 8), (8, 1, 32, 300, 4), (12, 4, 128, 1025, 0), (12, 2, 64, 333, 0),
                                                   (4, 2, 128, 200, 3), (16, 4, 256, 130, 2)])
def test_gqa_decode_matches_oracle(be, heads, kv, d, seq, splits):
    got, want = _run_flash_decode(be, heads, kv, d, seq, splits, 0xABC + heads + kv + seq)
    assert mixed_err(got, want) <= 1e-4


def test_split_count_independence(be):
    # FlashDecodeHipTests.cs:107-117
    base, _ = _run_flash_decode(be, 4, 4, 64, 2000, 1, 99)
    for s in (2, 3, 7, 8):
        other, _ = _run_flash_decode(be, 4, 4, 64, 2000, s, 99)
        assert np.max(np.abs(other - base)) <= 2e-6


def test_decode_guards(be):
    from aidotnet.tensors_amd import ArgumentException, ArgumentOutOfRangeException
    b = be.AllocateBuffer(1024)
    for bad in ((0, 1, 8, 4), (4, 3, 8, 4), (4, 4, 512, 4), (4, 4, 8, 0)):   # GpuKernelGuards.cs:41-52
        with pytest.raises(ArgumentOutOfRangeException):
            be.FlashDecode(b, b, b, bad[0], bad[1], bad[2], bad[3], 1.0)
    with pytest.raises(ArgumentException):
        be.FlashDecode(b, b, b, 8, 8, 64, 100, 1.0)                          # undersized K/V


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
@pytest.mark.parametrize("B,H,Hkv,S,D", [(3, 4, 4, 333, 64), (2, 8, 2, 1000, 128), (1, 2, 2, 65, 32)])
def test_batched_decode_all_types_and_layouts(be, kind, layout, B, H, Hkv, S, D):
    rng = np.random.default_rng(B + H + S + D)
    q = rng.standard_normal((B, H, 1, D)).astype(np.float32)
    k = rng.standard_normal((B, Hkv, S, D)).astype(np.float32)
    v = rng.standard_normal((B, Hkv, S, D)).astype(np.float32)
    scale = 1.0 / math.sqrt(D)
    if kind == "f32":
        qw, kw, vw = q, k, v
        tq, tk, tv = dev(q), dev(k), dev(v)
        tol = 1e-4
    else:
        (qb, qw), (kb, kw), (vb, vw) = round_to(q, kind), round_to(k, kind), round_to(v, kind)
        dt = TORCH16[kind]
        tq, tk, tv = from_bits16(qb, dt), from_bits16(kb, dt), from_bits16(vb, dt)
        tol = 2e-2
    o64, lse64 = oracle.attention_f64(qw, kw, vw, scale)
    if layout == "bshd":
        tk = tk.transpose(1, 2).contiguous(); tv = tv.transpose(1, 2).contiguous()
    out = torch.full((B, H, 1, D), float("nan"), device="cuda")
    lse = torch.empty(B, H, 1, device="cuda")
    be.DecodeAttention(kind, be.WrapTensor(tq), be.WrapTensor(tk), be.WrapTensor(tv), be.WrapTensor(out), B, H, S, D, scale,
                       Hkv, 0, False, be.WrapTensor(lse), layout)
    assert mixed_err(out.cpu().numpy(), o64) <= tol
    assert mixed_err(lse.cpu().numpy(), lse64) <= (1e-4 if kind == "f32" else 1e-3)
    if kind != "f32":
        out16 = torch.zeros((B, H, 1, D), dtype=TORCH16[kind], device="cuda")
        be.DecodeAttention(kind, be.WrapTensor(tq), be.WrapTensor(tk), be.WrapTensor(tv), be.WrapTensor(out16), B, H, S, D, scale,
                           Hkv, 3, True, None, layout)
        assert mixed_err(out16.float().cpu().numpy(), o64) <= tol


def _decode_truth_f64(q, k, v, scale):
    """float64 softmax(scale q K^T) V and log-sum-exp of EVERY (batch, head) slice on the device, from the same rounded inputs:
    the arithmetic of oracle.attention_f64 (the callers tie the two together on sampled slices).  q [B,H,1,D]; k, v [B,Hkv,S,D]."""
    B, H, _, D = q.shape
    Hkv = k.shape[1]
    o = torch.empty(B, H, D, dtype=torch.float64, device="cuda")
    lse = torch.empty(B, H, dtype=torch.float64, device="cuda")
    for b in range(B):              # one batch entry at a time: the float64 copy of a 2 GiB cache would be 8 GiB
        k64, v64 = k[b].double(), v[b].double()                                   # [Hkv, S, D]
        q64 = q[b, :, 0].double().reshape(Hkv, H // Hkv, D)                       # query head h reads K/V head h / (H / Hkv)
        logits = torch.einsum("ugd,usd->ugs", q64, k64) * scale
        lse[b] = torch.logsumexp(logits, dim=2).reshape(H)
        o[b] = torch.einsum("ugs,usd->ugd", torch.softmax(logits, dim=2), v64).reshape(H, D)
    return o, lse


def _check_every_slice(out, lse, q, k, v, scale, samples):
    o64, lse64 = _decode_truth_f64(q, k, v, scale)
    err = ((out[:, :, 0].double() - o64).abs() / (1 + o64.abs())).amax(dim=2)     # per (batch, head)
    worst = int(err.argmax())
    assert float(err.max()) <= 2e-2, ("slice", worst // err.shape[1], worst % err.shape[1], float(err.max()))
    # the row sum adds the probabilities as rounded to bf16 (the numbers the P V product uses): up to 2^-9 relative per term
    lerr = (lse.reshape(lse64.shape).double() - lse64).abs()
    assert float(lerr.max()) <= 4e-3, ("lse slice", int(lerr.argmax()), float(lerr.max()))
    G = q.shape[1] // k.shape[1]
    for (b, h) in samples:          # the device float64 arithmetic against the oracle's
        qs = q[b:b + 1, h:h + 1].float().cpu().numpy()
        ks, vs = (t[b:b + 1, h // G:h // G + 1].float().cpu().numpy() for t in (k, v))
        oo, ll = oracle.attention_f64(qs, ks, vs, scale)
        # (1e-6: the oracle takes the scale as the float the C ABI carries, the device expression as a double)
        assert np.max(np.abs(o64[b, h].cpu().numpy() - oo[0, 0, 0])) <= 1e-6
        assert abs(float(lse64[b, h]) - float(np.ravel(ll)[0])) <= 1e-6
        assert mixed_err(out[b, h].cpu().numpy(), oo[0, 0]) <= 2e-2


def test_config5_decode_bf16_b32_h32_s4096_d128(be):
    # B=32, H=32, q_len=1, KV length 4096, d=128, contiguous [32,32,4096,128] bf16 cache: every one of the 1024 (batch, head)
    # outputs and log-sum-exps against a float64 softmax of the same bf16 inputs; three slices tie that arithmetic to the oracle.
    B, H, S, D = 32, 32, 4096, 128
    g = torch.Generator(device="cuda"); g.manual_seed(4096)
    q = torch.randn(B, H, 1, D, device="cuda", generator=g).to(torch.bfloat16)
    k = torch.randn(B, H, S, D, device="cuda", generator=g).to(torch.bfloat16)
    v = torch.randn(B, H, S, D, device="cuda", generator=g).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((B, H, 1, D), float("nan"), device="cuda")
    lse = torch.empty(B, H, 1, device="cuda")
    be.DecodeAttention("bf16", be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out), B, H, S, D, scale,
                       0, 0, False, be.WrapTensor(lse))
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    _check_every_slice(out, lse, q, k, v, scale, [(0, 0), (13, 7), (31, 31)])
    # the prefill kernel run at Sq = 1 on the same cache is a second implementation of the same function
    ref = torch.full((B, H, 1, D), float("nan"), device="cuda")
    ref_lse = torch.empty(B, H, 1, device="cuda")
    be.FlashAttentionHalf("bf16", be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(ref), be.WrapTensor(ref_lse),
                          B, H, 1, S, D, scale, True, S - 1)
    assert mixed_err(out.cpu().numpy(), ref.cpu().numpy()) <= 2e-2
    assert mixed_err(lse.cpu().numpy(), ref_lse.cpu().numpy()) <= 1e-3


def test_grouped_decode_bf16_b32_h32_hkv8_s4096_d128_every_slice(be):
    # the grouped-query form of the same decode step (8 K/V heads for 32 query heads) at full size, every slice as above
    B, H, Hkv, S, D = 32, 32, 8, 4096, 128
    g = torch.Generator(device="cuda"); g.manual_seed(4097)
    q = torch.randn(B, H, 1, D, device="cuda", generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, S, D, device="cuda", generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, S, D, device="cuda", generator=g).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((B, H, 1, D), float("nan"), device="cuda")
    lse = torch.empty(B, H, 1, device="cuda")
    be.DecodeAttention("bf16", be.WrapTensor(q), be.WrapTensor(k), be.WrapTensor(v), be.WrapTensor(out), B, H, S, D, scale,
                       Hkv, 0, False, be.WrapTensor(lse))
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    _check_every_slice(out, lse, q, k, v, scale, [(0, 0), (17, 5), (31, 31)])


# Grouped-query decode at head dimension 128 in the 16-bit types: the query heads of a K/V head run as the rows of one query tile of
# the fast prefill kernel (one fetch of a K/V row for the whole group).  Checked against the fp64 oracle, against the per-head decode
# kernel (fast path switched off) and across split counts; G = H / Hkv from 2 to 48 (more than 32 rows: a second wave computes).
@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("B,H,Hkv,S,splits", [(2, 8, 4, 300, 0), (1, 32, 8, 4096, 0), (3, 12, 2, 1000, 3), (2, 32, 1, 777, 1), (5, 16, 8, 63, 0),
                                              (1, 48, 1, 500, 2), (2, 16, 2, 64, 1), (1, 8, 2, 129, 64), (4, 32, 8, 2048, 5)])
def test_grouped_decode_d128_matches_oracle_and_per_head_kernel(be, kind, B, H, Hkv, S, splits):
    D = 128
    rng = np.random.default_rng(B + 3 * H + 5 * Hkv + S)
    q = rng.standard_normal((B, H, 1, D)).astype(np.float32)
    k = rng.standard_normal((B, Hkv, S, D)).astype(np.float32)
    v = rng.standard_normal((B, Hkv, S, D)).astype(np.float32)
    scale = 1.0 / math.sqrt(D)
    (qb, qw), (kb, kw), (vb, vw) = round_to(q, kind), round_to(k, kind), round_to(v, kind)
    dt = TORCH16[kind]
    tq, tk, tv = from_bits16(qb, dt), from_bits16(kb, dt), from_bits16(vb, dt)
    o64, lse64 = oracle.attention_f64(qw, kw, vw, scale)

    def run(out16):
        out = torch.full((B, H, 1, D), float("nan"), device="cuda", dtype=dt if out16 else torch.float32)
        lse = torch.full((B, H, 1), float("nan"), device="cuda")
        be.DecodeAttention(kind, be.WrapTensor(tq), be.WrapTensor(tk), be.WrapTensor(tv), be.WrapTensor(out), B, H, S, D, scale,
                           Hkv, splits, out16, be.WrapTensor(lse))
        return out.float().cpu().numpy(), lse.cpu().numpy()

    got, lse = run(False)
    assert mixed_err(got, o64) <= 2e-2 and mixed_err(lse, lse64) <= 1e-3
    got16, _ = run(True)
    assert mixed_err(got16, o64) <= 2e-2
    be.SetAttentionFastPath(False)
    try:
        per_head, per_head_lse = run(False)
    finally:
        be.SetAttentionFastPath(True)
    assert mixed_err(got, per_head) <= 2e-2 and mixed_err(lse, per_head_lse) <= 1e-3
    assert mixed_err(per_head, o64) <= 2e-2
