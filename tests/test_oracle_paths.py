"""The reference's secondary CPU paths: the no-pack ``SimdGemm.SgemmDirect`` kernel, ``GotoGemmFp32.RunParallel`` and the tiled
``Simd.FusedAttention`` with ``FastExp256`` (restated in oracle/oracle_paths.c), pinned on the CPU and used as the checker of the
GPU fp32 GEMM / attention at the shapes the reference sends down those paths.

Shapes and bounds follow the reference's own tests: tests/AiDotNet.Tensors.Tests/Engines/BlasManagedThinMDirectTests.cs:27-52
((m,k,n) = (128,784,512), (256,512,512), (512,784,512), (130,520,512), (200,640,256), (64,1024,512), (1024,784,512), relative
error < 1e-3 against the scalar loop) and Engines/Compilation/CompilationComponentTests.cs:110-150 (FlashAttentionForward against
the naive softmax at seqQ = seqK = 16, d = 32, |diff| < 1e-3).  This build holds its own 1e-4 mixed bound on top.
"""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from _util import dev, dyadic, mixed_err, rel_frobenius

THIN_M = [(128, 784, 512), (256, 512, 512), (512, 784, 512), (130, 520, 512), (200, 640, 256), (64, 1024, 512), (1024, 784, 512)]   # (m, k, n)


def rnd(shape, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)


def f32(x):
    return np.float32(x)


def fused_chain_exact(arow, bcol):
    """One fused multiply-add chain from 0 in ascending k, evaluated in exact rationals with one rounding per step."""
    acc = Fraction(0)
    for x, y in zip(arow, bcol):
        acc = Fraction(float(f32(float(acc + Fraction(float(x)) * Fraction(float(y))))))
    return f32(float(acc))


def test_fraction_rounding_helper_is_a_single_rounding():
    # float(Fraction) rounds correctly (to double), and double -> float32 of a sum whose exact value has < 53 significant bits
    # is again a single rounding; products of two float32 are exact in double (48 bits).  Known case: fma(1+2^-23, 1+2^-23, -1)
    x = f32(1 + 2.0 ** -23)
    exact = Fraction(float(x)) * Fraction(float(x)) - 1
    assert exact == Fraction(2, 2 ** 23) + Fraction(1, 2 ** 46)           # the low term a separate multiply would lose
    assert f32(x * x) - f32(1) == f32(2.0 ** -22)                         # unfused: low term gone


# ------------------------------------------------------------------------------------------------- SgemmDirect
def test_direct_gate_follows_the_reference_thresholds():
    g = oracle.sgemm_direct_applies
    assert g(64, 512, 1024) and g(128, 64, 128)                           # per-head attention sized products
    assert not g(128, 784, 512)                                           # k > 512: reaches the kernel through the thin-M carve-out instead
    t = oracle.thin_m_direct_applies
    assert all(t(m, n, k) for (m, k, n) in THIN_M)                        # every shape of the reference's thin-M test is routed
    assert not t(63, 512, 512) and not t(1025, 512, 512) and not t(128, 520, 512) and not t(128, 512, 1025) and not t(128, 508, 512)
    assert not t(64, 64, 128)                                             # below 2^20 multiply-adds
    assert g(4096, 64, 4096)                                              # tall-thin: m >= 256, k <= 512, work <= 4 Gi
    assert not g(4096, 768, 3072)                                         # k > 512 and not tall-thin
    assert not g(128, 512, 780)                                           # n % 8 != 0
    assert not g(5, 64, 64)                                               # m < Mr
    assert not g(8192, 512, 8192)                                         # work > 4 Gi
    assert g(512, 128, 512) and not g(200, 1024, 256)                     # small work but k > 512 -> packed path


@pytest.mark.parametrize("m,k,n", THIN_M)
def test_direct_kernel_reference_shapes(m, k, n):
    a = rnd((m, k), m + n, 0.5); b = rnd((k, n), k + n, 0.5)
    got = oracle.sgemm_direct(a, b, m, k, n)
    t = a.astype(np.float64) @ b.astype(np.float64)
    assert np.max(np.abs(got - t) / np.maximum(np.abs(t), 1.0)) < 1e-3    # the reference test's own bound
    assert mixed_err(got, t) <= 3e-5                                      # one 512- to 1024-term fp32 chain per element


def test_direct_kernel_is_one_fused_chain_and_accumulate_adds_after():
    m, k, n = 13, 40, 24
    a = rnd((m, k), 1); b = rnd((k, n), 2); c0 = rnd((m, n), 3)
    store = oracle.sgemm_direct(a, b, m, k, n)
    acc = oracle.sgemm_direct(a, b, m, k, n, c0)
    for (i, j) in [(0, 0), (5, 17), (12, 23), (6, 8)]:
        e = fused_chain_exact(a[i], b[:, j])
        assert store[i, j] == e
        assert acc[i, j] == f32(c0[i, j] + e)                             # C + acc, not a chain that starts from C
    # an unfused chain differs somewhere: the pin would catch a restatement that rounds the product
    unf = np.zeros((m, n), np.float32)
    for p in range(k):
        unf = (unf + (a[:, p:p + 1] * b[p:p + 1, :]).astype(np.float32)).astype(np.float32)
    assert not np.array_equal(unf, store)


def test_direct_kernel_exact_on_dyadic_inputs_and_equals_the_tiled_restatement():
    rng = np.random.default_rng(5)
    m, k, n = 70, 300, 48
    a = dyadic(rng, (m, k)); b = dyadic(rng, (k, n))
    assert np.array_equal(oracle.sgemm_direct(a, b, m, k, n).astype(np.float64), a.astype(np.float64) @ b.astype(np.float64))
    # k <= 512 is one K-panel of the packed path: the 6x16 micro-kernel there is the same fused chain, written independently
    for (m, k, n) in [(64, 512, 96), (130, 256, 520), (19, 77, 40)]:
        a = rnd((m, k), m); b = rnd((k, n), n)
        assert np.array_equal(oracle.sgemm_direct(a, b, m, k, n), oracle.sgemm(a, b, m, k, n))
        assert np.array_equal(oracle.sgemm_direct(a, b, m, k, n, threads=4), oracle.sgemm_direct(a, b, m, k, n))


# ------------------------------------------------------------------------------------------------- GotoGemmFp32
def test_goto_block_choice_table():
    cb = oracle.goto_choose_blocks
    assert cb(2048, 2048, 16) == (192, 256, 256) and cb(1536, 1536, 4) == (192, 256, 256)
    assert cb(1024, 1024, 16) == (96, 128, 256) and cb(640, 4096, 16) == (96, 128, 256)
    # the source comment's worked cases for 16 workers: 256^2 -> 2 x 8 tiles of (128, 32); 512^2 -> 4 x 4 tiles of (128, 128)
    assert cb(256, 256, 16) == (128, 32, 256)
    assert cb(512, 512, 16) == (128, 128, 256)
    assert cb(64, 1024, 16) == (64, 64, 256)                              # ic clamps to 1, nc = 1024 / 16
    assert cb(192, 640, 16) == (96, 80, 256)                              # round(1.5) = 2 (ties to even), nc = 640 / 8
    assert cb(320, 640, 16) == (160, 80, 256)                             # round(2.5) = 2
    assert cb(600, 600, 16) == (120, 128, 256) and cb(2048, 600, 16) == (120, 128, 256)


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (512, 512, 768), (130, 520, 512), (200, 75, 300), (97, 50, 513), (6, 16, 1), (5, 3, 7)])
def test_goto_gemm_against_float64(m, n, k):
    a = rnd((m, k), m + k, 0.5); b = rnd((k, n), n + k, 0.5)
    got = oracle.goto_gemm(a, b, m, k, n)
    assert not np.isnan(got).any()
    assert mixed_err(got, a.astype(np.float64) @ b.astype(np.float64)) <= 1e-5
    assert np.array_equal(got, oracle.goto_gemm(a, b, m, k, n, threads=1))


def test_goto_gemm_panel_order_and_scalar_tails_by_hand():
    # tile (mc, nc, kc) = (10, 20, 8): rows 6..9 and columns 16..19 of a tile are scalar tails; k = 20 -> panels 8, 8, 4
    m, n, k = 17, 33, 20
    a = rnd((m, k), 11); b = rnd((k, n), 12)
    got = oracle.goto_gemm(a, b, m, k, n, blocks=(10, 20, 8))

    def element(i, j):
        ti, tj = i % 10, j % 20
        eff_mc = min(10, m - (i - ti)); eff_nc = min(20, n - (j - tj))
        vector = ti < eff_mc - eff_mc % 6 and tj < eff_nc - eff_nc % 16
        c = f32(0)
        for pc in range(0, k, 8):
            ar, bc = a[i, pc:pc + 8], b[pc:pc + 8, j]
            if vector:
                part = fused_chain_exact(ar, bc)
                c = part if pc == 0 else f32(c + part)
            else:
                s = f32(0)
                for x, y in zip(ar, bc):
                    s = f32(s + f32(x * y))
                c = f32(c + s)
        return c

    for (i, j) in [(0, 0), (5, 15), (5, 16), (6, 0), (9, 19), (10, 20), (15, 32), (16, 31), (16, 5), (3, 25)]:
        assert got[i, j] == element(i, j), (i, j)
    rng = np.random.default_rng(7)
    ad = dyadic(rng, (m, k)); bd = dyadic(rng, (k, n))
    assert np.array_equal(oracle.goto_gemm(ad, bd, m, k, n, blocks=(10, 20, 8)).astype(np.float64), ad.astype(np.float64) @ bd.astype(np.float64))


# ------------------------------------------------------------------------------------------------- FastExp256 + FusedAttention
def test_fast_exp_closed_forms_and_error():
    fe = oracle.fast_exp
    assert fe(np.float32(0.0)) == 1.0
    x = np.linspace(-87.0, 88.0, 20001, dtype=np.float32)
    rel = np.abs(fe(x).astype(np.float64) / np.exp(x.astype(np.float64)) - 1.0)
    assert rel.max() < 2e-6                                               # degree-6 polynomial on |r| <= ln2/2: ~1e-7 truncation + rounding
    assert rel.max() > 1e-9                                               # and it is the polynomial, not libm
    # clamp: everything below -87.3365 gives the same tiny positive value (a masked logit is not an exact zero)
    lo = fe(np.array([-87.3365, -100.0, -np.inf], np.float32))
    assert lo[0] == lo[1] == lo[2] and 0 < lo[0] < 2e-38
    assert fe(np.float32(np.inf)) == fe(np.float32(88.7228)) == fe(np.float32(1e9))     # upper clamp (n = 128 there: the exponent field overflows)
    # the exponent field carries n: shifting the argument by k * ln2hi (exact in fp32 for small k, so r is unchanged up to ln2lo * k)
    for kshift in (1, 2, 8):
        x0 = np.float32(0.125)
        ratio = float(np.ravel(fe(np.float32(x0 + kshift * 0.693359375)))[0]) / float(np.ravel(fe(x0))[0])
        assert abs(ratio / math.exp(kshift * 0.693359375) - 1.0) < 1e-6
    # monotone on a fine grid inside one reduction interval
    g = fe(np.linspace(-0.3, 0.3, 4001, dtype=np.float32))
    assert np.all(np.diff(g) >= 0)


def naive_attention64(q, k, v, scale, causal):
    s = np.einsum("...qd,...kd->...qk", q.astype(np.float64), k.astype(np.float64)) * scale
    if causal:
        sq, sk = s.shape[-2:]
        s = np.where(np.arange(sq)[:, None] < np.arange(sk)[None, :], -np.inf, s)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    return (p / p.sum(axis=-1, keepdims=True)) @ v.astype(np.float64)


@pytest.mark.parametrize("sq,sk,d,causal", [(16, 16, 32, False), (16, 16, 32, True), (70, 70, 64, True), (33, 97, 40, False), (5, 9, 7, False),
                                            (64, 64, 128, True), (1, 50, 64, False)])
def test_fused_attention_fastexp_against_naive_softmax(sq, sk, d, causal):
    q = rnd((3, sq, d), sq + d); k = rnd((3, sk, d), sk + d + 1); v = rnd((3, sk, d), sk + d + 2)
    got = oracle.fused_attention_fastexp(q, k, v, 1.0 / math.sqrt(d), causal)
    t = naive_attention64(q, k, v, 1.0 / math.sqrt(d), causal)
    assert np.max(np.abs(got - t)) < 1e-3                                 # the reference test's bound
    assert mixed_err(got, t) <= 2e-6 * 8                                  # fast exponential (2e-6 relative) on weights in [0, 1]
    assert np.array_equal(got, oracle.fused_attention_fastexp(q, k, v, 1.0 / math.sqrt(d), causal, threads=1))


def test_fused_attention_closed_forms():
    # equal keys: uniform weights, output = mean of V; one key: output = that V row exactly (weight fast_exp(0) = 1, 1/1 = 1)
    d = 16
    q = rnd((1, 40, d), 1); k = np.tile(rnd((1, 1, d), 2), (1, 40, 1)); v = rnd((1, 40, d), 3)
    got = oracle.fused_attention_fastexp(q, k, v, 0.25, False)
    assert np.allclose(got, v.mean(axis=1, keepdims=True), rtol=0, atol=2e-6)
    got = oracle.fused_attention_fastexp(q, k[:, :1], v[:, :1], 0.25, False)
    assert np.array_equal(got, np.tile(v[:, :1], (1, 40, 1)))
    # causal: query 0 sees key 0 only; the masked keys of its tile weigh exp(-87.3365) ~ 1e-38 each and vanish in fp32
    got = oracle.fused_attention_fastexp(q, rnd((1, 40, d), 4), v, 0.25, True)
    assert np.array_equal(got[0, 0], v[0, 0])
    # the tiled path and the engine's per-row softmax path (oracle_attention.c) are the same function within fp32 rounding
    qq = rnd((2, 3, 50, 32), 7); kk = rnd((2, 3, 50, 32), 8); vv = rnd((2, 3, 50, 32), 9)
    o, _, _ = oracle.attention_f32(qq, kk, vv, 0.2, causal=True)
    assert mixed_err(oracle.fused_attention_fastexp(qq, kk, vv, 0.2, True), o) <= 2e-5


# ----------------------------------------------------------------------------------------------------------------- GPU
@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    b = Mi355Backend()
    yield b
    b.Dispose()


def gpu_gemm(be, a, b, m, n, k, beta=0.0, c0=None):
    c = dev(c0) if c0 is not None else torch.full((m, n), float("nan"), device="cuda")
    be.Gemm(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(c), m, n, k, 1.0, beta)
    return c.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n", THIN_M)
def test_gpu_gemm_at_the_direct_kernel_shapes(be, m, k, n):
    assert oracle.thin_m_direct_applies(m, n, k)
    a = rnd((m, k), m + n, 0.5); b = rnd((k, n), k + n, 0.5)
    got = gpu_gemm(be, a, b, m, n, k)
    ref = oracle.sgemm_direct(a, b, m, k, n, threads=8)
    t = a.astype(np.float64) @ b.astype(np.float64)
    assert np.max(np.abs(got - t) / np.maximum(np.abs(t), 1.0)) < 1e-3
    assert mixed_err(got, ref) <= 1e-4 and mixed_err(got, t) <= 1e-4
    c0 = rnd((m, n), 99)
    acc = gpu_gemm(be, a, b, m, n, k, 1.0, c0)
    assert mixed_err(acc, oracle.sgemm_direct(a, b, m, k, n, c0, threads=8)) <= 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (512, 512, 768), (1024, 1024, 1024), (200, 75, 300), (97, 50, 513), (1536, 1536, 320)])
def test_gpu_gemm_against_the_goto_path(be, m, n, k):
    a = rnd((m, k), m + k, 0.5); b = rnd((k, n), n + k, 0.5)
    got = gpu_gemm(be, a, b, m, n, k)
    assert mixed_err(got, oracle.goto_gemm(a, b, m, k, n)) <= 1e-4
    assert rel_frobenius(got, a.astype(np.float64) @ b.astype(np.float64)) < 1e-5


@pytest.mark.gpu
def test_gpu_gemm_dyadic_equals_both_paths_bit_for_bit(be):
    rng = np.random.default_rng(3)
    m, k, n = 256, 512, 520
    a = dyadic(rng, (m, k)); b = dyadic(rng, (k, n))
    got = gpu_gemm(be, a, b, m, n, k)
    assert np.array_equal(got, oracle.sgemm_direct(a, b, m, k, n, threads=8))
    assert np.array_equal(got, oracle.goto_gemm(a, b, m, k, n))


@pytest.mark.gpu
@pytest.mark.parametrize("b_,h,sq,sk,d,causal", [(1, 1, 16, 16, 32, False), (1, 1, 16, 16, 32, True), (2, 4, 128, 128, 64, True), (1, 3, 70, 97, 40, False),
                                                 (2, 12, 512, 512, 64, True), (1, 2, 200, 200, 128, True)])
def test_gpu_attention_against_the_fused_fastexp_path(be, b_, h, sq, sk, d, causal):
    from aidotnet.tensors_amd import Mi355Engine
    eng = Mi355Engine(be)
    q = rnd((b_, h, sq, d), sq + d); k = rnd((b_, h, sk, d), sk + d + 1); v = rnd((b_, h, sk, d), sk + d + 2)
    scale = 1.0 / math.sqrt(d)
    out = eng.FlashAttention(dev(q), dev(k), dev(v), scale, causal)
    out = (out[0] if isinstance(out, tuple) else out).cpu().numpy()
    ref = oracle.fused_attention_fastexp(q, k, v, scale, causal)
    assert np.max(np.abs(out - ref)) < 1e-3                               # the reference test's bound
    assert mixed_err(out, ref) <= 1e-4
    assert mixed_err(out, naive_attention64(q, k, v, scale, causal)) <= 1e-4
