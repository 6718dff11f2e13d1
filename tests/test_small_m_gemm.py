"""The m <= 8 fp32 GEMM (decode / batch-1 projections): oracle restatement of ``SimdGemm.SgemmNParallelSmallM``
(src/AiDotNet.Tensors/Engines/Simd/SimdGemm.NParallelSmallM.cs:31-109) and the GPU small-M path behind ``Gemm`` /
``GemmBiasActivationInto`` / ``GemmFp16WeightB``.

Inputs follow tests/AiDotNet.Tensors.Tests/Engines/Simd/SimdGemmNParallelSmallMTests.cs:17-103: Gaussian values from the test's
own xorshift64 generator (restated below), shapes (m,k,n) = (1,256,512), (2,320,768), (5,256,500), (8,384,1024), the
accumulate case (4,256,512), the dispatcher case (1,1024,4096) and the fused [Wq|Wk|Wv] projection; bound: relative Frobenius
error < 1e-4 against the scalar triple loop (here: the float64 product), plus this build's 1e-4 mixed bound.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import dev, mixed_err, rel_frobenius

MASK = (1 << 64) - 1


class Xorshift:
    """The generator of SimdGemmNParallelSmallMTests.cs:17-23 (xorshift64, Box-Muller on two draws)."""

    def __init__(self, seed):
        self.s = (seed | 1) & MASK

    def unit(self):
        x = self.s
        x ^= (x << 13) & MASK; x ^= x >> 7; x ^= (x << 17) & MASK
        self.s = x
        return (x >> 11) * (1.0 / (1 << 53))

    def gaussian(self, std):
        u1 = max(1e-12, self.unit()); u2 = self.unit()
        return np.float32(std * math.sqrt(-2 * math.log(u1)) * math.cos(2 * math.pi * u2))

    def arr(self, n, std):
        return np.array([self.gaussian(std) for _ in range(n)], np.float32)


def case(m, k, n, seed, with_c0=False):
    rng = Xorshift(seed)
    a = rng.arr(m * k, 0.1).reshape(m, k); b = rng.arr(k * n, 0.05).reshape(k, n)
    c0 = rng.arr(m * n, 1.0).reshape(m, n) if with_c0 else None
    return a, b, c0


def truth64(a, b, c0=None):
    t = a.astype(np.float64) @ b.astype(np.float64)
    return t if c0 is None else t + c0.astype(np.float64)


SHAPES = [(1, 256, 512), (2, 320, 768), (5, 256, 500), (8, 384, 1024)]


def test_xorshift_restatement_known_values():
    # first outputs of xorshift64 from state 1 (13, 7, 17): fixed by the recurrence, computed by hand for the first step:
    # x = 1 -> x ^= x<<13 -> 0x2001 -> x ^= x>>7 -> 0x2041 -> x ^= x<<17 -> 0x40822041
    r = Xorshift(1)
    r.unit()
    assert r.s == 0x40822041


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_oracle_small_m_overwrite(m, k, n):
    a, b, _ = case(m, k, n, m * 31 + k + n)
    got = oracle.sgemm_small_m(a, b, m, k, n)
    assert rel_frobenius(got, truth64(a, b)) < 1e-4 and mixed_err(got, truth64(a, b)) <= 1e-5


def test_oracle_small_m_accumulate_and_order():
    m, k, n = 4, 256, 512
    a, b, c0 = case(m, k, n, 123, True)
    got = oracle.sgemm_small_m(a, b, m, k, n, c0)
    assert rel_frobenius(got, truth64(a, b, c0)) < 1e-4
    # the update order is fixed by the algorithm (ascending k, multiply then add, starting from C): one column by hand
    j = 77
    for i in range(m):
        c = np.float32(c0[i, j])
        for p in range(k):
            c = np.float32(c + np.float32(a[i, p] * b[p, j]))
        assert c == got[i, j]
    # dyadic inputs: every order is exact
    ai = np.random.default_rng(0).integers(-8, 9, (m, k)).astype(np.float32) / 8
    bi = np.random.default_rng(1).integers(-8, 9, (k, n)).astype(np.float32) / 8
    assert np.array_equal(oracle.sgemm_small_m(ai, bi, m, k, n).astype(np.float64), ai.astype(np.float64) @ bi.astype(np.float64))


def test_oracle_fused_projections_equal_separate():
    m, k, nq = 2, 512, 512
    rng = Xorshift(55)
    a = rng.arr(m * k, 0.1).reshape(m, k)
    ws = [rng.arr(k * nq, 0.05).reshape(k, nq) for _ in range(3)]
    fused = oracle.sgemm_small_m(a, np.concatenate(ws, axis=1), m, k, 3 * nq)
    for i, w in enumerate(ws):
        assert np.array_equal(fused[:, i * nq:(i + 1) * nq], oracle.sgemm_small_m(a, w, m, k, nq))


# ----------------------------------------------------------------------------------------------------------------- GPU
@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    b = Mi355Backend()
    yield b
    b.SetGemmTile(0)
    b.Dispose()


def gpu_gemm(be, a, b, m, n, k, alpha=1.0, beta=0.0, c0=None):
    c = dev(c0) if c0 is not None else torch.full((m, n), float("nan"), device="cuda")
    be.Gemm(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(c), m, n, k, alpha, beta)
    return c.cpu().numpy()


@pytest.mark.gpu
# (the last two: row strides of 32 KiB and 128 KiB, where the K ranges are moved off multiples of 4 MiB -- at N = 32768 every range
# size is such a multiple and the search must give up)
@pytest.mark.parametrize("m,k,n", SHAPES + [(1, 1024, 4096), (3, 4096, 4096), (8, 1000, 1001), (7, 33, 130), (1, 320, 1280), (6, 5000, 260),
                                            (2, 2048, 8192), (1, 512, 32768)])
def test_gpu_small_m_overwrite(be, m, k, n):
    a, b, _ = case(m, k, n, m * 31 + k + n) if m * k + k * n < 600000 else (None, None, None)
    if a is None:
        rng = np.random.default_rng(m + k + n)
        a = (rng.standard_normal((m, k)) * 0.1).astype(np.float32); b = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    got = gpu_gemm(be, a, b, m, n, k)
    t = truth64(a, b)
    assert rel_frobenius(got, t) < 1e-4 and mixed_err(got, t) <= 1e-4
    assert mixed_err(got, oracle.sgemm_small_m(a, b, m, k, n)) <= 1e-4
    # the same call through the general tiled kernel agrees
    be.SetGemmTile(64)
    try:
        tiled = gpu_gemm(be, a, b, m, n, k)
    finally:
        be.SetGemmTile(0)
    assert mixed_err(got, tiled) <= 1e-4


@pytest.mark.gpu
def test_gpu_small_m_accumulate_and_alpha_beta(be):
    m, k, n = 4, 256, 512
    a, b, c0 = case(m, k, n, 123, True)
    got = gpu_gemm(be, a, b, m, n, k, 1.0, 1.0, c0)
    assert rel_frobenius(got, truth64(a, b, c0)) < 1e-4
    assert mixed_err(got, oracle.sgemm_small_m(a, b, m, k, n, c0)) <= 1e-4
    got = gpu_gemm(be, a, b, m, n, k, 0.5, -2.0, c0)
    assert mixed_err(got, 0.5 * truth64(a, b) - 2.0 * c0.astype(np.float64)) <= 1e-4
    # beta == 0 ignores what C held (NaN included)
    got = gpu_gemm(be, a, b, m, n, k, 1.0, 0.0, np.full((m, n), np.nan, np.float32))
    assert mixed_err(got, truth64(a, b)) <= 1e-4


@pytest.mark.gpu
def test_gpu_small_m_exact_on_dyadic_inputs_and_repeatable(be):
    m, k, n = 8, 2048, 1536
    a = np.random.default_rng(0).integers(-8, 9, (m, k)).astype(np.float32) / 8
    b = np.random.default_rng(1).integers(-8, 9, (k, n)).astype(np.float32) / 8
    got = gpu_gemm(be, a, b, m, n, k)
    assert np.array_equal(got.astype(np.float64), a.astype(np.float64) @ b.astype(np.float64))
    a2, b2, _ = case(5, 256, 500, 9)
    r1 = gpu_gemm(be, a2, b2, 5, 500, 256); r2 = gpu_gemm(be, a2, b2, 5, 500, 256)
    assert np.array_equal(r1, r2)                       # split order is fixed: no atomics


@pytest.mark.gpu
def test_gpu_fused_projections_equal_separate(be):
    m, k, nq = 2, 512, 512
    rng = Xorshift(55)
    a = rng.arr(m * k, 0.1).reshape(m, k)
    ws = [rng.arr(k * nq, 0.05).reshape(k, nq) for _ in range(3)]
    fused = gpu_gemm(be, a, np.ascontiguousarray(np.concatenate(ws, axis=1)), m, 3 * nq, k)
    for i, w in enumerate(ws):
        sep = gpu_gemm(be, a, w, m, nq, k)
        assert rel_frobenius(fused[:, i * nq:(i + 1) * nq], sep) < 1e-4
        assert rel_frobenius(sep, truth64(a, w)) < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n", [(1, 320, 1280), (4, 4096, 4096), (8, 1000, 1002), (2, 64, 65)])
def test_gpu_small_m_fp16_weights_and_epilogue(be, m, k, n):
    from _util import from_bits16, round_to
    rng = np.random.default_rng(m * k + n)
    a = rng.standard_normal((m, k)).astype(np.float32); b = (rng.standard_normal((k, n)) / math.sqrt(k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    bb, br = round_to(b, "f16")
    W = be.WrapTensor
    c = torch.full((m * n,), float("nan"), device="cuda")
    be.GemmFp16WeightB(W(dev(a)), W(from_bits16(bb, torch.float16)), W(dev(bias)), W(c), m, n, k, 1)
    t = np.maximum(truth64(a, br) + bias[None, :], 0.0)
    assert mixed_err(c.cpu().numpy().reshape(m, n), t) <= 1e-4
    c2 = torch.full((m * n,), float("nan"), device="cuda")
    be.GemmBiasActivationInto(W(dev(a)), W(dev(br)), W(dev(bias)), W(c2), m, n, k, 1)
    assert mixed_err(c2.cpu().numpy().reshape(m, n), t) <= 1e-4


# ------------------------------------------------------------------------------- fp32: 9 <= M <= 32 and split-K (few tiles, long K)
# M, K, N: the skinny path needs N % 128 == 0 and K % 32 == 0 (unequal K ranges included: 5 slabs x 37 K-tiles); the others go through
# K ranges run as batches of the tiled kernel (K >= 1024, K % 32 == 0, tiles that do not fill the chip) or stay unsplit
SKINNY32_SHAPES = [(9, 1024, 128), (16, 4096, 4096), (32, 1184, 640), (20, 2048, 1536), (32, 96, 256), (17, 32, 128),
                   (16, 1024, 1000), (33, 2048, 512), (128, 4096, 1024), (200, 3072, 768), (64, 11008, 320), (100, 1056, 300)]


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n", SKINNY32_SHAPES)
def test_gpu_fp32_skinny_and_split_k_match_oracle(be, m, k, n):
    rng = np.random.default_rng(m * 7 + k + 3 * n)
    a = (rng.standard_normal((m, k)) * 0.1).astype(np.float32); b = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    got = gpu_gemm(be, a, b, m, n, k)
    t = truth64(a, b)
    assert rel_frobenius(got, t) < 1e-4 and mixed_err(got, t) <= 1e-4
    assert mixed_err(got, oracle.sgemm(a, b, m, k, n, threads=oracle.max_threads())) <= 1e-4
    assert np.array_equal(got, gpu_gemm(be, a, b, m, n, k))          # fixed summation order: repeatable
    # alpha, beta and a NaN-filled C under beta == 0
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    got = gpu_gemm(be, a, b, m, n, k, 0.5, -2.0, c0)
    assert mixed_err(got, 0.5 * t - 2.0 * c0.astype(np.float64)) <= 1e-4
    got = gpu_gemm(be, a, b, m, n, k, 1.0, 0.0, np.full((m, n), np.nan, np.float32))
    assert mixed_err(got, t) <= 1e-4
    # B stored [N, K]
    c = torch.full((m, n), float("nan"), device="cuda")
    be.MatMulTransposed(be.WrapTensor(dev(a)), be.WrapTensor(dev(np.ascontiguousarray(b.T))), be.WrapTensor(c), m, n, k)
    assert mixed_err(c.cpu().numpy(), t) <= 1e-4
    # fused bias + activation
    bias = rng.standard_normal(n).astype(np.float32)
    c = torch.full((m, n), float("nan"), device="cuda")
    be.GemmBiasActivationInto(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(dev(bias)), be.WrapTensor(c), m, n, k, be.ACT_RELU)
    assert mixed_err(c.cpu().numpy(), np.maximum(t + bias.astype(np.float64), 0.0)) <= 1e-4


@pytest.mark.gpu
def test_gpu_fp32_skinny_exact_on_dyadic_inputs(be):
    m, k, n = 24, 2048, 1536
    a = np.random.default_rng(0).integers(-8, 9, (m, k)).astype(np.float32) / 8
    b = np.random.default_rng(1).integers(-8, 9, (k, n)).astype(np.float32) / 8
    assert np.array_equal(gpu_gemm(be, a, b, m, n, k).astype(np.float64), a.astype(np.float64) @ b.astype(np.float64))
    m, k, n = 128, 4096, 512                                          # split-K through the tiled kernel
    a = np.random.default_rng(2).integers(-8, 9, (m, k)).astype(np.float32) / 8
    b = np.random.default_rng(3).integers(-8, 9, (k, n)).astype(np.float32) / 8
    assert np.array_equal(gpu_gemm(be, a, b, m, n, k).astype(np.float64), a.astype(np.float64) @ b.astype(np.float64))
