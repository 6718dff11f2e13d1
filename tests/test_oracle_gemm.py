"""Pins the CPU GEMM restatement (oracle/oracle_gemm.c) without running the reference.

Checks are chosen so that a dropped term, a transposed operand, a wrong panel index or a
wrong edge mask fails: exact integer arithmetic on dyadic inputs, the reference's literal
known answers and edge shapes, numpy float64 matmul, and thread-count independence.
"""
import numpy as np
import pytest

import oracle

# (m, k, n): reference edge shapes -- TensorMatMulSimdFallbackTests.cs:69-73 (m,n,k)=(7,13,11),(96,130,80),(37,53,71);
# SgemmCachedBTests.cs:10-41 13x17x10; Fp16Bf16GemmTests.cs:23-62; plus shapes that cross Kc=512, Nc=4096, Mc=128.
SHAPES = [(1, 1, 1), (7, 11, 13), (96, 80, 130), (37, 71, 53), (13, 17, 10), (4, 8, 32), (16, 20, 24),
          (3, 7, 5), (1, 1, 64), (6, 512, 16), (5, 513, 15), (129, 1030, 33), (256, 64, 512), (130, 70, 4100)]


def _dyadic(rng, shape, hi=8):
    """Small integers / 8: every partial sum is exact in fp32, so any summation order gives the same bits."""
    return (rng.integers(-hi, hi + 1, size=shape).astype(np.float32)) / np.float32(8.0)


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_sgemm_exact_on_dyadic_inputs(m, k, n):
    rng = np.random.default_rng(m * 1000003 + k * 1009 + n)
    a = _dyadic(rng, (m, k)); b = _dyadic(rng, (k, n))
    want = ((a.astype(np.float64) * 8).astype(np.int64) @ (b.astype(np.float64) * 8).astype(np.int64)).astype(np.float64) / 64.0
    for threads in (1, 4):
        got = oracle.sgemm(a, b, m, k, n, threads=threads)
        assert got.dtype == np.float32 and got.shape == (m, n)
        assert np.array_equal(got.astype(np.float64), want), f"threads={threads}"


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_sgemm_close_to_float64_and_thread_independent(m, k, n):
    rng = np.random.default_rng(7 + m + k + n)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    truth = a.astype(np.float64) @ b.astype(np.float64)
    c1 = oracle.sgemm(a, b, m, k, n, threads=1)
    c8 = oracle.sgemm(a, b, m, k, n, threads=8)
    assert np.array_equal(c1, c8)                      # DeterministicParallelGemmContractTests.cs:49-54
    assert np.all(np.abs(c1 - truth) <= 1e-4 * (1 + np.abs(truth)))
    assert np.allclose(oracle.gemm_f64(a, b, m, k, n), truth, rtol=1e-12, atol=1e-12)


def test_sgemm_identity_and_scaling_known_answers():
    # BatchMatMulAndAttentionTests.cs:17-56 style: A*I = A, A*(2I) = 2A
    rng = np.random.default_rng(3)
    a = rng.standard_normal((19, 23)).astype(np.float32)
    eye = np.eye(23, dtype=np.float32)
    assert np.array_equal(oracle.sgemm(a, eye, 19, 23, 23), a)
    assert np.array_equal(oracle.sgemm(a, 2 * eye, 19, 23, 23), 2 * a)
    # non-symmetric known answer: catches a transposed operand
    a2 = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    b2 = np.array([[7, 8], [9, 10], [11, 12]], np.float32)
    assert np.array_equal(oracle.sgemm(a2, b2, 2, 3, 2), np.array([[58, 64], [139, 154]], np.float32))


def test_sgemm_degenerate_k_zero_clears_output():
    # SimdGemm.cs:1292-1301: k <= 0 leaves a zeroed C
    c = oracle.sgemm(np.zeros(0, np.float32), np.zeros(0, np.float32), 3, 0, 4)
    assert np.array_equal(c, np.zeros((3, 4), np.float32))


def test_sgemm_ex_transposes():
    rng = np.random.default_rng(5)
    m, k, n = 21, 34, 18
    a = _dyadic(rng, (m, k)); b = _dyadic(rng, (k, n))
    want = oracle.sgemm(a, b, m, k, n)
    assert np.array_equal(oracle.sgemm_ex(a, k, False, np.ascontiguousarray(b.T), k, True, m, k, n), want)
    assert np.array_equal(oracle.sgemm_ex(np.ascontiguousarray(a.T), m, True, b, n, False, m, k, n), want)


def test_gemm_alpha_beta_contract():
    rng = np.random.default_rng(6)
    m, n, k = 9, 14, 11
    a = _dyadic(rng, (m, k)); b = _dyadic(rng, (k, n)); c0 = _dyadic(rng, (m, n))
    ab = a.astype(np.float64) @ b.astype(np.float64)
    got = oracle.gemm_alpha_beta(a, b, c0, m, n, k, alpha=0.5, beta=2.0)
    assert np.array_equal(got.astype(np.float64), 0.5 * ab + 2.0 * c0)
    # beta = 0 must ignore (possibly NaN) stale contents -- GemmBeta0BitExactTests.cs:24-34
    poisoned = np.full((m, n), np.nan, np.float32)
    got0 = oracle.gemm_alpha_beta(a, b, poisoned, m, n, k, alpha=1.0, beta=0.0)
    assert np.array_equal(got0.astype(np.float64), ab)
    gotT = oracle.gemm_alpha_beta(a, np.ascontiguousarray(b.T), poisoned, m, n, k, trans_b=True)
    assert np.array_equal(gotT.astype(np.float64), ab)


def test_bf16_literal_known_answer():
    # BFloat16KernelsTests.cs:55-68
    a = oracle.f32_to_bf16(np.array([[1, 2, 3], [4, 5, 6]], np.float32))
    b = oracle.f32_to_bf16(np.array([[7, 8], [9, 10], [11, 12]], np.float32))
    o16, o32 = oracle.bf16gemm(a, b, 2, 3, 2)
    assert np.array_equal(oracle.bf16_to_f32(o16), np.array([[58, 64], [139, 154]], np.float32))
    assert np.array_equal(o32, np.array([[58, 64], [139, 154]], np.float32))
    ah = oracle.f32_to_f16(np.array([[1, 2, 3], [4, 5, 6]], np.float32))
    bh = oracle.f32_to_f16(np.array([[7, 8], [9, 10], [11, 12]], np.float32))
    h16, h32 = oracle.hgemm(ah, bh, 2, 3, 2)
    assert np.array_equal(oracle.f16_to_f32(h16), np.array([[58, 64], [139, 154]], np.float32))


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("m,n,k", [(4, 32, 8), (16, 24, 20), (3, 5, 7), (1, 64, 1), (96, 96, 96), (7, 13, 11)])
def test_half_gemms_against_fp64_of_rounded_inputs(kind, m, n, k):
    # Fp16Bf16GemmTests.cs:23-62, 108-121: truth = fp64 sum over the SAME rounded inputs,
    # bound relTol * max(1, |truth|) with relTol 6e-3 (fp16) / 2e-2 (bf16)
    rng = np.random.default_rng(11 + m + n + k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    if kind == "f16":
        ab, bb = oracle.f32_to_f16(a), oracle.f32_to_f16(b)
        aw, bw = oracle.f16_to_f32(ab), oracle.f16_to_f32(bb)
        o16, o32 = oracle.hgemm(ab, bb, m, k, n)
        back, tol = oracle.f16_to_f32(o16), 6e-3
        assert np.array_equal(o16, oracle.f32_to_f16(o32))
    else:
        ab, bb = oracle.f32_to_bf16(a), oracle.f32_to_bf16(b)
        aw, bw = oracle.bf16_to_f32(ab), oracle.bf16_to_f32(bb)
        o16, o32 = oracle.bf16gemm(ab, bb, m, k, n)
        back, tol = oracle.bf16_to_f32(o16), 2e-2
        assert np.array_equal(o16, oracle.f32_to_bf16(o32))
    truth = aw.astype(np.float64) @ bw.astype(np.float64)
    assert np.all(np.abs(back - truth) <= tol * np.maximum(1.0, np.abs(truth)))
    assert np.all(np.abs(o32 - truth) <= 1e-5 * (1 + np.abs(truth)))


def test_half_gemm_exact_on_dyadic_inputs():
    rng = np.random.default_rng(21)
    m, k, n = 9, 29, 12            # k % 8 != 0 exercises the scalar tail
    a = _dyadic(rng, (m, k), hi=4); b = _dyadic(rng, (k, n), hi=4)
    want = a.astype(np.float64) @ b.astype(np.float64)
    _, h32 = oracle.hgemm(oracle.f32_to_f16(a), oracle.f32_to_f16(b), m, k, n)
    _, b32 = oracle.bf16gemm(oracle.f32_to_bf16(a), oracle.f32_to_bf16(b), m, k, n)
    assert np.array_equal(h32.astype(np.float64), want)
    assert np.array_equal(b32.astype(np.float64), want)
