"""Pre-packed weight operand (aidn_mi355_pack_b / aidn_mi355_gemm_packed_b): the GPU form of the reference's cached packed B
(SimdGemm.SgemmWithCachedB, src/AiDotNet.Tensors/Engines/Simd/SimdGemm.cs:327-684; its identity test
tests/AiDotNet.Tensors.Tests/Engines/Simd/SgemmCachedBTests.cs:10-41 holds the cached product equal to the plain one on
13 x 17 x 10).  The packed product must equal the plain product -- bit for bit on inputs whose partial sums are exact -- and the
oracle's restatement of the plain GEMM."""
import numpy as np
import pytest
import torch

import oracle
from _util import TORCH16, bits16, dev, dyadic, from_bits16, mixed_err, round_to

pytestmark = pytest.mark.gpu

# the reference's own shape, odd and even widths, few and many rows, short and long K, narrow N (padded C), wide N (direct stores)
SHAPES = [(13, 10, 17), (64, 1001, 300), (300, 301, 299), (1000, 1025, 130), (16, 1024, 512), (700, 4099, 77), (8, 4096, 1030),
          (2049, 2051, 70), (256, 1152, 1088), (40, 50257, 64), (4, 1001, 300), (1, 50257, 40), (8, 130, 515)]


@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    b = Mi355Backend()
    yield b
    b.Dispose()


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_packed_fp32_equals_plain_and_oracle(be, M, N, K):
    rng = np.random.default_rng(M + 3 * N + 5 * K)
    a = dyadic(rng, (M, K), hi=4); b = dyadic(rng, (K, N), hi=4)
    want = oracle.sgemm(a, b, M, K, N, threads=4)
    A = be.WrapTensor(dev(a))
    for transB in (False, True):
        bm = np.ascontiguousarray(b.T) if transB else b
        packed = be.PackB("f32", be.WrapTensor(dev(bm)), K, N, transB)
        c = torch.full(((M + 1) * N,), -7.0, device="cuda")
        be.GemmPackedB("f32", A, packed, None, be.WrapTensor(c), M, N, K, transB)
        assert np.array_equal(c[:M * N].cpu().numpy().reshape(M, N), want), transB
        assert bool((c[M * N:] == -7.0).all()), transB                      # nothing past the matrix
    # random data: same tolerance as the plain call, and bias / activation ride along
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32); b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    packed = be.PackB("f32", be.WrapTensor(dev(b)), K, N)
    c = torch.empty(M * N, device="cuda")
    be.GemmPackedB("f32", be.WrapTensor(dev(a)), packed, be.WrapTensor(dev(bias)), be.WrapTensor(c), M, N, K, False, 1)
    truth = np.maximum(a.astype(np.float64) @ b.astype(np.float64) + bias.astype(np.float64)[None, :], 0.0)
    assert mixed_err(c.cpu().numpy().reshape(M, N), truth) <= 1e-4


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_packed_half_equals_plain_and_oracle(be, kind, M, N, K):
    rng = np.random.default_rng(2 * M + N + 7 * K)
    a = dyadic(rng, (M, K), hi=4); b = dyadic(rng, (K, N), hi=4)
    ab, _ = round_to(a, kind); bb, _ = round_to(b, kind)
    want16, want32 = (oracle.hgemm if kind == "f16" else oracle.bf16gemm)(ab, bb, M, K, N)
    A = be.WrapTensor(from_bits16(ab, TORCH16[kind])); B = be.WrapTensor(from_bits16(bb, TORCH16[kind]))
    packed = be.PackB(kind, B, K, N)
    c32 = torch.full(((M + 1) * N,), -7.0, device="cuda")
    be.GemmPackedB(kind, A, packed, None, be.WrapTensor(c32), M, N, K, outputIsFp32=True)
    assert np.array_equal(c32[:M * N].cpu().numpy().reshape(M, N), want32.reshape(M, N))
    assert bool((c32[M * N:] == -7.0).all())
    c16 = torch.full(((M + 1) * N,), -7.0, device="cuda").to(TORCH16[kind])
    be.GemmPackedB(kind, A, packed, None, be.WrapTensor(c16), M, N, K, outputIsFp32=False)
    assert np.array_equal(bits16(c16[:M * N]).reshape(M, N), want16.reshape(M, N))
    assert bool((c16[M * N:].float() == -7.0).all())
    # the plain entry point on the same operands gives the same bits
    plain = torch.empty(M * N, device="cuda")
    (be.GemmFp16In32fOut if kind == "f16" else be.GemmBf16In32fOut)(A, B, be.WrapTensor(plain), M, N, K)
    assert torch.equal(plain, c32[:M * N])


def test_packed_b_is_reused_and_argument_errors(be):
    from aidotnet.tensors_amd import NotSupportedException
    rng = np.random.default_rng(5)
    K, N = 130, 1001
    b = dyadic(rng, (K, N), hi=4)
    bb, _ = round_to(b, "bf16")
    packed = be.PackB("bf16", be.WrapTensor(from_bits16(bb, torch.bfloat16)), K, N)
    assert packed.SizeInBytes == 192 * 1024 * 2                             # K to a multiple of 64, N to a multiple of 128
    for M in (1, 33, 600):                                                  # one packed weight, several activations
        a = dyadic(rng, (M, K), hi=4)
        ab, _ = round_to(a, "bf16")
        _, want32 = oracle.bf16gemm(ab, bb, M, K, N)
        c = torch.empty(M * N, device="cuda")
        be.GemmPackedB("bf16", be.WrapTensor(from_bits16(ab, torch.bfloat16)), packed, None, be.WrapTensor(c), M, N, K)
        assert np.array_equal(c.cpu().numpy().reshape(M, N), want32.reshape(M, N))
    with pytest.raises(NotSupportedException):
        be.PackB("int8", packed, K, N)
    with pytest.raises(NotSupportedException):
        be.PackB("bf16", be.WrapTensor(from_bits16(bb, torch.bfloat16)), K, N, transB=True)        # 16-bit B is [K,N] only
    small = be.AllocateByteBuffer(1024)
    with pytest.raises(Exception):
        be.GemmPackedB("bf16", be.WrapTensor(torch.zeros(4 * K, dtype=torch.bfloat16, device="cuda")), small, None,
                       be.WrapTensor(torch.zeros(4 * N, device="cuda")), 4, N, K)                     # packed buffer too small


def test_engine_cached_weight_matmul_repacks_a_changed_weight():
    from aidotnet.tensors_amd import Mi355Engine
    eng = Mi355Engine()
    g = torch.Generator(device="cuda").manual_seed(3)
    w = (torch.randint(-4, 5, (130, 1001), device="cuda", generator=g).float() / 8).bfloat16()
    x = (torch.randint(-4, 5, (3, 7, 130), device="cuda", generator=g).float() / 8).bfloat16()
    first = eng.TensorMatMulCachedB(x, w)
    assert first.shape == (3, 7, 1001) and first.dtype == torch.bfloat16
    assert torch.equal(first, eng.TensorMatMul(x, w))                       # the values of the plain product
    assert len(eng._packed_b) == 1
    packed_before = next(iter(eng._packed_b.values()))[3]
    again = eng.TensorMatMulCachedB(x, w)
    assert torch.equal(again, first) and next(iter(eng._packed_b.values()))[3] is packed_before     # packed once
    w.mul_(2)                                                               # in place: same storage, new version
    doubled = eng.TensorMatMulCachedB(x, w)
    assert torch.equal(doubled.float(), 2 * first.float())
    assert next(iter(eng._packed_b.values()))[3] is not packed_before
    xf = x.float(); wf = w.float()
    assert torch.equal(eng.TensorMatMulCachedB(xf, wf), eng.TensorMatMul(xf, wf))
    assert len(eng._packed_b) == 2
    with pytest.raises(Exception):
        eng.TensorMatMulCachedB(x, w.float())
    eng.backend.Dispose()
