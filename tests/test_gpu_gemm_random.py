"""Seeded random shapes through every GEMM kernel family (general 64 / 128 tiles in both loop forms, the 256 x 256 kernel with
and without ragged edges, the skinny and small-M split-K paths, transposed B, batched, alpha / beta) against the float64
product of the same stored inputs.  Bars: 1e-4 mixed error for fp32 inputs, 2e-2 for fp16 / bf16 outputs, 1e-4 for 16-bit inputs
with fp32 output (products of 16-bit values are exact in fp32, only the summation order differs)."""
import numpy as np
import pytest
import torch

from _util import TORCH16, bits16, dev, from_bits16, mixed_err, round_to
import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    b = Mi355Backend()
    yield b
    b.SetGemmTile(0)
    b.Dispose()


def shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        cls = rng.integers(0, 6)
        if cls == 0:      # anything small
            m, n, k = rng.integers(1, 200, 3)
        elif cls == 1:    # aligned N / K, ragged M: the branch-free loops with clamped rows
            m = rng.integers(1, 700); n = 8 * rng.integers(1, 90); k = 64 * rng.integers(1, 9)
        elif cls == 2:    # few rows, many columns: split-K streams
            m = rng.integers(1, 33); n = 128 * rng.integers(1, 24); k = 64 * rng.integers(1, 40)
        elif cls == 3:    # multiples of the large tiles
            m = 128 * rng.integers(1, 6); n = 128 * rng.integers(1, 6); k = 32 * rng.integers(1, 20)
        elif cls == 4:    # unaligned everything
            m = rng.integers(30, 400); n = rng.integers(30, 400) | 1; k = rng.integers(30, 400) | 1
        else:             # ragged M and N with K a multiple of 64, large enough for the 256 tile when forced
            m = rng.integers(200, 900); n = 8 * rng.integers(20, 120); k = 64 * rng.integers(1, 6)
        out.append((int(m), int(n), int(k)))
    return out


@pytest.mark.parametrize("tile", [0, 64, 128])
def test_random_fp32_gemm(be, tile):
    be.SetGemmTile(tile)
    try:
        rng = np.random.default_rng(100 + tile)
        for (m, n, k) in shapes(tile, 40):
            a = rng.uniform(-1, 1, (m, k)).astype(np.float32); b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
            c0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
            alpha, beta = (1.0, 0.0) if rng.integers(0, 2) else (float(rng.uniform(-2, 2)), float(rng.uniform(-2, 2)))
            trans = bool(rng.integers(0, 2))
            c = dev(c0.copy())
            bm = np.ascontiguousarray(b.T) if trans else b
            (be.MatMulTransposed if trans else be.Gemm)(be.WrapTensor(dev(a)), be.WrapTensor(dev(bm)), be.WrapTensor(c), m, n, k, alpha, beta)
            truth = alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0.astype(np.float64)
            assert mixed_err(c.cpu().numpy(), truth) <= 1e-4, (tile, m, n, k, alpha, beta, trans)
    finally:
        be.SetGemmTile(0)


@pytest.mark.parametrize("tile", [256, 129, 65])
def test_random_fp32_direct_kernel_alpha_beta_and_batches(be, tile):
    be.SetGemmTile(tile)
    try:
        rng = np.random.default_rng(400 + tile)
        for (m, n, k) in shapes(90 + tile, 24):
            if n % 4 or k % 4 or m % 4:                     # batch strides m*k, k*n must keep 16-byte alignment
                continue
            batch = int(rng.integers(1, 5))
            a = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32); b = rng.uniform(-1, 1, (batch, k, n)).astype(np.float32)
            c0 = rng.uniform(-1, 1, (batch, m, n)).astype(np.float32)
            alpha, beta = float(rng.uniform(-2, 2)), float(rng.uniform(-2, 2))
            c = dev(c0.copy())
            be.BatchedGemm(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(c), m, n, k, batch, alpha, beta)
            truth = alpha * np.einsum("bmk,bkn->bmn", a.astype(np.float64), b.astype(np.float64)) + beta * c0.astype(np.float64)
            assert mixed_err(c.cpu().numpy(), truth) <= 1e-4, (tile, m, n, k, batch, alpha, beta)
    finally:
        be.SetGemmTile(0)


@pytest.mark.parametrize("tile", [256, 129, 65])
def test_random_fp32_gemm_direct_kernel(be, tile):
    be.SetGemmTile(tile)
    try:
        rng = np.random.default_rng(300 + tile)
        for (m, n, k) in shapes(70 + tile, 40):
            if n % 4 or k % 4:
                continue                                     # rows must be whole 16-byte chunks for this kernel
            a = rng.uniform(-1, 1, (m, k)).astype(np.float32); b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
            c = torch.full((m, n), float("nan"), device="cuda")
            be.Gemm(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(c), m, n, k, 1.0, 0.0)
            assert mixed_err(c.cpu().numpy(), a.astype(np.float64) @ b.astype(np.float64)) <= 1e-4, (tile, m, n, k)
            c = torch.full((m, n), float("nan"), device="cuda")
            be.MatMulTransposed(be.WrapTensor(dev(a)), be.WrapTensor(dev(np.ascontiguousarray(b.T))), be.WrapTensor(c), m, n, k, 1.0, 0.0)
            assert mixed_err(c.cpu().numpy(), a.astype(np.float64) @ b.astype(np.float64)) <= 1e-4, ("transposed", tile, m, n, k)
    finally:
        be.SetGemmTile(0)


def test_random_fp32_batched_gemm(be):
    rng = np.random.default_rng(5)
    for (m, n, k) in shapes(9, 12):
        batch = int(rng.integers(1, 7))
        a = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32); b = rng.uniform(-1, 1, (batch, k, n)).astype(np.float32)
        c = torch.full((batch, m, n), float("nan"), device="cuda")
        be.BatchedGemm(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(c), m, n, k, batch)
        truth = np.einsum("bmk,bkn->bmn", a.astype(np.float64), b.astype(np.float64))
        assert mixed_err(c.cpu().numpy(), truth) <= 1e-4, (m, n, k, batch)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("tile", [0, 64, 65, 128, 129, 256])
def test_random_half_gemm(be, kind, tile):
    from aidotnet.tensors_amd import HipException
    be.SetGemmTile(tile)
    try:
        rng = np.random.default_rng(200 + tile)
        for (m, n, k) in shapes(50 + tile, 30):
            if tile in (65, 129, 256) and (k % 8 or n % 8):
                continue                                     # outside the large-tile kernel's contract (refused, tested elsewhere)
            a = rng.uniform(-1, 1, (m, k)).astype(np.float32); b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
            ab, aw = round_to(a, kind); bb, bw = round_to(b, kind)
            truth = aw.astype(np.float64) @ bw.astype(np.float64)
            A = be.WrapTensor(from_bits16(ab, TORCH16[kind])); B = be.WrapTensor(from_bits16(bb, TORCH16[kind]))
            c32 = torch.full((m, n), float("nan"), device="cuda")
            (be.GemmFp16In32fOut if kind == "f16" else be.GemmBf16In32fOut)(A, B, be.WrapTensor(c32), m, n, k)
            assert mixed_err(c32.cpu().numpy(), truth) <= 1e-4, (kind, tile, m, n, k)
            c16 = torch.zeros((m, n), dtype=TORCH16[kind], device="cuda")
            (be.Hgemm if kind == "f16" else be.Bf16Gemm)(A, B, be.WrapTensor(c16), m, n, k)
            got = (oracle.f16_to_f32 if kind == "f16" else oracle.bf16_to_f32)(bits16(c16)).reshape(m, n)
            assert mixed_err(got, truth) <= 2e-2, (kind, tile, m, n, k)
    finally:
        be.SetGemmTile(0)


def test_random_fp16_weight_and_epilogue(be):
    rng = np.random.default_rng(77)
    for (m, n, k) in shapes(31, 30):
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32); b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        bias = rng.uniform(-1, 1, n).astype(np.float32)
        bb, bw = round_to(b, "f16")
        c = torch.full((m * n,), float("nan"), device="cuda")
        be.GemmFp16WeightB(be.WrapTensor(dev(a)), be.WrapTensor(from_bits16(bb, torch.float16)), be.WrapTensor(dev(bias)), be.WrapTensor(c), m, n, k, 1)
        truth = np.maximum(a.astype(np.float64) @ bw.astype(np.float64) + bias[None, :], 0.0)
        assert mixed_err(c.cpu().numpy().reshape(m, n), truth) <= 1e-4, (m, n, k)
        c2 = torch.full((m * n,), float("nan"), device="cuda")
        be.GemmBiasActivationInto(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(dev(bias)), be.WrapTensor(c2), m, n, k, 4)
        truth = np.tanh(a.astype(np.float64) @ b.astype(np.float64) + bias[None, :])
        assert mixed_err(c2.cpu().numpy().reshape(m, n), truth) <= 1e-4, (m, n, k)


def _offset_view(x: np.ndarray, elems: int, dtype=None) -> torch.Tensor:
    """Device copy of x whose first element sits `elems` elements past a 256-byte aligned allocation."""
    flat = torch.from_numpy(np.ascontiguousarray(x).reshape(-1))
    if dtype is not None:
        flat = flat.view(dtype)
    buf = torch.zeros(flat.numel() + elems, dtype=flat.dtype, device="cuda")
    buf[elems:] = flat.cuda()
    return buf[elems:]


# The workspace of a GEMM call is sized from the dimensions alone, while the plan that runs also depends on the alignment of the
# operands: a sub-view pointer passes over the padded-copy / streamed-weight plans and lands on a later one, which must then find
# its own partials inside the bytes it was handed (or pass as well).  Results against float64, and a guard band behind C.
@pytest.mark.parametrize("off_a,off_b", [(1, 0), (0, 1), (1, 1), (3, 2)])
def test_fp32_gemm_with_sub_view_pointers_stays_inside_its_workspace(be, off_a, off_b):
    be.SetGemmTile(0)
    rng = np.random.default_rng(7 + off_a * 4 + off_b)
    for (m, n, k) in [(16, 256, 4096), (24, 1024, 2048), (128, 256, 4096), (8, 512, 1024), (32, 4096, 4096), (100, 130, 4100), (512, 768, 3072)]:
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32); b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        c = torch.full((m * n + 64,), 7.0, device="cuda")
        be.Gemm(be.WrapTensor(_offset_view(a, off_a)), be.WrapTensor(_offset_view(b, off_b)), be.WrapTensor(c), m, n, k)
        got = c.cpu().numpy()
        assert np.all(got[m * n:] == 7.0), (m, n, k)
        assert mixed_err(got[:m * n].reshape(m, n), a.astype(np.float64) @ b.astype(np.float64)) <= 1e-4, (m, n, k, off_a, off_b)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("off_a,off_b", [(1, 0), (0, 1), (4, 4), (3, 5)])
def test_16bit_gemm_with_sub_view_pointers_stays_inside_its_workspace(be, kind, off_a, off_b):
    be.SetGemmTile(0)
    rng = np.random.default_rng(11 + off_a * 8 + off_b)
    for (m, n, k) in [(16, 4096, 4096), (32, 1024, 2048), (256, 4096, 4096), (128, 4096, 4096), (1000, 768, 3072), (100, 130, 4100), (300, 1001, 520)]:
        abits, a = round_to(rng.standard_normal((m, k)).astype(np.float32), kind)
        bbits, b = round_to((0.05 * rng.standard_normal((k, n))).astype(np.float32), kind)
        c = torch.full((m * n + 64,), 7.0, device="cuda")
        A = _offset_view(abits.view(np.int16), off_a, torch.int16).view(TORCH16[kind])
        B = _offset_view(bbits.view(np.int16), off_b, torch.int16).view(TORCH16[kind])
        (be.GemmFp16In32fOut if kind == "f16" else be.GemmBf16In32fOut)(be.WrapTensor(A), be.WrapTensor(B), be.WrapTensor(c), m, n, k)
        got = c.cpu().numpy()
        assert np.all(got[m * n:] == 7.0), (m, n, k)
        assert mixed_err(got[:m * n].reshape(m, n), a.astype(np.float64) @ b.astype(np.float64)) <= 1e-4, (kind, m, n, k, off_a, off_b)
