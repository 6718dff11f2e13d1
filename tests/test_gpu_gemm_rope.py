"""Projection + rotary embedding in one call (aidn_mi355_hgemm_rope / aidn_mi355_bf16gemm_rope) against the two calls it replaces
and against the oracle's product followed by the interleaved rotation in float64."""
import numpy as np
import pytest
import torch

from _util import TORCH16, from_bits16, round_to

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    return Mi355Backend()


def _caches(maxseq, D):
    half = D // 2
    ang = np.arange(maxseq, dtype=np.float64)[:, None] * (10000.0 ** (-np.arange(half, dtype=np.float64) * 2.0 / D))[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def _rope64(c, cos, sin, D, cols, seq_len, start):
    out = c.astype(np.float64).copy()
    M = c.shape[0]
    pos = start + np.arange(M) % seq_len
    for h0 in range(0, cols, D):
        xe, xo = out[:, h0:h0 + D:2].copy(), out[:, h0 + 1:h0 + D:2].copy()
        cc, ss = cos[pos].astype(np.float64), sin[pos].astype(np.float64)
        out[:, h0:h0 + D:2] = xe * cc - xo * ss
        out[:, h0 + 1:h0 + D:2] = xe * ss + xo * cc
    return out


# (M, N, K, head_dim, rope_cols, seq_len, start): decode-step shapes (the summing pass carries the rotation), a concatenated
# [Wq|Wk|Wv] projection rotated over Q and K only, prefill rows (position = start + row % seq_len), and shapes that take a tiled
# kernel and rotate in a second launch
CASES = [
    (4, 2048, 2048, 128, 2048, 1, 1023),
    (32, 6144, 4096, 128, 4096 + 1024, 1, 4095),
    (32, 12288, 4096, 128, 8192, 1, 17),
    (16, 1024, 512, 64, 1024, 8, 5),
    (300, 768, 256, 64, 512, 100, 3),
    (512, 1024, 1024, 128, 1024, 256, 0),
    (7, 130, 96, 26, 104, 7, 2),
]


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,D,cols,seq_len,start", CASES)
def test_gemm_rope_matches_product_then_rotation(be, kind, M, N, K, D, cols, seq_len, start):
    rng = np.random.default_rng(M + 3 * N + 5 * K + len(kind))
    a = rng.standard_normal((M, K)).astype(np.float32); b = (0.05 * rng.standard_normal((K, N))).astype(np.float32)
    (ab, aw), (bb, bw) = round_to(a, kind), round_to(b, kind)
    cos, sin = _caches(start + seq_len, D)
    dt = TORCH16[kind]
    W = be.WrapTensor
    A, B = from_bits16(ab, dt), from_bits16(bb, dt)
    cs, sn = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    fused = torch.zeros(M, N, dtype=dt, device="cuda")
    be.GemmRope(kind, W(A), W(B), W(fused), M, N, K, W(cs), W(sn), D, cols, seq_len, start)
    # the two calls it replaces: same values, rounding included (the rotation kernel works on dense [rows, head_dim] rows, so the
    # rotated columns are taken out, rotated and put back)
    plain = torch.zeros(M, N, dtype=dt, device="cuda")
    (be.Hgemm if kind == "f16" else be.Bf16Gemm)(W(A), W(B), W(plain), M, N, K)
    want = plain.clone()
    if M % seq_len == 0:
        part = plain[:, :cols].reshape(M, cols // D, D).permute(1, 0, 2).contiguous()       # [heads, M, D]: row % seq_len is the position
        be.RopeInterleaved(W(part), W(cs), W(sn), W(part), (cols // D) * M, D, seq_len, start, kind)
        want[:, :cols] = part.permute(1, 0, 2).reshape(M, cols)
        assert torch.equal(fused, want)
    # and the float64 product of the rounded inputs, rotated in float64 (16-bit tolerance of the metric: 2e-2 relative)
    ref = _rope64(aw.astype(np.float64) @ bw.astype(np.float64), cos, sin, D, cols, seq_len, start)
    got = fused.float().cpu().numpy().astype(np.float64)
    scale = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 2e-2 * scale
    # columns past rope_cols are the plain product
    assert torch.equal(fused[:, cols:], plain[:, cols:])


def test_gemm_rope_exact_on_dyadic_inputs(be):
    # small integers and a quarter-turn table: every product, sum and rotation is exact, so the fused call, the two separate calls
    # and integer arithmetic agree to the bit
    M, N, K, D = 8, 256, 128, 64
    rng = np.random.default_rng(3)
    a = rng.integers(-2, 3, (M, K)).astype(np.float64); b = rng.integers(-2, 3, (K, N)).astype(np.float64)
    quarter = rng.integers(0, 4, (4, D // 2))
    cos = np.array([1, 0, -1, 0], dtype=np.float32)[quarter]; sin = np.array([0, 1, 0, -1], dtype=np.float32)[quarter]
    for kind in ("f16", "bf16"):
        dt = TORCH16[kind]
        W = be.WrapTensor
        A = torch.from_numpy(a).to(dt).cuda(); B = torch.from_numpy(b).to(dt).cuda()
        cs, sn = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
        fused = torch.zeros(M, N, dtype=dt, device="cuda")
        be.GemmRope(kind, W(A), W(B), W(fused), M, N, K, W(cs), W(sn), D, N, 4, 0)
        ref = _rope64(a @ b, cos, sin, D, N, 4, 0)
        assert np.array_equal(fused.float().cpu().numpy().astype(np.float64), ref)


def test_gemm_rope_argument_checks(be):
    from aidotnet.tensors_amd.backend import ArgumentException
    W = be.WrapTensor
    A = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda"); B = torch.zeros(64, 128, dtype=torch.bfloat16, device="cuda")
    C = torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda"); cs = torch.zeros(8, 16, device="cuda")
    with pytest.raises(ArgumentException):
        be.GemmRope("bf16", W(A), W(B), W(C), 4, 128, 64, W(cs), W(cs), 32, 48, 1, 0)        # rope_cols not a multiple of head_dim
    with pytest.raises(ArgumentException):
        be.GemmRope("bf16", W(A), W(B), W(C), 4, 128, 64, W(cs), W(cs), 32, 128, 1, 100)     # caches too short
