"""Multi-head attention forward (QKV projection -> attention over the packed activation -> output projection).

Reference: CpuEngine.MultiHeadAttentionForward (src/AiDotNet.Tensors/Engines/CpuEngine.MultiHeadAttention.cs:68-285, 358-522).
Tolerances: mixed error <= 1e-4 (fp32) / 2e-2 (fp16, bf16) against the float64 closed form on the same rounded inputs.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import dev, mixed_err, round_to, from_bits16, bits16, TORCH16


def mha64(x, wq, wk, wv, wo, heads, keep=None):
    """Independent float64 restatement with numpy (not the oracle's code path)."""
    x = np.asarray(x, np.float64); B, S, dM = x.shape; d = dM // heads
    def split(w):
        return (x @ np.asarray(w, np.float64)).reshape(B, S, heads, d).transpose(0, 2, 1, 3)
    q, k, v = split(wq), split(wk), split(wv)
    s = np.einsum("bhid,bhjd->bhij", q, k) / math.sqrt(d)
    if keep is not None:
        s = np.where(np.broadcast_to(keep, s.shape), s, -np.inf)
    m = s.max(-1, keepdims=True); m = np.where(np.isfinite(m), m, 0.0)
    p = np.exp(s - m); z = p.sum(-1, keepdims=True)
    p = np.divide(p, z, out=np.zeros_like(p), where=z > 0)
    o = np.einsum("bhij,bhjd->bhid", p, v).transpose(0, 2, 1, 3).reshape(B, S, dM)
    return o @ np.asarray(wo, np.float64)


def _inputs(B, S, dM, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B, S, dM)).astype(np.float32)
    ws = [(rng.standard_normal((dM, dM)) / math.sqrt(dM)).astype(np.float32) for _ in range(4)]
    return x, ws


# ------------------------------------------------------------------------------------------------ oracle (CPU)
@pytest.mark.parametrize("B,S,dM,heads", [(1, 4, 8, 2), (2, 9, 24, 3), (3, 17, 32, 4), (2, 33, 64, 1)])
def test_oracle_mha_matches_float64(B, S, dM, heads):
    x, (wq, wk, wv, wo) = _inputs(B, S, dM, 10 + S)
    assert mixed_err(oracle.mha_forward(x, wq, wk, wv, wo, heads), mha64(x, wq, wk, wv, wo, heads)) <= 1e-5


def test_oracle_mha_mask_and_identity_projections():
    B, S, dM, heads = 2, 6, 8, 2
    x, (wq, wk, wv, wo) = _inputs(B, S, dM, 3)
    keep = np.tril(np.ones((S, S), bool))[None, None]
    assert mixed_err(oracle.mha_forward(x, wq, wk, wv, wo, heads, keep), mha64(x, wq, wk, wv, wo, heads, keep)) <= 1e-5
    # identity V and output projections, zero Q projection: every row is the mean of the input rows
    eye = np.eye(dM, dtype=np.float32); zero = np.zeros((dM, dM), np.float32)
    out = oracle.mha_forward(x, zero, wk, eye, eye, heads)
    assert np.max(np.abs(out - x.mean(axis=1, keepdims=True))) < 1e-5


# ------------------------------------------------------------------------------------------------ HIP path (GPU)
CASES = [(1, 4, 8, 2), (2, 9, 24, 3), (2, 64, 128, 4), (3, 100, 192, 6), (2, 128, 256, 2), (4, 512, 768, 12)]


@pytest.mark.gpu
@pytest.mark.parametrize("B,S,dM,heads", CASES)
def test_gpu_mha_fp32(B, S, dM, heads):
    from aidotnet.tensors_amd import Mi355Engine
    eng = Mi355Engine()
    x, (wq, wk, wv, wo) = _inputs(B, S, dM, 100 + S)
    out = eng.MultiHeadAttentionForward(dev(x), dev(wq), dev(wk), dev(wv), dev(wo), heads).cpu().numpy()
    assert out.shape == (B, S, dM)
    assert mixed_err(out, mha64(x, wq, wk, wv, wo, heads)) <= 1e-4
    if B * S * dM <= 1 << 16:
        assert mixed_err(out, oracle.mha_forward(x, wq, wk, wv, wo, heads)) <= 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("shared", [True, False])
def test_gpu_mha_fp32_boolean_mask(shared):
    from aidotnet.tensors_amd import Mi355Engine
    eng = Mi355Engine()
    B, S, dM, heads = 2, 40, 96, 3
    x, (wq, wk, wv, wo) = _inputs(B, S, dM, 7)
    rng = np.random.default_rng(8)
    keep = rng.random((1, 1, S, S) if shared else (B, heads, S, S)) > 0.3
    keep[..., 5, :] = False                                     # one fully masked query row: its attention output is zero
    out = eng.MultiHeadAttentionForward(dev(x), dev(wq), dev(wk), dev(wv), dev(wo), heads, torch.from_numpy(keep).cuda()).cpu().numpy()
    assert mixed_err(out, mha64(x, wq, wk, wv, wo, heads, keep)) <= 1e-4
    assert mixed_err(out, oracle.mha_forward(x, wq, wk, wv, wo, heads, keep)) <= 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("B,S,dM,heads", [(2, 64, 128, 4), (2, 256, 512, 4), (1, 100, 192, 3)])
def test_gpu_mha_half(kind, B, S, dM, heads):
    from aidotnet.tensors_amd import Mi355Engine
    eng = Mi355Engine()
    x, ws = _inputs(B, S, dM, 200 + S)
    xb, xr = round_to(x, kind)
    wb, wr = zip(*[round_to(w, kind) for w in ws])
    t = [from_bits16(b, TORCH16[kind]) for b in (xb,) + wb]
    out = eng.MultiHeadAttentionForward(t[0].reshape(B, S, dM), *[w.reshape(dM, dM) for w in t[1:]], heads)
    assert out.dtype == TORCH16[kind]
    widen = oracle.f16_to_f32 if kind == "f16" else oracle.bf16_to_f32
    got = widen(bits16(out)).reshape(B, S, dM)
    assert mixed_err(got, mha64(xr, *wr, heads)) <= 2e-2


@pytest.mark.gpu
def test_gpu_mha_argument_errors():
    from aidotnet.tensors_amd import Mi355Engine
    from aidotnet.tensors_amd.backend import ArgumentException, ArgumentNullException, ArgumentOutOfRangeException
    eng = Mi355Engine()
    x = torch.zeros(2, 4, 8, device="cuda"); w = torch.zeros(8, 8, device="cuda")
    with pytest.raises(ArgumentNullException):
        eng.MultiHeadAttentionForward(x, None, w, w, w, 2)
    with pytest.raises(ArgumentException):
        eng.MultiHeadAttentionForward(x[0], w, w, w, w, 2)
    with pytest.raises(ArgumentOutOfRangeException):
        eng.MultiHeadAttentionForward(x, w, w, w, w, 0)
    with pytest.raises(ArgumentException):
        eng.MultiHeadAttentionForward(x, w, w, w, w, 3)
    with pytest.raises(ArgumentException):
        eng.MultiHeadAttentionForward(x, w, w[:4], w, w, 2)
