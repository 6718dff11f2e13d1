"""Interleaved rotary position embedding.  Reference: IDirectGpuBackend.RopeInterleaved
(src/AiDotNet.Tensors/Engines/DirectGpu/IDirectGpuBackend.cs:1427-1446; kernel HIP/Kernels/HipAttentionKernels.cs:958-989).
Tolerances: 1e-4 mixed error for fp32 (the kernel may contract multiply-adds), one 16-bit rounding for fp16 / bf16."""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import dev, mixed_err, round_to, from_bits16, bits16, TORCH16


def caches(max_seq, hd, base=10000.0):
    inv = base ** (-np.arange(hd // 2, dtype=np.float64) * 2 / hd)
    ang = np.arange(max_seq, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def rope64(x, cos, sin, seq_len, start):
    x = np.asarray(x, np.float64); rows, hd = x.shape
    pos = start + np.arange(rows) % seq_len
    z = (x[:, 0::2] + 1j * x[:, 1::2]) * (cos[pos].astype(np.float64) + 1j * sin[pos].astype(np.float64))    # rotation as complex multiply
    out = np.empty_like(x); out[:, 0::2] = z.real; out[:, 1::2] = z.imag
    return out


def test_oracle_rope_matches_complex_rotation_and_preserves_norm():
    rng = np.random.default_rng(0)
    hd, seq, lead, start = 16, 7, 3, 5
    cos, sin = caches(start + seq, hd)
    x = rng.standard_normal((lead * seq, hd)).astype(np.float32)
    got = oracle.rope_interleaved(x, cos, sin, seq, start)
    assert mixed_err(got, rope64(x, cos, sin, seq, start)) <= 1e-6
    assert np.allclose(np.linalg.norm(got, axis=1), np.linalg.norm(x, axis=1), rtol=1e-5)
    # position 0 is the identity
    c0, s0 = caches(4, hd)
    assert np.array_equal(oracle.rope_interleaved(x[:1], c0, s0, 1, 0), x[:1])


@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    return Mi355Backend()


@pytest.mark.gpu
@pytest.mark.parametrize("lead,seq,hd,start", [(1, 1, 2, 0), (3, 7, 16, 5), (8, 128, 64, 0), (32, 1, 128, 4095), (4, 333, 96, 17)])
def test_gpu_rope_fp32(be, lead, seq, hd, start):
    rng = np.random.default_rng(lead + seq + hd)
    cos, sin = caches(start + seq, hd)
    x = rng.standard_normal((lead * seq, hd)).astype(np.float32)
    xin = dev(x.ravel()); out = torch.full_like(xin, 3e30)
    W = be.WrapTensor
    be.RopeInterleaved(W(xin), W(dev(cos.ravel())), W(dev(sin.ravel())), W(out), lead * seq, hd, seq, start)
    got = out.cpu().numpy().reshape(lead * seq, hd)
    assert mixed_err(got, rope64(x, cos, sin, seq, start)) <= 1e-6
    assert mixed_err(got, oracle.rope_interleaved(x, cos, sin, seq, start)) <= 1e-6
    be.RopeInterleaved(W(xin), W(dev(cos.ravel())), W(dev(sin.ravel())), W(xin), lead * seq, hd, seq, start)      # in place
    assert np.array_equal(xin.cpu().numpy().reshape(lead * seq, hd), got)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_gpu_rope_half(be, kind):
    rng = np.random.default_rng(4)
    lead, seq, hd, start = 6, 50, 128, 9
    cos, sin = caches(start + seq, hd)
    x = rng.standard_normal((lead * seq, hd)).astype(np.float32)
    xb, xr = round_to(x, kind)
    T = TORCH16[kind]; W = be.WrapTensor
    out = torch.empty(lead * seq * hd, device="cuda", dtype=T)
    be.RopeInterleaved(W(from_bits16(xb.ravel(), T)), W(dev(cos.ravel())), W(dev(sin.ravel())), W(out), lead * seq, hd, seq, start, kind)
    widen = oracle.f16_to_f32 if kind == "f16" else oracle.bf16_to_f32
    got = widen(bits16(out)).reshape(lead * seq, hd)
    tol = 2 ** -10 if kind == "f16" else 2 ** -7
    assert mixed_err(got, rope64(xr, cos, sin, seq, start)) <= tol


@pytest.mark.gpu
def test_gpu_rope_guards(be):
    from aidotnet.tensors_amd.backend import ArgumentException, ArgumentOutOfRangeException
    W = be.WrapTensor
    x = W(torch.zeros(64, device="cuda")); c = W(torch.zeros(64, device="cuda"))
    with pytest.raises(ArgumentOutOfRangeException):
        be.RopeInterleaved(x, c, c, x, 0, 8, 4, 0)
    with pytest.raises(ArgumentException):
        be.RopeInterleaved(x, c, c, x, 4, 7, 4, 0)
    with pytest.raises(ArgumentException):
        be.RopeInterleaved(x, c, c, x, 16, 8, 4, 0)            # buffers smaller than rows * headDim
    with pytest.raises(ArgumentException):
        be.RopeInterleaved(x, c, c, x, 8, 8, 8, 100)           # caches shorter than the positions used
