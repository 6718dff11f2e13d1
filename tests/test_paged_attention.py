"""Attention over a paged K/V cache (block-table gather): decode, causal prefill, GQA.

Reference: IDirectGpuBackend.PagedAttentionDecode[Gqa] / PagedAttentionPrefill[Gqa]
(src/AiDotNet.Tensors/Engines/DirectGpu/IDirectGpuBackend.cs:3614-3633; kernels HIP/Kernels/HipPagedAttentionKernels.cs).
Tolerances: mixed error <= 1e-4 (fp32) / 2e-2 (fp16, bf16) against float64 on the same rounded inputs.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import dev, mixed_err, round_to, from_bits16, TORCH16


def make_cache(rng, key_len, block_size, kv_heads, d, extra_blocks=3):
    """Logical K/V [keyLen, kvHeads, d] scattered into a shuffled pool; returns (k, v, kpool, vpool, table)."""
    nblk = (key_len + block_size - 1) // block_size
    pool_blocks = nblk + extra_blocks
    table = rng.permutation(pool_blocks)[:nblk].astype(np.int32)
    k = rng.standard_normal((key_len, kv_heads, d)).astype(np.float32); v = rng.standard_normal((key_len, kv_heads, d)).astype(np.float32)
    kp = rng.standard_normal((pool_blocks, block_size, kv_heads, d)).astype(np.float32) * 50     # poison in unused slots
    vp = rng.standard_normal((pool_blocks, block_size, kv_heads, d)).astype(np.float32) * 50
    t = np.arange(key_len)
    kp[table[t // block_size], t % block_size] = k
    vp[table[t // block_size], t % block_size] = v
    return k, v, kp, vp, table


def paged64(q, k, v, heads, kv_heads, start_pos, scale):
    """Independent float64 closed form on the logical (gathered) K/V."""
    nq, _, d = q.shape
    out = np.zeros((nq, heads, d))
    for h in range(heads):
        kh = k[:, h // (heads // kv_heads)].astype(np.float64); vh = v[:, h // (heads // kv_heads)].astype(np.float64)
        for i in range(nq):
            n = start_pos + i + 1
            s = kh[:n] @ q[i, h].astype(np.float64) * scale
            p = np.exp(s - s.max()); p /= p.sum()
            out[i, h] = p @ vh[:n]
    return out


# ------------------------------------------------------------------------------------------------ oracle (CPU)
@pytest.mark.parametrize("heads,kv,d,bs,nq,start", [(4, 4, 16, 4, 1, 9), (8, 2, 32, 16, 1, 40), (4, 4, 8, 3, 5, 0), (6, 3, 20, 7, 9, 13)])
def test_oracle_paged_attention_matches_float64(heads, kv, d, bs, nq, start):
    rng = np.random.default_rng(heads + d + nq)
    k, v, kp, vp, table = make_cache(rng, start + nq, bs, kv, d)
    q = rng.standard_normal((nq, heads, d)).astype(np.float32)
    got = oracle.paged_attention(q, kp, vp, table, heads, kv, d, bs, nq, start, 1 / math.sqrt(d))
    assert mixed_err(got, paged64(q, k, v, heads, kv, start, 1 / math.sqrt(d))) <= 1e-5


def test_oracle_paged_decode_equals_contiguous_decode_oracle():
    rng = np.random.default_rng(1)
    heads, kv, d, bs, seq = 8, 2, 64, 16, 50
    k, v, kp, vp, table = make_cache(rng, seq, bs, kv, d)
    q = rng.standard_normal((1, heads, d)).astype(np.float32)
    a = oracle.paged_attention(q, kp, vp, table, heads, kv, d, bs, 1, seq - 1, 0.125)[0]
    b = oracle.decode_f32(q[0], k, v, heads, kv, d, seq, 0.125)
    assert mixed_err(a, b) <= 1e-6


# ------------------------------------------------------------------------------------------------ HIP path (GPU)
@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    return Mi355Backend()


DECODE = [(4, 4, 64, 16, 40), (8, 8, 32, 8, 100), (4, 4, 64, 16, 7), (6, 6, 48, 5, 77), (8, 2, 64, 16, 50), (8, 1, 64, 32, 40),
          (32, 8, 128, 16, 1000), (16, 16, 128, 64, 4096)]


@pytest.mark.gpu
@pytest.mark.parametrize("heads,kv,d,bs,seq", DECODE)
def test_gpu_paged_decode_fp32(be, heads, kv, d, bs, seq):
    rng = np.random.default_rng(heads + seq)
    k, v, kp, vp, table = make_cache(rng, seq, bs, kv, d)
    q = rng.standard_normal((1, heads, d)).astype(np.float32)
    W = be.WrapTensor
    args = (W(dev(q.ravel())), W(dev(kp.ravel())), W(dev(vp.ravel())), W(torch.from_numpy(table).cuda()))
    scale = 1 / math.sqrt(d)
    out = be.PagedAttentionDecodeGqa(*args, heads, kv, d, bs, seq, scale) if kv != heads else be.PagedAttentionDecode(*args, heads, d, bs, seq, scale)
    got = be.DownloadBuffer(out).numpy().reshape(1, heads, d)
    assert mixed_err(got, paged64(q, k, v, heads, kv, seq - 1, scale)) <= 1e-4
    if seq <= 1000:
        assert mixed_err(got, oracle.paged_attention(q, kp, vp, table, heads, kv, d, bs, 1, seq - 1, scale)) <= 1e-4


PREFILL = [(4, 4, 64, 16, 8, 0), (4, 4, 64, 16, 5, 11), (8, 2, 32, 8, 33, 20), (6, 3, 48, 7, 70, 3), (8, 8, 128, 16, 200, 56)]


@pytest.mark.gpu
@pytest.mark.parametrize("heads,kv,d,bs,nq,start", PREFILL)
def test_gpu_paged_prefill_fp32(be, heads, kv, d, bs, nq, start):
    rng = np.random.default_rng(heads + nq + start)
    k, v, kp, vp, table = make_cache(rng, start + nq, bs, kv, d)
    q = rng.standard_normal((nq, heads, d)).astype(np.float32)
    W = be.WrapTensor
    args = (W(dev(q.ravel())), W(dev(kp.ravel())), W(dev(vp.ravel())), W(torch.from_numpy(table).cuda()))
    scale = 1 / math.sqrt(d)
    out = (be.PagedAttentionPrefillGqa(*args, heads, kv, d, bs, nq, start, scale) if kv != heads
           else be.PagedAttentionPrefill(*args, heads, d, bs, nq, start, scale))
    got = be.DownloadBuffer(out).numpy().reshape(nq, heads, d)
    assert mixed_err(got, paged64(q, k, v, heads, kv, start, scale)) <= 1e-4
    assert mixed_err(got, oracle.paged_attention(q, kp, vp, table, heads, kv, d, bs, nq, start, scale)) <= 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("heads,kv,d,bs,nq,start", [(32, 8, 128, 16, 1, 2047), (8, 8, 128, 32, 1, 300), (8, 2, 64, 16, 24, 40)])
def test_gpu_paged_half(be, kind, heads, kv, d, bs, nq, start):
    rng = np.random.default_rng(heads + nq + start)
    k, v, kp, vp, table = make_cache(rng, start + nq, bs, kv, d)
    q = rng.standard_normal((nq, heads, d)).astype(np.float32)
    qb, qr = round_to(q, kind); kb, kr = round_to(kp, kind); vb, vr = round_to(vp, kind)
    _, klr = round_to(k, kind); _, vlr = round_to(v, kind)
    W = be.WrapTensor; T = TORCH16[kind]
    out = be.PagedAttentionHalf(kind, W(from_bits16(qb.ravel(), T)), W(from_bits16(kb.ravel(), T)), W(from_bits16(vb.ravel(), T)),
                                W(torch.from_numpy(table).cuda()), heads, kv, d, bs, nq, start, 1 / math.sqrt(d))
    got = be.DownloadBuffer(out).numpy().reshape(nq, heads, d)
    assert mixed_err(got, paged64(qr, klr, vlr, heads, kv, start, 1 / math.sqrt(d))) <= 2e-2


@pytest.mark.gpu
def test_gpu_paged_guards(be):
    from aidotnet.tensors_amd.backend import ArgumentException, ArgumentOutOfRangeException
    W = be.WrapTensor
    q = W(torch.zeros(4 * 16, device="cuda")); pool = W(torch.zeros(3 * 4 * 4 * 16, device="cuda"))
    bt = W(torch.tensor([0, 1, 2], dtype=torch.int32, device="cuda"))
    with pytest.raises(ArgumentOutOfRangeException):
        be.PagedAttentionDecode(q, pool, pool, bt, 0, 16, 4, 8, 1.0)
    with pytest.raises(ArgumentOutOfRangeException):
        be.PagedAttentionDecode(q, pool, pool, bt, 4, 300, 4, 8, 1.0)
    with pytest.raises(ArgumentOutOfRangeException):
        be.PagedAttentionDecodeGqa(q, pool, pool, bt, 4, 3, 16, 4, 8, 1.0)
    with pytest.raises(ArgumentException):
        be.PagedAttentionDecode(q, pool, pool, bt, 4, 16, 4, 100, 1.0)          # block table too short
    with pytest.raises(ArgumentException):
        be.PagedAttentionDecode(q, pool, W(torch.zeros(5, device="cuda")), bt, 4, 16, 4, 8, 1.0)
    bad = W(torch.tensor([0, 7, 2], dtype=torch.int32, device="cuda"))
    assert be.ValidateBlockTables is None   # the content check runs by default whenever the stream is not being captured
    with pytest.raises(ArgumentException):
        be.PagedAttentionDecode(q, pool, pool, bad, 4, 16, 4, 12, 1.0)          # block id outside the pool
