"""CPU oracle: ctypes/numpy front end of ``liboracle.so``.

TEST INFRASTRUCTURE ONLY.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` import this package; the shipped library
(``aidotnet.tensors_amd``) never does.  Each C function cites the reference
file:line it restates in its own source comment.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_i32p = ctypes.POINTER(ctypes.c_int)


def build(force: bool = False) -> str:
    """Compile ``liboracle.so`` with the Makefile beside this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_bf16_from_float.argtypes = [ctypes.c_float]
        L.orc_bf16_from_float.restype = ctypes.c_uint16
        L.orc_bf16_to_float.argtypes = [ctypes.c_uint16]
        L.orc_bf16_to_float.restype = ctypes.c_float
        L.orc_f16_from_float.argtypes = [ctypes.c_float]
        L.orc_f16_from_float.restype = ctypes.c_uint16
        L.orc_f16_to_float.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_float.restype = ctypes.c_float
        L.orc_hash_uniform.argtypes = [ctypes.c_uint32]
        L.orc_hash_uniform.restype = ctypes.c_float
        L.orc_max_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a: np.ndarray, typ):
    return a.ctypes.data_as(typ)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def max_threads() -> int:
    return int(lib().orc_max_threads())


# ----------------------------------------------------------------- conversions
def f32_to_bf16(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_convert_f32_to_bf16(_p(x, _f32p), _p(out, _u16p), ctypes.c_long(x.size))
    return out


def bf16_to_f32(x) -> np.ndarray:
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib().orc_convert_bf16_to_f32(_p(x, _u16p), _p(out, _f32p), ctypes.c_long(x.size))
    return out


def f32_to_f16(x) -> np.ndarray:
    """float32 -> IEEE binary16 bit patterns (uint16)."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_convert_f32_to_f16(_p(x, _f32p), _p(out, _u16p), ctypes.c_long(x.size))
    return out


def f16_to_f32(x) -> np.ndarray:
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib().orc_convert_f16_to_f32(_p(x, _u16p), _p(out, _f32p), ctypes.c_long(x.size))
    return out


def hash_uniform(n: int, seed: int = 0) -> np.ndarray:
    """The reference test-suite's portable PCG-style hash generator, values in [-0.5, 0.5]."""
    out = np.empty(int(n), np.float32)
    lib().orc_fill_hash_uniform(_p(out, _f32p), ctypes.c_long(int(n)), ctypes.c_uint32(seed & 0xFFFFFFFF))
    return out


# ------------------------------------------------------------------------ GEMM
def sgemm(a, b, m: int, k: int, n: int, threads: int = 1) -> np.ndarray:
    """``SimdGemm.Sgemm(a, b, c, m, k, n)``: C[m,n] = A[m,k] * B[k,n], overwrite."""
    a = _c(a, np.float32); b = _c(b, np.float32)
    assert a.size >= m * k and b.size >= k * n
    c = np.full((max(m, 0), max(n, 0)), np.nan, np.float32)
    lib().orc_sgemm(_p(a, _f32p), _p(b, _f32p), _p(c, _f32p), m, k, n, threads)
    return c


def sgemm_ex(a, lda, trans_a, b, ldb, trans_b, m, k, n, threads: int = 1) -> np.ndarray:
    a = _c(a, np.float32); b = _c(b, np.float32)
    c = np.full((m, n), np.nan, np.float32)
    lib().orc_sgemm_ex(_p(a, _f32p), lda, int(trans_a), _p(b, _f32p), ldb, int(trans_b),
                       _p(c, _f32p), m, k, n, threads)
    return c


def gemm_alpha_beta(a, b, c, m, n, k, alpha=1.0, beta=0.0, trans_b=False, threads: int = 1) -> np.ndarray:
    """Backend contract ``C = alpha*A*B + beta*C`` (argument order M, N, K). Returns the new C."""
    a = _c(a, np.float32); b = _c(b, np.float32)
    c = np.array(c, dtype=np.float32, copy=True).reshape(m, n)
    lib().orc_gemm_alpha_beta(_p(a, _f32p), _p(b, _f32p), _p(c, _f32p), m, n, k,
                              ctypes.c_float(alpha), ctypes.c_float(beta), int(trans_b), threads)
    return c


def sgemm_fp16_weight_b(a, b_bits, m: int, k: int, n: int, threads: int = 1) -> np.ndarray:
    """``SimdGemm.SgemmFp16WeightB`` (src/AiDotNet.Tensors/Engines/Simd/SimdGemm.Fp16Weight.cs:22-91): fp32 A times fp16
    weights (bit patterns) -> fp32.  The reference widens the weights exactly while packing B (``PackBFromHalf``, :208-261) and
    then runs the ordinary fp32 macro-kernel, so the value is the restated SimdGemm on the widened weights."""
    return sgemm(a, f16_to_f32(np.asarray(b_bits, np.uint16)).reshape(k, n), m, k, n, threads)


def sgemm_small_m(a, b, m: int, k: int, n: int, c0=None) -> np.ndarray:
    """``SimdGemm.SgemmNParallelSmallM`` (src/AiDotNet.Tensors/Engines/Simd/SimdGemm.NParallelSmallM.cs:31-85): the m <= 8 GEMM that
    splits the output columns among workers; ``c0`` None = overwrite (``clearedOutput``), else accumulate into a copy of it.
    ``SgemmConcatenatedProjections`` (:95-109) is this call on the concatenated weight."""
    a = _c(a, np.float32); b = _c(b, np.float32)
    assert a.size == m * k and b.size == k * n
    c = np.zeros((m, n), np.float32) if c0 is None else np.array(c0, np.float32).reshape(m, n).copy()
    lib().orc_sgemm_small_m(_p(a, _f32p), k, _p(b, _f32p), n, _p(c, _f32p), m, k, n, 1 if c0 is None else 0)
    return c


def bias_activation(c, bias, act: int = 0, param: float = 0.0) -> np.ndarray:
    """The FusedLinear epilogue act(c + bias) on a [M, N] fp32 matrix (bias [N] or None); returns a new array."""
    out = np.array(c, np.float32, copy=True, order="C")
    m, n = out.shape
    b = _c(bias, np.float32) if bias is not None else None
    lib().orc_bias_act_f32(_p(out, _f32p), _p(b, _f32p) if b is not None else None, ctypes.c_long(m), ctypes.c_long(n),
                           int(act), ctypes.c_float(param))
    return out


def gemm_f64(a, b, m, k, n, trans_b=False, threads: int = 0) -> np.ndarray:
    a = _c(a, np.float32); b = _c(b, np.float32)
    c = np.empty((m, n), np.float64)
    lib().orc_gemm_f64(_p(a, _f32p), _p(b, _f32p), _p(c, _f64p), m, k, n, int(trans_b),
                       threads or max_threads())
    return c


def _gemm16(fn, a, b, m, k, n, threads):
    a = _c(a, np.uint16); b = _c(b, np.uint16)
    assert a.size >= m * k and b.size >= k * n
    o16 = np.empty((m, n), np.uint16)
    o32 = np.empty((m, n), np.float32)
    fn(_p(a, _u16p), k, _p(b, _u16p), n, _p(o16, _u16p), _p(o32, _f32p), n, m, k, n,
       threads or max_threads())
    return o16, o32


def hgemm(a_bits, b_bits, m, k, n, threads: int = 0):
    """``HalfKernels.Matmul`` on fp16 bit patterns: returns (rounded fp16 bits, fp32 accumulator)."""
    return _gemm16(lib().orc_hgemm, a_bits, b_bits, m, k, n, threads)


def bf16gemm(a_bits, b_bits, m, k, n, threads: int = 0):
    """``BFloat16Kernels.Matmul`` on bf16 bit patterns: returns (rounded bf16 bits, fp32 accumulator)."""
    return _gemm16(lib().orc_bf16gemm, a_bits, b_bits, m, k, n, threads)


# ------------------------------------------------------------------- attention
def attention_f32(q, k, v, scale, causal=False, query_offset=0, bias=None, keep=None,
                  softcap=0.0, want_weights=False, threads: int = 0):
    """fp32 attention as the reference CPU engine computes it.

    q [B,H,Sq,D]; k, v [B,Hkv,Sk,D]; bias [B,H,Sq,Sk] or [H,Sq,Sk]; keep: bool array of
    rank 4 broadcastable to [B,H,Sq,Sk].  Returns (out, lse, weights-or-None).
    """
    q = _c(q, np.float32); k = _c(k, np.float32); v = _c(v, np.float32)
    B, H, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    out = np.full((B, H, Sq, D), np.nan, np.float32)
    lse = np.full((B, H, Sq), np.nan, np.float32)
    w = np.full((B, H, Sq, Sk), np.nan, np.float32) if want_weights else None
    bias_p, bstride = None, 0
    if bias is not None:
        bias = _c(bias, np.float32)
        bstride = H * Sq * Sk if bias.ndim == 4 else 0
        bias_p = _p(bias, _f32p)
    keep_p, shape_p = None, None
    if keep is not None:
        keep = _c(keep, np.uint8)
        assert keep.ndim == 4
        shape = np.array(keep.shape, np.int32)
        keep_p, shape_p = _p(keep, _u8p), _p(shape, _i32p)
    lib().orc_attention_f32(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), bias_p, ctypes.c_long(bstride),
                            keep_p, shape_p, _p(out, _f32p), _p(lse, _f32p),
                            _p(w, _f32p) if w is not None else None,
                            B, H, Hkv, Sq, Sk, D, ctypes.c_float(scale), int(causal), int(query_offset),
                            ctypes.c_float(softcap), threads or max_threads())
    return out, lse, w


def attention_f64(q, k, v, scale, causal=False, query_offset=0, bias=None, keep=None,
                  softcap=0.0, threads: int = 0):
    q = _c(q, np.float32); k = _c(k, np.float32); v = _c(v, np.float32)
    B, H, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    out = np.empty((B, H, Sq, D), np.float64)
    lse = np.empty((B, H, Sq), np.float64)
    bias_p, bstride = None, 0
    if bias is not None:
        bias = _c(bias, np.float32)
        bstride = H * Sq * Sk if bias.ndim == 4 else 0
        bias_p = _p(bias, _f32p)
    keep_p, shape_p = None, None
    if keep is not None:
        keep = _c(keep, np.uint8)
        shape = np.array(keep.shape, np.int32)
        keep_p, shape_p = _p(keep, _u8p), _p(shape, _i32p)
    lib().orc_attention_f64(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), bias_p, ctypes.c_long(bstride),
                            keep_p, shape_p, _p(out, _f64p), _p(lse, _f64p),
                            B, H, Hkv, Sq, Sk, D, ctypes.c_double(scale), int(causal), int(query_offset),
                            ctypes.c_double(softcap), threads or max_threads())
    return out, lse


def paged_attention(q, kcache, vcache, block_table, heads: int, kv_heads: int, head_dim: int, block_size: int,
                    num_queries: int, start_pos: int, scale: float) -> np.ndarray:
    """The reference's paged-attention kernels (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/Kernels/HipPagedAttentionKernels.cs:
    decode :26-58, causal prefill :61-105, GQA head map h / (heads / kvHeads)): pools ``[numBlocks, blockSize, kvHeads, d]``,
    logical key t in pool row ``blockTable[t / blockSize] * blockSize + t % blockSize``, query i sees keys 0 .. startPos + i
    (decode = one query with startPos = seqLen - 1).  q ``[numQueries, heads, d]`` -> ``[numQueries, heads, d]`` fp32.
    Restated as gather + the attention above (the kernels' per-key online softmax is the same function)."""
    q = _c(q, np.float32).reshape(num_queries, heads, head_dim)
    kc = _c(kcache, np.float32).reshape(-1, block_size, kv_heads, head_dim)
    vc = _c(vcache, np.float32).reshape(-1, block_size, kv_heads, head_dim)
    key_len = start_pos + num_queries
    t = np.arange(key_len)
    rows = np.asarray(block_table, np.int64)[t // block_size]
    k = kc[rows, t % block_size]                  # [keyLen, kvHeads, d]
    v = vc[rows, t % block_size]
    o, _, _ = attention_f32(q.transpose(1, 0, 2)[None], k.transpose(1, 0, 2)[None], v.transpose(1, 0, 2)[None], scale,
                            causal=True, query_offset=start_pos)
    return np.ascontiguousarray(o[0].transpose(1, 0, 2))


def rope_interleaved(x, cos, sin, seq_len: int, start_position: int) -> np.ndarray:
    """``rope_interleaved`` (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/Kernels/HipAttentionKernels.cs:958-989) in fp32:
    x ``[rows, headDim]``, caches ``[maxSeq, headDim/2]``; pair (2i, 2i+1) of row r rotated by position start + r % seqLen."""
    x = _c(x, np.float32); cos = _c(cos, np.float32); sin = _c(sin, np.float32)
    rows, hd = x.shape
    pos = start_position + np.arange(rows) % seq_len
    c = cos.reshape(-1, hd // 2)[pos]; s = sin.reshape(-1, hd // 2)[pos]
    xe = x[:, 0::2]; xo = x[:, 1::2]
    out = np.empty_like(x)
    out[:, 0::2] = (xe * c).astype(np.float32) - (xo * s).astype(np.float32)
    out[:, 1::2] = (xe * s).astype(np.float32) + (xo * c).astype(np.float32)
    return out


def mha_forward(x, wq, wk, wv, wo, heads: int, keep=None) -> np.ndarray:
    """``MultiHeadAttentionForwardFloat`` (src/AiDotNet.Tensors/Engines/CpuEngine.MultiHeadAttention.cs:155-285): fused
    ``[Wq|Wk|Wv]`` SimdGemm on ``[B*S, dModel]``, per-(b, h) attention with scale 1/sqrt(dHead) and an optional boolean
    keep-mask broadcastable to ``[B,H,S,S]``, heads concatenated back to ``[B*S, dModel]``, output SimdGemm.
    Composed from the restated GEMM and attention above, as the reference composes ``SimdGemm.Sgemm`` and its SDPA."""
    x = _c(x, np.float32)
    B, S, dM = x.shape
    d = dM // heads
    wf = np.concatenate([_c(wq, np.float32), _c(wk, np.float32), _c(wv, np.float32)], axis=1)
    qkv = sgemm(x.reshape(B * S, dM), wf, B * S, dM, 3 * dM, threads=max_threads()).reshape(B, S, 3, heads, d)
    q = np.ascontiguousarray(qkv[:, :, 0].transpose(0, 2, 1, 3)); k = np.ascontiguousarray(qkv[:, :, 1].transpose(0, 2, 1, 3))
    v = np.ascontiguousarray(qkv[:, :, 2].transpose(0, 2, 1, 3))
    if keep is not None:
        keep = np.broadcast_to(np.asarray(keep, bool), (B, heads, S, S))
    o, _, _ = attention_f32(q, k, v, 1.0 / float(np.sqrt(d)), keep=keep)
    cc = np.ascontiguousarray(o.transpose(0, 2, 1, 3)).reshape(B * S, dM)
    return sgemm(cc, _c(wo, np.float32), B * S, dM, dM, threads=max_threads()).reshape(B, S, dM)


def decode_f32(q, k, v, heads, kv_heads, head_dim, seq_len, scale) -> np.ndarray:
    """The reference decode test's oracle: q [heads, d], k/v [seqLen, kvHeads, d] -> [heads, d]."""
    q = _c(q, np.float32); k = _c(k, np.float32); v = _c(v, np.float32)
    out = np.empty((heads, head_dim), np.float32)
    lib().orc_decode_f32(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(out, _f32p),
                         heads, kv_heads, head_dim, seq_len, ctypes.c_float(scale))
    return out


# ------------------------------------------------- secondary reference paths
def sgemm_direct_applies(m: int, k: int, n: int) -> bool:
    """The gate of ``SgemmAddInternal`` that sends a product to the no-pack kernel (SimdGemm.cs:1575-1613)."""
    return bool(lib().orc_sgemm_direct_applies(int(m), int(k), int(n)))


def thin_m_direct_applies(m: int, n: int, k: int) -> bool:
    """The thin-M carve-out of ``BlasManaged.Gemm`` to the same kernel (BlasManaged.cs:116-124, 139-154)."""
    return bool(lib().orc_thin_m_direct_applies(int(m), int(n), int(k)))


def sgemm_direct(a, b, m: int, k: int, n: int, c0=None, threads: int = 1) -> np.ndarray:
    """``SimdGemm.SgemmDirect`` (src/AiDotNet.Tensors/Engines/Simd/SimdGemm.cs:1888-2075): one fused chain over k per element;
    ``c0`` None = cleared output (store), else accumulate into a copy of it."""
    a = _c(a, np.float32); b = _c(b, np.float32)
    assert a.size == m * k and b.size == k * n
    c = np.zeros((m, n), np.float32) if c0 is None else np.array(c0, np.float32).reshape(m, n).copy()
    lib().orc_sgemm_direct(_p(a, _f32p), k, _p(b, _f32p), n, _p(c, _f32p), m, k, n, 1 if c0 is None else 0, threads)
    return c


def goto_choose_blocks(m: int, n: int, cores: int):
    """``GotoGemmFp32.ChooseParallelBlocks`` (src/AiDotNet.Tensors/Engines/BlasManaged/GotoGemmFp32.cs:91-121) -> (mc, nc, kc)."""
    out = np.zeros(3, np.int32)
    lib().orc_goto_choose_blocks(int(m), int(n), int(cores), _p(out, _i32p))
    return int(out[0]), int(out[1]), int(out[2])


def goto_gemm(a, b, m: int, k: int, n: int, blocks=None, cores: int = 16, threads: int = 0) -> np.ndarray:
    """``GotoGemmFp32.RunParallel`` (GotoGemmFp32.cs:319-480): tile grid of (mc, nc), K-panels of kc, scalar tails.
    ``blocks`` None = the reference's choice for a host with ``cores`` workers."""
    a = _c(a, np.float32); b = _c(b, np.float32)
    assert a.size == m * k and b.size == k * n
    mc, nc, kc = blocks if blocks is not None else goto_choose_blocks(m, n, cores)
    c = np.full((m, n), np.nan, np.float32)
    lib().orc_goto_gemm(_p(a, _f32p), k, _p(b, _f32p), n, _p(c, _f32p), n, m, n, k, mc, nc, kc, threads or max_threads())
    return c


def fast_exp(x) -> np.ndarray:
    """``SimdKernels.FastExp256`` per lane (src/AiDotNet.Tensors/Engines/Simd/SimdKernels.cs:3025-3077)."""
    x = _c(x, np.float32)
    L = lib()
    L.orc_fast_exp.argtypes = [ctypes.c_float]
    L.orc_fast_exp.restype = ctypes.c_float
    return np.array([L.orc_fast_exp(float(t)) for t in x.ravel()], np.float32).reshape(x.shape)


def fused_attention_fastexp(q, k, v, scale: float, causal: bool = False, threads: int = 0) -> np.ndarray:
    """``FusedAttention.BatchedFlashAttention`` / ``FlashAttentionForward`` (src/AiDotNet.Tensors/Engines/Simd/FusedAttention.cs:
    39-90, 292-325): q ``[..., seqQ, d]``, k and v ``[..., seqK, d]`` with equal leading dimensions -> out like q."""
    q = _c(q, np.float32); k = _c(k, np.float32); v = _c(v, np.float32)
    seq_q, d = q.shape[-2:]
    seq_k = k.shape[-2]
    bh = int(np.prod(q.shape[:-2], dtype=np.int64)) if q.ndim > 2 else 1
    out = np.full(q.shape, np.nan, np.float32)
    lib().orc_fused_attention_fastexp(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(out, _f32p), bh, seq_q, seq_k, d,
                                      ctypes.c_float(scale), int(causal), threads or max_threads())
    return out
