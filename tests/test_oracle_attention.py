"""Pins the CPU attention restatement (oracle/oracle_attention.c) without running the reference.

An independent numpy float64 softmax attention written here from the definition is the
cross-check; the rest are invariants and closed forms from the reference's own tests.
"""
import numpy as np
import pytest
from scipy.special import logsumexp

import oracle


def numpy_attention(q, k, v, scale, causal=False, offset=0, bias=None, keep=None, softcap=0.0):
    q = q.astype(np.float64); k = k.astype(np.float64); v = v.astype(np.float64)
    B, H, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    g = H // Hkv
    k = np.repeat(k, g, axis=1); v = np.repeat(v, g, axis=1)
    s = np.einsum("bhid,bhjd->bhij", q, k) * scale
    if softcap > 0:
        s = softcap * np.tanh(s / softcap)
    if bias is not None:
        s = s + bias.astype(np.float64)
    if keep is not None:
        s = np.where(np.broadcast_to(keep, s.shape), s, -np.inf)
    if causal:
        i = np.arange(Sq)[:, None]; j = np.arange(Sk)[None, :]
        s = np.where(j > i + offset, -np.inf, s)
    with np.errstate(invalid="ignore"):
        lse = logsumexp(s, axis=-1)
        p = np.exp(s - lse[..., None])
    p = np.where(np.isfinite(lse)[..., None], p, 0.0)
    return p @ v, lse, p


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("B,H,Hkv,Sq,Sk,D,causal,offset", [
    (1, 2, 2, 4, 4, 8, True, 0),          # OpParityRegistry.cs:1896-1899 FlashAttention [1,2,4,8]
    (2, 3, 3, 33, 65, 20, False, 0),      # FusedAttentionFp32PrecisionTests.cs:30-58 Sq != Sk, d = 20
    (1, 4, 4, 70, 70, 64, True, 0),       # non block-aligned S
    (2, 4, 2, 17, 40, 32, True, 23),      # GQA + bottom-right causal (offset = Sk - Sq)
    (1, 2, 1, 1, 77, 48, True, 76),       # decode shape
    (1, 1, 1, 100, 100, 16, False, 0),
])
def test_matches_independent_float64_attention(B, H, Hkv, Sq, Sk, D, causal, offset):
    rng = np.random.default_rng(B + 3 * H + 7 * Sq + 11 * Sk + D)
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, Hkv, Sk, D), _rand(rng, B, Hkv, Sk, D)
    scale = 1.0 / np.sqrt(D)
    o, lse, w = oracle.attention_f32(q, k, v, scale, causal, offset, want_weights=True)
    o64, lse64 = oracle.attention_f64(q, k, v, scale, causal, offset)
    wo, wl, wp = numpy_attention(q, k, v, scale, causal, offset)
    assert np.allclose(o64, wo, rtol=1e-10, atol=1e-12)
    assert np.allclose(lse64, wl, rtol=1e-10, atol=1e-12)
    assert np.max(np.abs(o - wo)) < 2e-5 * (1 + np.max(np.abs(wo)))
    assert np.max(np.abs(lse - wl)) < 1e-5 * (1 + np.max(np.abs(wl)))
    assert np.max(np.abs(w - wp)) < 1e-6
    assert np.allclose(w.sum(-1), 1.0, atol=1e-5)          # rows of P sum to 1


def test_causal_row0_returns_v0_and_zero_q_gives_running_mean():
    rng = np.random.default_rng(2)
    B, H, S, D = 1, 2, 9, 8
    q, k, v = _rand(rng, B, H, S, D), _rand(rng, B, H, S, D), _rand(rng, B, H, S, D)
    o, _, _ = oracle.attention_f32(q, k, v, 0.3, causal=True)
    assert np.allclose(o[:, :, 0], v[:, :, 0], atol=1e-6)
    o0, lse0, _ = oracle.attention_f32(np.zeros_like(q), k, v, 0.3, causal=True)
    means = np.cumsum(v.astype(np.float64), axis=2) / np.arange(1, S + 1)[None, None, :, None]
    assert np.allclose(o0, means, atol=1e-6)
    assert np.allclose(lse0, np.log(np.arange(1, S + 1))[None, None, :], atol=1e-6)   # LSE = log(count)


def test_key_permutation_invariance_non_causal():
    rng = np.random.default_rng(3)
    q, k, v = _rand(rng, 1, 2, 5, 16), _rand(rng, 1, 2, 31, 16), _rand(rng, 1, 2, 31, 16)
    perm = rng.permutation(31)
    o1, l1, _ = oracle.attention_f32(q, k, v, 0.25)
    o2, l2, _ = oracle.attention_f32(q, k[:, :, perm], v[:, :, perm], 0.25)
    assert np.allclose(o1, o2, atol=2e-6) and np.allclose(l1, l2, atol=2e-6)


def test_bias_after_scale_on_identity_qkv():
    # FlashAttentionBiasTests.cs:89-115: Q = K = V = I, bias added AFTER the scale, before softmax
    S = 4
    eye = np.eye(S, dtype=np.float32)[None, None]
    bias = np.zeros((1, 1, S, S), np.float32); bias[0, 0, :, 2] = 5.0
    scale = 0.5
    o, lse, w = oracle.attention_f32(eye, eye, eye, scale, bias=bias, want_weights=True)
    logits = scale * np.eye(S) + bias[0, 0]
    p = np.exp(logits) / np.exp(logits).sum(-1, keepdims=True)
    assert np.allclose(w[0, 0], p, atol=1e-6)
    assert np.allclose(o[0, 0], p, atol=1e-6)             # V = I so O = P
    # a 3-D bias is broadcast over the batch
    q = np.repeat(eye, 2, axis=0)
    o3, _, _ = oracle.attention_f32(q, q, q, scale, bias=bias[0])
    assert np.allclose(o3[0], o[0], atol=1e-7) and np.allclose(o3[1], o[0], atol=1e-7)


def test_softcap_closed_form():
    # BatchMatMulAndAttentionTests.cs:288-317: logits = cap * tanh(scale*qk / cap)
    rng = np.random.default_rng(4)
    q, k, v = _rand(rng, 1, 1, 3, 4) * 3, _rand(rng, 1, 1, 6, 4) * 3, _rand(rng, 1, 1, 6, 4)
    cap = 2.0
    o, _, w = oracle.attention_f32(q, k, v, 1.0, softcap=cap, want_weights=True)
    wo, _, wp = numpy_attention(q, k, v, 1.0, softcap=cap)
    assert np.allclose(w, wp, atol=1e-6) and np.allclose(o, wo, atol=1e-5)
    o_nc, _, _ = oracle.attention_f32(q, k, v, 1.0)
    assert np.max(np.abs(o - o_nc)) > 1e-3                # the cap really changed something


def test_boolean_mask_broadcast_and_all_masked_rows():
    # SdpaMaskBroadcastTests.cs:73-125; all-masked row -> zeros (CpuEngine.cs:27817-27822), LSE = -inf (:29243-29249)
    rng = np.random.default_rng(5)
    B, H, Sq, Sk, D = 2, 3, 4, 6, 8
    q, k, v = _rand(rng, B, H, Sq, D), _rand(rng, B, H, Sk, D), _rand(rng, B, H, Sk, D)
    keep = rng.random((1, 1, Sq, Sk)) > 0.4
    keep[0, 0, 1, :] = False
    o, lse, w = oracle.attention_f32(q, k, v, 0.35, keep=keep, want_weights=True)
    full = np.broadcast_to(keep, (B, H, Sq, Sk)).copy()
    o2, lse2, w2 = oracle.attention_f32(q, k, v, 0.35, keep=full, want_weights=True)
    assert np.array_equal(o, o2) and np.array_equal(w, w2)
    wo, _, wp = numpy_attention(q, k, v, 0.35, keep=keep)
    assert np.allclose(o, wo, atol=1e-5) and np.allclose(w, wp, atol=1e-6)
    assert np.all(o[:, :, 1] == 0) and np.all(w[:, :, 1] == 0) and np.all(np.isneginf(lse[:, :, 1]))
    keep_b = rng.random((B, 1, 1, Sk)) > 0.3
    keep_b[:, :, :, 0] = True
    o3, _, _ = oracle.attention_f32(q, k, v, 0.35, keep=keep_b)
    assert np.allclose(o3, numpy_attention(q, k, v, 0.35, keep=keep_b)[0], atol=1e-5)


def test_decode_equals_last_row_of_causal_prefill():
    # FusedAttentionAuditTests.cs:47-79: Sq=1, QueryOffset=t, Sk=t+1 equals row t of the full causal run
    rng = np.random.default_rng(6)
    B, H, S, D = 1, 4, 12, 16
    q, k, v = _rand(rng, B, H, S, D), _rand(rng, B, H, S, D), _rand(rng, B, H, S, D)
    full, lse_full, _ = oracle.attention_f32(q, k, v, 0.25, causal=True)
    for t in (0, 5, 11):
        o, lse, _ = oracle.attention_f32(q[:, :, t:t + 1], k[:, :, :t + 1], v[:, :, :t + 1], 0.25, causal=True, query_offset=t)
        assert np.allclose(o[:, :, 0], full[:, :, t], atol=1e-6)
        assert np.allclose(lse[:, :, 0], lse_full[:, :, t], atol=1e-6)


@pytest.mark.parametrize("heads,kv,d,seq", [(4, 4, 64, 40), (8, 8, 32, 100), (4, 4, 64, 7), (6, 6, 48, 77), (8, 2, 64, 50)])
def test_decode_oracle_matches_attention_oracle(heads, kv, d, seq):
    # FlashDecodeHipTests.cs:107-130 shapes; layout [seqLen, kvHeads, d]
    rng = np.random.default_rng(heads + kv + d + seq)
    q = rng.uniform(-1, 1, (heads, d)).astype(np.float32)
    k = rng.uniform(-1, 1, (seq, kv, d)).astype(np.float32)
    v = rng.uniform(-1, 1, (seq, kv, d)).astype(np.float32)
    scale = 1.0 / np.sqrt(d)
    got = oracle.decode_f32(q, k, v, heads, kv, d, seq, scale)
    kk = np.ascontiguousarray(k.transpose(1, 0, 2))[None]
    vv = np.ascontiguousarray(v.transpose(1, 0, 2))[None]
    want, _, _ = numpy_attention(q[None, :, None, :], kk, vv, scale)
    assert np.all(np.abs(got - want[0, :, 0]) <= 2e-5 + 2e-5 * np.abs(want[0, :, 0]))
    o, _, _ = oracle.attention_f32(q[None, :, None, :], kk, vv, scale)
    assert np.allclose(o[0, :, 0], got, atol=2e-6)


def test_fp32_error_vs_fp64_is_small_but_nonzero():
    # FusedAttentionFp32PrecisionTests.cs:30-58: max-abs < 2e-3 and > 0 on U[-1,1] inputs
    rng = np.random.default_rng(8)
    q = rng.uniform(-1, 1, (2, 4, 64, 32)).astype(np.float32)
    k = rng.uniform(-1, 1, (2, 4, 64, 32)).astype(np.float32)
    v = rng.uniform(-1, 1, (2, 4, 64, 32)).astype(np.float32)
    o, _, _ = oracle.attention_f32(q, k, v, 1 / np.sqrt(32), causal=True)
    o64, _ = oracle.attention_f64(q, k, v, 1 / np.sqrt(32), causal=True)
    err = np.max(np.abs(o - o64))
    assert 0 < err < 2e-3
