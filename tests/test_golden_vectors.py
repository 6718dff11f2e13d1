"""The reference's own known-answer vectors and case tables (tests/golden/reference_known_answers.json).

CPU part: pins the oracle.  GPU part (marked ``gpu``): the HIP path through the C ABI against the same vectors.
Every fixture entry cites the reference test it was transcribed from.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

import oracle
from _util import dev, mixed_err, round_to, from_bits16, bits16

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))
TABLES = GOLD["case_tables"]


def _f32(x, shape=None):
    a = np.asarray(x, np.float32)
    return a.reshape(shape) if shape is not None else a


def _hash_u(shape, seed):
    """U[-0.5, 0.5) from the portable hash generator the reference's GPU/CPU consistency tests use."""
    n = int(np.prod(shape))
    return oracle.hash_uniform(n, seed).reshape(shape)


# ----------------------------------------------------------------------------------------------- CPU: the oracle
@pytest.mark.parametrize("case", GOLD["batch_matmul"], ids=lambda c: c["source"].split("(")[1][:-1])
def test_oracle_batch_matmul_known_answers(case):
    b_, m, k, n = case["batch"], case["m"], case["k"], case["n"]
    a = _f32(case["a"], (b_, m, k)); b = _f32(case["b"], (b_, k, n))
    got = np.stack([oracle.sgemm(a[i], b[i], m, k, n) for i in range(b_)]).ravel()
    assert np.max(np.abs(got - _f32(case["expected"]))) <= case["abs_tol"]


def test_oracle_bf16_matmul_known_answer():
    c = GOLD["bf16_matmul"][0]
    a_bits = oracle.f32_to_bf16(_f32(c["a"])); b_bits = oracle.f32_to_bf16(_f32(c["b"]))
    o16, o32 = oracle.bf16gemm(a_bits, b_bits, c["m"], c["k"], c["n"])
    assert oracle.bf16_to_f32(o16).ravel().tolist() == [float(x) for x in c["expected"]]
    assert o32.ravel().tolist() == [float(x) for x in c["expected"]]


def _softcap_expected(c):
    s = [c["scale"] * c["q"][0] * kk for kk in c["k"]]
    t = [c["softcap"] * math.tanh(x / c["softcap"]) for x in s]
    m = max(t); e = [math.exp(x - m) for x in t]
    return [x / sum(e) for x in e]


def test_oracle_softcap_known_answer():
    c = GOLD["sdpa_softcap"]; sh = c["shape"]
    q = _f32(c["q"], (1, 1, sh["Sq"], sh["D"])); k = _f32(c["k"], (1, 1, sh["Sk"], sh["D"])); v = _f32(c["v"], (1, 1, sh["Sk"], sh["D"]))
    _, _, w = oracle.attention_f32(q, k, v, c["scale"], softcap=c["softcap"], want_weights=True)
    exp = _softcap_expected(c)
    assert np.max(np.abs(w.ravel() - np.array(exp))) < 0.5 * 10 ** -c["decimals"]
    _, _, wp = oracle.attention_f32(q, k, v, c["scale"], want_weights=True)
    assert wp.ravel()[1] < c["plain_low_weight_below"]
    assert w.ravel()[1] > c["capped_over_plain_ratio_above"] * wp.ravel()[1]


def test_oracle_bias_after_scale_known_answer():
    c = GOLD["flash_attention_bias_identity"]; sh = c["shape"]
    q = _f32(c["q"], (1, 1, sh["Sq"], sh["D"])); k = _f32(c["k"], (1, 1, sh["Sk"], sh["D"])); v = _f32(c["v"], (1, 1, sh["Sk"], sh["D"]))
    bias = _f32(c["bias"], (1, 1, sh["Sq"], sh["Sk"]))
    out, _, _ = oracle.attention_f32(q, k, v, 1.0 / math.sqrt(sh["D"]), bias=bias)
    assert out.ravel()[0] < c["expect_out0_below"] and out.ravel()[1] > c["expect_out1_above"]


def test_oracle_decode_equals_last_prefill_row():
    sh = GOLD["decode_equals_last_prefill_row"]["shape"]; t = sh["t"]; D = sh["Dk"]
    qs = _hash_u((1, 1, 1, D), 301); k = _hash_u((1, 1, t + 1, D), 302); v = _hash_u((1, 1, t + 1, D), 303)
    o1, _, _ = oracle.attention_f32(qs, k, v, 1 / math.sqrt(D), causal=True, query_offset=t)
    qf = np.zeros((1, 1, t + 1, D), np.float32); qf[0, 0, t] = qs[0, 0, 0]
    o2, _, _ = oracle.attention_f32(qf, k, v, 1 / math.sqrt(D), causal=True, query_offset=0)
    assert np.max(np.abs(o1[0, 0, 0] - o2[0, 0, t])) < 0.5e-4


@pytest.mark.parametrize("m,k,n", [tuple(c) for c in TABLES["fp32_matmul_shapes_m_k_n"]["cases"]])
def test_oracle_fp32_matmul_reference_shapes(m, k, n):
    a = 2 * _hash_u((m, k), 42); b = 2 * _hash_u((k, n), 43)
    truth = a.astype(np.float64) @ b.astype(np.float64)
    assert mixed_err(oracle.sgemm(a, b, m, k, n), truth) <= 1e-4


@pytest.mark.parametrize("b,h,sq,sk,d", [tuple(c) for c in TABLES["fp32_attention_vs_fp64_b_h_sq_sk_d"]["cases"]])
def test_oracle_fp32_attention_drift_from_fp64(b, h, sq, sk, d):
    q = 2 * _hash_u((b, h, sq, d), 11); k = 2 * _hash_u((b, h, sk, d), 12); v = 2 * _hash_u((b, h, sk, d), 13)
    o32, _, _ = oracle.attention_f32(q, k, v, 1 / math.sqrt(d))
    o64, _ = oracle.attention_f64(q, k, v, 1 / math.sqrt(d))
    diff = float(np.max(np.abs(o32 - o64)))
    assert 0.0 < diff < TABLES["fp32_attention_vs_fp64_b_h_sq_sk_d"]["max_abs_below"]


@pytest.mark.parametrize("b,h,sq,sk,d,causal", [tuple(c) for c in TABLES["flash_attention2_tiny_b_h_sq_sk_d_causal"]["cases"]])
def test_oracle_matches_naive_softmax_matmul(b, h, sq, sk, d, causal):
    q = _hash_u((b, h, sq, d), 1); k = _hash_u((b, h, sk, d), 2); v = _hash_u((b, h, sk, d), 3)
    out, _, _ = oracle.attention_f32(q, k, v, 1 / math.sqrt(d), causal=causal)
    s = np.einsum("bhid,bhjd->bhij", q.astype(np.float64), k.astype(np.float64)) / math.sqrt(d)
    if causal:
        s = np.where(np.arange(sk)[None, :] > np.arange(sq)[:, None], -np.inf, s)
    p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
    ref = np.einsum("bhij,bhjd->bhid", p, v.astype(np.float64))
    assert np.max(np.abs(out - ref)) < 0.5e-4


# ----------------------------------------------------------------------------------------------- GPU: the HIP path
@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    return Mi355Backend()


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLD["batch_matmul"], ids=lambda c: c["source"].split("(")[1][:-1])
def test_gpu_batch_matmul_known_answers(be, case):
    b_, m, k, n = case["batch"], case["m"], case["k"], case["n"]
    A = be.WrapTensor(dev(_f32(case["a"]))); B = be.WrapTensor(dev(_f32(case["b"])))
    c = torch.full((b_ * m * n,), 3.0e30, device="cuda")
    be.BatchedGemm(A, B, be.WrapTensor(c), m, n, k, b_)
    assert np.max(np.abs(c.cpu().numpy() - _f32(case["expected"]))) <= case["abs_tol"]


@pytest.mark.gpu
def test_gpu_bf16_matmul_known_answer(be):
    c = GOLD["bf16_matmul"][0]
    a = from_bits16(oracle.f32_to_bf16(_f32(c["a"])), torch.bfloat16); b = from_bits16(oracle.f32_to_bf16(_f32(c["b"])), torch.bfloat16)
    out = torch.empty(c["m"] * c["n"], device="cuda", dtype=torch.bfloat16)
    be.Bf16Gemm(be.WrapTensor(a), be.WrapTensor(b), be.WrapTensor(out), c["m"], c["n"], c["k"])
    assert oracle.bf16_to_f32(bits16(out)).tolist() == [float(x) for x in c["expected"]]
    out32 = torch.empty(c["m"] * c["n"], device="cuda")
    be.GemmBf16In32fOut(be.WrapTensor(a), be.WrapTensor(b), be.WrapTensor(out32), c["m"], c["n"], c["k"])
    assert out32.cpu().numpy().tolist() == [float(x) for x in c["expected"]]


@pytest.mark.gpu
def test_gpu_softcap_known_answer(be):
    c = GOLD["sdpa_softcap"]; sh = c["shape"]
    q = dev(_f32(c["q"])); k = dev(_f32(c["k"])); v = dev(_f32(c["v"]))
    W = be.WrapTensor

    def run(cap):
        o = torch.empty(sh["Sq"] * sh["D"], device="cuda"); w = torch.empty(sh["Sq"] * sh["Sk"], device="cuda")
        be.ScaledDotProductAttention(W(q), W(k), W(v), W(o), W(w), None, 1, 1, sh["Sq"], sh["Sk"], sh["D"], c["scale"], False, cap)
        return w.cpu().numpy()
    w = run(c["softcap"]); wp = run(0.0)
    assert np.max(np.abs(w - np.array(_softcap_expected(c)))) < 0.5 * 10 ** -c["decimals"]
    assert wp[1] < c["plain_low_weight_below"] and w[1] > c["capped_over_plain_ratio_above"] * wp[1]


@pytest.mark.gpu
def test_gpu_bias_after_scale_known_answer(be):
    c = GOLD["flash_attention_bias_identity"]; sh = c["shape"]
    W = be.WrapTensor
    q = dev(_f32(c["q"])); k = dev(_f32(c["k"])); v = dev(_f32(c["v"])); bias = dev(_f32(c["bias"]))
    o = torch.empty(sh["Sq"] * sh["D"], device="cuda"); st = torch.empty(sh["Sq"], device="cuda")
    be.FlashAttentionV2(W(q), W(k), W(v), W(o), W(st), 1, 1, sh["Sq"], sh["Sk"], sh["D"], 1 / math.sqrt(sh["D"]), False, W(bias), 0)
    out = o.cpu().numpy()
    assert out[0] < c["expect_out0_below"] and out[1] > c["expect_out1_above"]


@pytest.mark.gpu
def test_gpu_query_offset_out_of_bounds_is_an_argument_error():
    from aidotnet.tensors_amd import Mi355Engine
    from aidotnet.tensors_amd.backend import ArgumentException
    c = GOLD["query_offset_out_of_bounds"]; sh = c["shape"]
    eng = Mi355Engine()
    q = torch.zeros(sh["B"], sh["H"], sh["Sq"], sh["D"], device="cuda"); k = torch.zeros(sh["B"], sh["H"], sh["Sk"], sh["D"], device="cuda")
    with pytest.raises(ArgumentException):
        eng.FlashAttention(q, k, k.clone(), None, True, None, c["query_offset"])


@pytest.mark.gpu
def test_gpu_decode_equals_last_prefill_row():
    from aidotnet.tensors_amd import Mi355Engine
    sh = GOLD["decode_equals_last_prefill_row"]["shape"]; t = sh["t"]; D = sh["Dk"]
    eng = Mi355Engine()
    qs = _hash_u((1, 1, 1, D), 301); k = _hash_u((1, 1, t + 1, D), 302); v = _hash_u((1, 1, t + 1, D), 303)
    o1 = eng.FlashAttention(dev(qs), dev(k), dev(v), None, True, None, t)[0].cpu().numpy()
    qf = np.zeros((1, 1, t + 1, D), np.float32); qf[0, 0, t] = qs[0, 0, 0]
    o2 = eng.FlashAttention(dev(qf), dev(k), dev(v), None, True, None, 0)[0].cpu().numpy()
    assert np.max(np.abs(o1[0, 0, 0] - o2[0, 0, t])) < 0.5e-4


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n", [tuple(c) for c in TABLES["fp32_matmul_shapes_m_k_n"]["cases"]])
def test_gpu_fp32_matmul_reference_shapes(be, m, k, n):
    a = 2 * _hash_u((m, k), 42); b = 2 * _hash_u((k, n), 43)
    c = torch.full((m * n,), 3.0e30, device="cuda")
    be.Gemm(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(c), m, n, k)
    truth = a.astype(np.float64) @ b.astype(np.float64)
    assert mixed_err(c.cpu().numpy().reshape(m, n), truth) <= 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [tuple(c) for c in TABLES["fp16_in_fp32_out_gemm_m_n_k"]["cases"]])
def test_gpu_fp16_in_fp32_out_reference_shapes(be, m, n, k):
    tab = TABLES["fp16_in_fp32_out_gemm_m_n_k"]
    a = 2 * _hash_u((m, k), 1234 + m + k); b = 2 * _hash_u((k, n), 5678 + n + k)
    a16 = torch.empty(m * k, device="cuda", dtype=torch.float16); b16 = torch.empty(k * n, device="cuda", dtype=torch.float16)
    be.ConvertToFp16(be.WrapTensor(dev(a.ravel())), be.WrapTensor(a16), m * k)      # the reference test converts on the device too
    be.ConvertToFp16(be.WrapTensor(dev(b.ravel())), be.WrapTensor(b16), k * n)
    c = torch.empty(m * n, device="cuda")
    be.GemmFp16In32fOut(be.WrapTensor(a16), be.WrapTensor(b16), be.WrapTensor(c), m, n, k)
    _, ar = round_to(a, "f16"); _, br = round_to(b, "f16")
    exp = ar.astype(np.float64) @ br.astype(np.float64)
    got = c.cpu().numpy().reshape(m, n)
    assert np.all(np.abs(got - exp) <= tab["abs_tol"] + tab["rel_tol"] * np.abs(exp))
    assert mixed_err(got, exp) <= 2e-2


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [tuple(c) for c in TABLES["non_positive_dims_rejected"]["cases"]])
def test_gpu_non_positive_dims_rejected(be, m, n, k):
    from aidotnet.tensors_amd.backend import ArgumentOutOfRangeException
    d16 = be.WrapTensor(torch.zeros(16, device="cuda", dtype=torch.float16)); d32 = be.WrapTensor(torch.zeros(16, device="cuda"))
    with pytest.raises(ArgumentOutOfRangeException):
        be.GemmFp16In32fOut(d16, d16, d32, m, n, k)


def _decode_case(be, heads, kv, d, seq, splits):
    tab = TABLES["flash_decode_mha_heads_d_seq_splits"]
    seed = 0xFDE + heads + kv + seq + splits
    k = 2 * _hash_u((seq, kv, d), seed); v = 2 * _hash_u((seq, kv, d), seed + 1); q = 2 * _hash_u((heads, d), seed + 2)
    scale = 1.0 / math.sqrt(d)
    out = be.FlashDecode(be.WrapTensor(dev(q.ravel())), be.WrapTensor(dev(k.ravel())), be.WrapTensor(dev(v.ravel())),
                         heads, kv, d, seq, scale, splits)
    got = be.DownloadBuffer(out).numpy().reshape(heads, d)
    exp = oracle.decode_f32(q, k, v, heads, kv, d, seq, scale)
    assert np.all(np.abs(got - exp) <= tab["abs_tol"] + tab["rel_tol"] * np.abs(exp))


@pytest.mark.gpu
@pytest.mark.parametrize("heads,d,seq,splits", [tuple(c) for c in TABLES["flash_decode_mha_heads_d_seq_splits"]["cases"]])
def test_gpu_flash_decode_mha_reference_cases(be, heads, d, seq, splits):
    _decode_case(be, heads, heads, d, seq, splits)


@pytest.mark.gpu
@pytest.mark.parametrize("heads,kv,d,seq,splits", [tuple(c) for c in TABLES["flash_decode_gqa_heads_kv_d_seq_splits"]["cases"]])
def test_gpu_flash_decode_gqa_reference_cases(be, heads, kv, d, seq, splits):
    _decode_case(be, heads, kv, d, seq, splits)


@pytest.mark.gpu
@pytest.mark.parametrize("b,h,sq,sk,d", [tuple(c) for c in TABLES["fp32_attention_vs_fp64_b_h_sq_sk_d"]["cases"]])
def test_gpu_fp32_attention_drift_from_fp64(be, b, h, sq, sk, d):
    q = 2 * _hash_u((b, h, sq, d), 11); k = 2 * _hash_u((b, h, sk, d), 12); v = 2 * _hash_u((b, h, sk, d), 13)
    W = be.WrapTensor
    o = torch.empty(b, h, sq, d, device="cuda"); st = torch.empty(b, h, sq, device="cuda")
    be.FlashAttentionV2(W(dev(q)), W(dev(k)), W(dev(v)), W(o), W(st), b, h, sq, sk, d, 1 / math.sqrt(d), False)
    o64, _ = oracle.attention_f64(q, k, v, 1 / math.sqrt(d))
    diff = float(np.max(np.abs(o.cpu().numpy() - o64)))
    assert 0.0 < diff < TABLES["fp32_attention_vs_fp64_b_h_sq_sk_d"]["max_abs_below"]


@pytest.mark.gpu
@pytest.mark.parametrize("b,h,sq,sk,d,causal", [tuple(c) for c in TABLES["flash_attention2_tiny_b_h_sq_sk_d_causal"]["cases"]])
def test_gpu_matches_naive_softmax_matmul(be, b, h, sq, sk, d, causal):
    q = _hash_u((b, h, sq, d), 1); k = _hash_u((b, h, sk, d), 2); v = _hash_u((b, h, sk, d), 3)
    W = be.WrapTensor
    o = torch.empty(b, h, sq, d, device="cuda"); st = torch.empty(b, h, sq, device="cuda")
    be.FlashAttentionV2(W(dev(q)), W(dev(k)), W(dev(v)), W(o), W(st), b, h, sq, sk, d, 1 / math.sqrt(d), causal)
    ref, _, _ = oracle.attention_f32(q, k, v, 1 / math.sqrt(d), causal=causal)
    assert np.max(np.abs(o.cpu().numpy() - ref)) < 0.5e-4
