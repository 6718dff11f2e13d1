"""Fused projection epilogues C = act(A B + bias): oracle pins (CPU) and HIP parity (GPU).

Reference: IDirectGpuBackend.GemmBias* (src/AiDotNet.Tensors/Engines/DirectGpu/IDirectGpuBackend.cs:227-275),
IEngine.FusedLinear (Engines/IEngine.cs:5166), CPU epilogue Helpers/CpuFusedOperations.cs:590-700, 1268-1280, 1452-1460.
Tolerances: mixed error <= 1e-4 (fp32), <= 2e-2 (fp16 / bf16) against the float64 closed form on the same rounded inputs.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import dev, mixed_err, round_to, from_bits16, bits16, TORCH16

ACTS = {0: "none", 1: "relu", 2: "gelu", 3: "sigmoid", 4: "tanh", 5: "leaky_relu", 6: "swish"}


def act64(x, act, p=0.0):
    """Independent float64 closed forms (numpy), not the oracle's code."""
    x = np.asarray(x, np.float64)
    if act == 0: return x
    if act == 1: return np.where(x < 0, 0.0, x)
    if act == 2: return 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))
    if act == 3: return 1.0 / (1.0 + np.exp(-x))
    if act == 4: return np.tanh(x)
    if act == 5: return np.where(x > 0, x, p * x)
    if act == 6: return x / (1.0 + np.exp(-x))
    raise ValueError(act)


# ------------------------------------------------------------------------------------------------ oracle (CPU)
def test_oracle_activation_known_values():
    x = np.array([[-2.0, -1.0, 0.0, 0.5, 3.0, 20.0]], np.float32)
    assert oracle.bias_activation(x, None, 1).tolist() == [[0.0, 0.0, 0.0, 0.5, 3.0, 20.0]]
    assert oracle.bias_activation(x, None, 5, 0.1)[0, 0] == np.float32(-0.2) and oracle.bias_activation(x, None, 5, 0.1)[0, 4] == 3.0
    assert oracle.bias_activation(x, None, 3)[0, 2] == 0.5 and oracle.bias_activation(x, None, 6)[0, 2] == 0.0
    assert oracle.bias_activation(x, None, 2)[0, 2] == 0.0 and oracle.bias_activation(x, None, 4)[0, 2] == 0.0
    assert abs(oracle.bias_activation(x, None, 2)[0, 5] - 20.0) < 1e-5          # GELU(x) -> x for large x
    assert abs(oracle.bias_activation(x, None, 2)[0, 1] - (-0.15880801)) < 1e-6  # GELU tanh form at -1
    assert abs(oracle.bias_activation(x, None, 6)[0, 1] - (-0.26894142)) < 1e-6  # swish(-1) = -sigmoid(-1)... = -1/(1+e)
    nan = oracle.bias_activation(np.array([[np.nan]], np.float32), None, 1)
    assert np.isnan(nan[0, 0])                                                     # the reference's ReLU keeps NaN


@pytest.mark.parametrize("act", sorted(ACTS))
def test_oracle_epilogue_matches_float64_closed_form(act):
    rng = np.random.default_rng(100 + act)
    c = (3 * rng.standard_normal((37, 53))).astype(np.float32); bias = rng.standard_normal(53).astype(np.float32)
    got = oracle.bias_activation(c, bias, act, 0.07)
    exp = act64(c.astype(np.float64) + bias.astype(np.float64)[None, :], act, 0.07)
    assert mixed_err(got, exp) <= 2e-6
    no_bias = oracle.bias_activation(c, None, act, 0.07)
    assert mixed_err(no_bias, act64(c, act, 0.07)) <= 2e-6
    assert not np.array_equal(got, no_bias)


# ------------------------------------------------------------------------------------------------ HIP path (GPU)
@pytest.fixture(scope="module")
def be():
    from aidotnet.tensors_amd import Mi355Backend
    return Mi355Backend()


FP32_SHAPES = [(7, 13, 11), (96, 80, 130), (128, 256, 64), (256, 512, 192), (33, 1000, 40)]


@pytest.mark.gpu
@pytest.mark.parametrize("act", sorted(ACTS))
@pytest.mark.parametrize("m,n,k", FP32_SHAPES)
def test_gpu_sgemm_bias_act_matches_oracle_and_truth(be, act, m, n, k):
    rng = np.random.default_rng(7 * act + m + n + k)
    a = rng.standard_normal((m, k)).astype(np.float32); b = (rng.standard_normal((k, n)) / math.sqrt(k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c = torch.full((m * n,), 3.0e30, device="cuda")
    be.GemmBiasActivationInto(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(dev(bias)), be.WrapTensor(c), m, n, k, act, 0.07)
    got = c.cpu().numpy().reshape(m, n)
    truth = act64(a.astype(np.float64) @ b.astype(np.float64) + bias.astype(np.float64)[None, :], act, 0.07)
    orc = oracle.bias_activation(oracle.sgemm(a, b, m, k, n), bias, act, 0.07)
    assert mixed_err(got, truth) <= 1e-4
    assert mixed_err(got, orc) <= 1e-4


@pytest.mark.gpu
def test_gpu_named_members_allocate_and_agree(be):
    rng = np.random.default_rng(5)
    m, n, k = 64, 96, 48
    a = rng.standard_normal((m, k)).astype(np.float32); b = rng.standard_normal((k, n)).astype(np.float32) * 0.2
    bias = rng.standard_normal(n).astype(np.float32)
    A, B, BI = be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(dev(bias))
    pre = a.astype(np.float64) @ b.astype(np.float64) + bias[None, :]
    for fn, act, kw in ((be.GemmBias, 0, {}), (be.GemmBiasRelu, 1, {}), (be.GemmBiasGelu, 2, {}), (be.GemmBiasSigmoid, 3, {}),
                        (be.GemmBiasTanh, 4, {}), (be.GemmBiasSwish, 6, {}), (be.GemmBiasLeakyRelu, 5, {"alpha": 0.2})):
        out = fn(A, B, BI, m, n, k, **kw)
        assert out.Size == m * n
        got = be.DownloadBuffer(out).numpy().reshape(m, n)
        assert mixed_err(got, act64(pre, act, kw.get("alpha", 0.0))) <= 1e-4, fn.__name__
    # default leaky slope is 0.01 (IDirectGpuBackend.cs:275)
    got = be.DownloadBuffer(be.GemmBiasLeakyRelu(A, B, BI, m, n, k)).numpy().reshape(m, n)
    assert mixed_err(got, act64(pre, 5, 0.01)) <= 1e-4


@pytest.mark.gpu
def test_gpu_bias_exact_on_dyadic_inputs_and_relu_zeroes(be):
    rng = np.random.default_rng(9)
    m, n, k = 128, 128, 64
    a = rng.integers(-4, 5, (m, k)).astype(np.float32) / 4; b = rng.integers(-4, 5, (k, n)).astype(np.float32) / 4
    bias = rng.integers(-8, 9, n).astype(np.float32) / 2
    exact = a.astype(np.float64) @ b.astype(np.float64) + bias[None, :]
    for act in (0, 1):
        c = torch.empty(m * n, device="cuda")
        be.GemmBiasActivationInto(be.WrapTensor(dev(a)), be.WrapTensor(dev(b)), be.WrapTensor(dev(bias)), be.WrapTensor(c), m, n, k, act)
        assert np.array_equal(c.cpu().numpy().reshape(m, n).astype(np.float64), act64(exact, act))


HALF_SHAPES = [(64, 128, 64), (37, 53, 71), (256, 256, 128), (512, 768, 256), (32, 256, 128), (8, 128, 64)]


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("act", [0, 1, 2, 6])
@pytest.mark.parametrize("m,n,k", HALF_SHAPES)
def test_gpu_half_gemm_bias_act(be, kind, act, m, n, k):
    rng = np.random.default_rng(31 * act + m + n + k)
    a = rng.standard_normal((m, k)).astype(np.float32); b = (rng.standard_normal((k, n)) / math.sqrt(k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    ab, ar = round_to(a, kind); bb, br = round_to(b, kind)
    truth = act64(ar.astype(np.float64) @ br.astype(np.float64) + bias.astype(np.float64)[None, :], act, 0.0)
    A = be.WrapTensor(from_bits16(ab, TORCH16[kind])); B = be.WrapTensor(from_bits16(bb, TORCH16[kind])); BI = be.WrapTensor(dev(bias))
    c32 = torch.full((m * n,), 3.0e30, device="cuda")
    be.GemmBiasActivationHalf(kind, A, B, BI, be.WrapTensor(c32), m, n, k, act, 0.0, outputIsFp32=True)
    got32 = c32.cpu().numpy().reshape(m, n)
    assert mixed_err(got32, truth) <= 2e-2
    c16 = torch.empty(m * n, device="cuda", dtype=TORCH16[kind])
    be.GemmBiasActivationHalf(kind, A, B, BI, be.WrapTensor(c16), m, n, k, act, 0.0, outputIsFp32=False)
    narrow = oracle.f32_to_f16 if kind == "f16" else oracle.f32_to_bf16
    assert np.array_equal(bits16(c16).reshape(m, n), narrow(got32).reshape(m, n))      # 16-bit out = one RNE of the fp32 result


@pytest.mark.gpu
def test_gpu_large_tile_and_skinny_paths_take_the_epilogue(be):
    rng = np.random.default_rng(77)
    # 256 x 256 direct-to-LDS tiles; split-K skinny path; 128 x 128 tiles of the 16x16x32 kernel; its split-K form (8 K ranges)
    for (m, n, k) in ((2048, 2048, 256), (16, 4096, 512), (1024, 1024, 192), (256, 1024, 4096)):
        a = rng.standard_normal((m, k)).astype(np.float32); b = (rng.standard_normal((k, n)) / math.sqrt(k)).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        ab, ar = round_to(a, "bf16"); bb, br = round_to(b, "bf16")
        truth = act64(ar.astype(np.float64) @ br.astype(np.float64) + bias.astype(np.float64)[None, :], 2)
        c = torch.empty(m * n, device="cuda")
        be.GemmBiasActivationHalf("bf16", be.WrapTensor(from_bits16(ab, torch.bfloat16)), be.WrapTensor(from_bits16(bb, torch.bfloat16)),
                                  be.WrapTensor(dev(bias)), be.WrapTensor(c), m, n, k, 2, 0.0, outputIsFp32=True)
        assert mixed_err(c.cpu().numpy().reshape(m, n), truth) <= 2e-2


@pytest.mark.gpu
def test_engine_fused_linear_shapes_and_errors():
    from aidotnet.tensors_amd import Mi355Engine
    from aidotnet.tensors_amd.backend import ArgumentException, NotSupportedException
    eng = Mi355Engine()
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 5, 24)).astype(np.float32); w = rng.standard_normal((24, 40)).astype(np.float32) * 0.2
    bias = rng.standard_normal(40).astype(np.float32)
    out = eng.FusedLinear(dev(x), dev(w), dev(bias), "GELU")
    assert tuple(out.shape) == (2, 5, 40)
    exp = act64(x.reshape(10, 24).astype(np.float64) @ w.astype(np.float64) + bias[None, :], 2).reshape(2, 5, 40)
    assert mixed_err(out.cpu().numpy(), exp) <= 1e-4
    out = eng.FusedLinear(dev(x), dev(w), None, "ReLU")
    assert mixed_err(out.cpu().numpy(), act64(x.reshape(10, 24).astype(np.float64) @ w.astype(np.float64), 1).reshape(2, 5, 40)) <= 1e-4
    h = eng.FusedLinear(dev(x).half(), dev(w).half(), dev(bias), "Swish", out_dtype=torch.float32)
    assert h.dtype == torch.float32 and tuple(h.shape) == (2, 5, 40)
    with pytest.raises(ArgumentException):
        eng.FusedLinear(dev(x), dev(w[:20]), dev(bias))
    with pytest.raises(ArgumentException):
        eng.FusedLinear(dev(x), dev(w), dev(bias[:7]))
    with pytest.raises(NotSupportedException):
        eng.FusedLinear(dev(x), dev(w), dev(bias), "Softmax")


@pytest.mark.gpu
def test_gpu_unknown_activation_is_an_argument_error(be):
    from aidotnet.tensors_amd.backend import ArgumentException
    t = be.WrapTensor(torch.zeros(16, device="cuda"))
    with pytest.raises(ArgumentException):
        be.GemmBiasActivationInto(t, t, None, t, 4, 4, 4, 9)


# ------------------------------------------------------------------------------------------------ weight-only fp16 GEMM
def test_oracle_fp16_weight_gemm_matches_float64_of_widened_weights():
    rng = np.random.default_rng(12)
    m, k, n = 37, 71, 53
    a = rng.standard_normal((m, k)).astype(np.float32); b = rng.standard_normal((k, n)).astype(np.float32)
    bb, br = round_to(b, "f16")
    got = oracle.sgemm_fp16_weight_b(a, bb, m, k, n)
    assert mixed_err(got, a.astype(np.float64) @ br.astype(np.float64)) <= 1e-5
    assert not np.array_equal(got, oracle.sgemm(a, b, m, k, n))          # the weights really are the rounded ones


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(7, 13, 11), (96, 130, 80), (37, 53, 71), (256, 512, 192), (8, 4096, 1024), (4096, 768, 768)])
def test_gpu_fp16_weight_gemm(be, m, n, k):
    rng = np.random.default_rng(m + n + k)
    a = rng.standard_normal((m, k)).astype(np.float32); b = (rng.standard_normal((k, n)) / math.sqrt(k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    bb, br = round_to(b, "f16")
    W = be.WrapTensor
    c = torch.full((m * n,), 3.0e30, device="cuda")
    be.GemmFp16WeightB(W(dev(a)), W(from_bits16(bb, torch.float16)), None, W(c), m, n, k)
    got = c.cpu().numpy().reshape(m, n)
    truth = a.astype(np.float64) @ br.astype(np.float64)
    assert mixed_err(got, truth) <= 1e-4
    if m * n * k <= 1 << 24:
        assert mixed_err(got, oracle.sgemm_fp16_weight_b(a, bb, m, k, n)) <= 1e-4
    be.GemmFp16WeightB(W(dev(a)), W(from_bits16(bb, torch.float16)), W(dev(bias)), W(c), m, n, k, 2)
    assert mixed_err(c.cpu().numpy().reshape(m, n), act64(truth + bias[None, :], 2)) <= 1e-4


@pytest.mark.gpu
def test_gpu_fp16_weight_gemm_exact_on_dyadic_inputs_and_engine_route(be):
    from aidotnet.tensors_amd import Mi355Engine
    rng = np.random.default_rng(2)
    m, n, k = 128, 192, 96
    a = rng.integers(-4, 5, (m, k)).astype(np.float32) / 4; b = rng.integers(-4, 5, (k, n)).astype(np.float32) / 4
    eng = Mi355Engine(be)
    out = eng.TensorMatMulFp16WeightB(dev(a), dev(b).half())
    assert np.array_equal(out.cpu().numpy().astype(np.float64), a.astype(np.float64) @ b.astype(np.float64))
    out = eng.FusedLinearFp16WeightB(dev(a).reshape(2, 64, k), dev(b).half(), None, "ReLU")
    assert tuple(out.shape) == (2, 64, n)


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n", [(64, 128, 100), (48, 96, 96), (3, 5, 7), (1, 320, 1280)])
def test_gpu_fp16_weight_matmul_matches_upcast_then_matmul(be, m, k, n):
    """The shapes and the bound (1e-3 + 1e-4 |e|) of tests/AiDotNet.Tensors.Tests/Engines/Fp16WeightGemmTests.cs:43-73: the fused
    path and 'widen the whole weight, then MatMul' decode the same fp16 bit patterns."""
    from aidotnet.tensors_amd import Mi355Engine
    rng = np.random.default_rng(1234 + m * 31 + k * 7 + n)
    a = (rng.random((m, k)) * 2 - 1).astype(np.float32)
    w = dev((rng.random((k, n)) * 2 - 1).astype(np.float32)).half()
    eng = Mi355Engine(be)
    fused = eng.TensorMatMulFp16WeightB(dev(a), w).cpu().numpy()
    assert fused.shape == (m, n)
    upcast = eng.TensorMatMul(dev(a), w.float()).cpu().numpy()
    assert np.all(np.abs(fused - upcast) < 1e-3 + 1e-4 * np.abs(upcast))
    assert mixed_err(fused, oracle.sgemm_fp16_weight_b(a, w.cpu().view(torch.int16).numpy().view(np.uint16), m, k, n)) <= 1e-4


@pytest.mark.gpu
def test_gpu_fused_linear_fp16_weight_bias_and_rank_one_input(be):
    """Fp16WeightGemmTests.cs:75-120: bias without activation, and a rank-1 input giving a rank-1 result."""
    from aidotnet.tensors_amd import Mi355Engine
    rng = np.random.default_rng(99)
    eng = Mi355Engine(be)
    m, k, n = 32, 64, 48
    a = dev((rng.random((m, k)) * 2 - 1).astype(np.float32)); w = dev((rng.random((k, n)) * 2 - 1).astype(np.float32)).half()
    bias = dev((rng.random(n) - 0.5).astype(np.float32))
    ref = (a.cpu().double() @ w.cpu().double() + bias.cpu().double()).numpy()
    got = eng.FusedLinearFp16WeightB(a, w, bias, "None").cpu().numpy()
    assert got.shape == (m, n) and np.all(np.abs(got - ref) < 1e-3 + 1e-4 * np.abs(ref))
    k, n = 40, 24
    a1 = dev((rng.random(k) * 2 - 1).astype(np.float32)); w = dev((rng.random((k, n)) * 2 - 1).astype(np.float32)).half()
    got = eng.FusedLinearFp16WeightB(a1, w, None, "None")
    assert tuple(got.shape) == (n,)
    ref = (a1.cpu().double() @ w.cpu().double()).numpy()
    assert np.all(np.abs(got.cpu().numpy() - ref) < 1e-3 + 1e-4 * np.abs(ref))
