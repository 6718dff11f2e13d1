"""The precision planner and the engine routes that consult it: ``GpuPrecisionPlanner.CreatePlan`` under a
``GpuExecutionPolicyScope`` (src/AiDotNet.Tensors/Engines/Gpu/GpuPrecisionPolicy.cs:331-381, 511-551), ``ExecutePlannedGemm`` /
``ExecutePlannedBatchedGemm`` (src/AiDotNet.Tensors/Engines/DirectGpuTensorEngine.cs:19547-19624) and ``TensorMatMulTransposed``
(src/AiDotNet.Tensors/Engines/CpuEngine.cs:12337-12452, DirectGpuTensorEngine.cs:19860-19905).

The planning rules follow the reference's own planner tests in spirit (explicit Float16 on fp32 data selects fp16 storage with
fp32 accumulation and output; Throw refuses what UseHigherPrecision resolves to Float32; PreserveInputType never narrows).
"""
import numpy as np
import pytest
import torch

import oracle
from _util import dev, mixed_err, round_to
from aidotnet.tensors_amd import (ArgumentException, ArgumentNullException, GpuAccuracyMode, GpuComputePreference, GpuExecutionPolicy,
                                  GpuExecutionPolicyScope, GpuExecutionRoute, GpuPrecisionDiagnostics, GpuPrecisionFallbackBehavior,
                                  GpuPrecisionOperation, GpuPrecisionPlanner, GpuScalarType, NotSupportedException)

Op, Pref, ST = GpuPrecisionOperation, GpuComputePreference, GpuScalarType


def plan(dtype, op=Op.MatMul, **policy):
    if not policy:
        return GpuPrecisionPlanner.CreatePlan(dtype, op, "test")
    with GpuExecutionPolicyScope(GpuExecutionPolicy(**policy)):
        return GpuPrecisionPlanner.CreatePlan(dtype, op, "test")


def test_auto_keeps_reduced_public_types_and_maps_the_rest_to_float32():
    p = plan(torch.float32)
    assert (p.Route, p.InputStorage, p.AccumulatorType, p.OutputStorage, p.FallbackReason) == (GpuExecutionRoute.Gpu, ST.Float32, ST.Float32, ST.Float32, None)
    for dt, st in ((torch.float16, ST.Float16), (torch.bfloat16, ST.BFloat16)):
        p = plan(dt)
        assert (p.InputStorage, p.MultiplyType, p.AccumulatorType, p.OutputStorage, p.ReducesStorageBytes) == (st, st, ST.Float32, ST.Float32, True)
        assert p.FallbackReason is None and p.PublicType == st
    p = plan(torch.float64)                                     # every other public type runs on the fp32 boundary, and says so
    assert p.InputStorage == ST.Float32 and "Auto converts public Float64 through Float32" in p.FallbackReason
    assert plan(torch.int32).InputStorage == ST.Float32          # Generic


def test_explicit_preference_fallbacks_and_throw():
    p = plan(torch.float32, ComputePreference=Pref.Float16)
    assert (p.InputStorage, p.AccumulatorType, p.OutputStorage, p.RequestedPreference) == (ST.Float16, ST.Float32, ST.Float32, Pref.Float16)
    assert plan(torch.float32, ComputePreference=Pref.BFloat16).InputStorage == ST.BFloat16
    assert plan(torch.float16, ComputePreference=Pref.Float32).InputStorage == ST.Float32
    # fp8 is not executed: BFloat16 is the first safe fallback; TensorFloat32 falls to Float32; Float64 has no fallback
    p = plan(torch.float32, ComputePreference=Pref.Float8E4M3)
    assert p.InputStorage == ST.BFloat16 and "Requested Float8E4M3 is unavailable" in p.FallbackReason
    assert plan(torch.float32, ComputePreference=Pref.TensorFloat32).InputStorage == ST.Float32
    with pytest.raises(NotSupportedException):
        plan(torch.float32, ComputePreference=Pref.Float64)
    with pytest.raises(NotSupportedException):
        plan(torch.float32, ComputePreference=Pref.Float8E5M2, FallbackBehavior=GpuPrecisionFallbackBehavior.Throw)
    # the batched and transposed contracts are fp32 only
    for op in (Op.BatchMatMul, Op.MatMulTransposed):
        p = plan(torch.float32, op, ComputePreference=Pref.Float16)
        assert p.InputStorage == ST.Float32 and "Requested Float16 is unavailable" in p.FallbackReason
        with pytest.raises(NotSupportedException):
            plan(torch.float32, op, ComputePreference=Pref.Float16, FallbackBehavior=GpuPrecisionFallbackBehavior.Throw)
        assert plan(torch.float16, op).InputStorage == ST.Float32
    with pytest.raises(NotSupportedException):
        plan(torch.float32, Op.Convolution)                      # nothing advertised: the reference would plan its CPU route
    with pytest.raises(ArgumentException):
        GpuPrecisionPlanner.CreatePlan(torch.float32, Op.MatMul, "  ")


def test_preserve_input_type_never_narrows():
    assert plan(torch.float32, AccuracyMode=GpuAccuracyMode.PreserveInputType, ComputePreference=Pref.Float16).InputStorage == ST.Float32
    assert plan(torch.float16, AccuracyMode=GpuAccuracyMode.PreserveInputType).InputStorage == ST.Float16     # fp32 accumulate/output widen only
    with pytest.raises(NotSupportedException):
        plan(torch.float64, AccuracyMode=GpuAccuracyMode.PreserveInputType)
    with pytest.raises(NotSupportedException):
        plan(torch.float16, Op.BatchMatMul, AccuracyMode=GpuAccuracyMode.PreserveInputType)


def test_scopes_nest_and_restore():
    assert GpuExecutionPolicyScope.Current() is None and GpuExecutionPolicyScope.CurrentPolicy() is GpuExecutionPolicy.Default
    with GpuExecutionPolicyScope(GpuExecutionPolicy(ComputePreference=Pref.Float16)) as outer:
        with GpuExecutionPolicyScope(GpuExecutionPolicy.Preserve):
            assert GpuExecutionPolicyScope.CurrentPolicy().AccuracyMode == GpuAccuracyMode.PreserveInputType
        assert GpuExecutionPolicyScope.Current() is outer and GpuExecutionPolicyScope.CurrentPolicy().ComputePreference == Pref.Float16
        outer.Dispose(); outer.Dispose()                         # idempotent
        assert GpuExecutionPolicyScope.Current() is None
    with pytest.raises(ArgumentNullException):
        GpuExecutionPolicyScope(None)
    seen = []
    observer = seen.append
    GpuPrecisionDiagnostics.PlanExecuted.append(observer)
    try:
        GpuPrecisionDiagnostics.Clear()
        assert GpuPrecisionDiagnostics.LastPlan() is None
        p = plan(torch.float32)
        GpuPrecisionDiagnostics.Publish(p)
        assert GpuPrecisionDiagnostics.LastPlan() is p and seen == [p]
    finally:
        GpuPrecisionDiagnostics.PlanExecuted.remove(observer)


# ----------------------------------------------------------------------------------------------------------------- GPU
@pytest.fixture(scope="module")
def eng():
    from aidotnet.tensors_amd import Mi355Backend, Mi355Engine
    b = Mi355Backend()
    yield Mi355Engine(b)
    b.Dispose()


def rnd(shape, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("kind,pref", [("f16", Pref.Float16), ("bf16", Pref.BFloat16)])
def test_planned_gemm_converts_fp32_operands_and_matches_the_oracle_chain(eng, kind, pref):
    m, k, n = 96, 320, 200
    a = rnd((3, 32, k), 1); b = rnd((k, n), 2, 0.1)
    GpuPrecisionDiagnostics.Clear()
    with GpuExecutionPolicyScope(GpuExecutionPolicy(ComputePreference=pref)):
        out = eng.TensorMatMul(dev(a), dev(b))
    p = GpuPrecisionDiagnostics.LastPlan()
    assert p.Operation == "TensorMatMul.NDx2D" and p.InputStorage == {"f16": ST.Float16, "bf16": ST.BFloat16}[kind]
    assert out.dtype == torch.float32 and tuple(out.shape) == (3, 32, n)
    # the same chain on the CPU: round both operands to the storage type, multiply with fp32 accumulation, keep the fp32 result
    ab, ar = round_to(a.reshape(m, k), kind); bb, br = round_to(b, kind)
    _, o32 = (oracle.hgemm if kind == "f16" else oracle.bf16gemm)(ab, bb, m, k, n)
    got = out.cpu().numpy().reshape(m, n)
    assert mixed_err(got, o32) <= 1e-4
    assert mixed_err(got, ar.astype(np.float64) @ br.astype(np.float64)) <= 1e-4
    # and it is a different number from the fp32 product: the plan really ran in the reduced format
    assert mixed_err(got, a.reshape(m, k).astype(np.float64) @ b.astype(np.float64)) > 1e-4


@pytest.mark.gpu
def test_planned_gemm_float32_preference_on_half_tensors_and_default_routes(eng):
    m, k, n = 64, 256, 128
    a = rnd((m, k), 3); b = rnd((k, n), 4, 0.1)
    ab, ar = round_to(a, "f16"); bb, br = round_to(b, "f16")
    from _util import bits16, from_bits16
    A, B = from_bits16(ab, torch.float16), from_bits16(bb, torch.float16)
    with GpuExecutionPolicyScope(GpuExecutionPolicy(ComputePreference=Pref.Float32)):
        out = eng.TensorMatMul(A, B)
    assert GpuPrecisionDiagnostics.LastPlan().InputStorage == ST.Float32 and out.dtype == torch.float16
    want = oracle.f32_to_f16(oracle.sgemm(ar, br, m, k, n))
    assert np.max(np.abs(oracle.f16_to_f32(bits16(out)) - oracle.f16_to_f32(want))) <= 2e-2 * (1 + np.abs(oracle.f16_to_f32(want)).max())
    assert mixed_err(oracle.f16_to_f32(bits16(out)), ar.astype(np.float64) @ br.astype(np.float64)) <= 2e-2
    # default policy: the 16-bit route, result in the operands' dtype; equals the fp32-output route rounded once
    out16 = eng.TensorMatMul(A, B)
    assert GpuPrecisionDiagnostics.LastPlan().InputStorage == ST.Float16 and out16.dtype == torch.float16
    out32 = eng.TensorMatMul(A, B, out_dtype=torch.float32)
    assert np.array_equal(bits16(out16), oracle.f32_to_f16(out32.cpu().numpy()))
    # a batched product ignores a reduced preference (fp32 contract) unless the policy says Throw
    x = rnd((4, 32, 48), 5); y = rnd((4, 48, 40), 6)
    with GpuExecutionPolicyScope(GpuExecutionPolicy(ComputePreference=Pref.Float16)):
        o = eng.TensorMatMul(dev(x), dev(y))
    assert GpuPrecisionDiagnostics.LastPlan().Operation == "BatchMatMul" and GpuPrecisionDiagnostics.LastPlan().InputStorage == ST.Float32
    assert mixed_err(o.cpu().numpy(), x.astype(np.float64) @ y.astype(np.float64)) <= 1e-4
    with GpuExecutionPolicyScope(GpuExecutionPolicy(ComputePreference=Pref.Float16, FallbackBehavior=GpuPrecisionFallbackBehavior.Throw)):
        with pytest.raises(NotSupportedException):
            eng.TensorMatMul(dev(x), dev(y))


@pytest.mark.gpu
def test_tensor_matmul_transposed(eng):
    m, k, n = 70, 130, 45
    a = rnd((m, k), 7); b = rnd((n, k), 8)
    out = eng.TensorMatMulTransposed(dev(a), dev(b))
    assert tuple(out.shape) == (m, n) and out.dtype == torch.float32
    want = oracle.sgemm_ex(a, k, False, b, k, True, m, k, n)          # SimdGemm.Sgemm(..., transB: true), the reference's fp32 fast path
    assert mixed_err(out.cpu().numpy(), want) <= 1e-4
    assert mixed_err(out.cpu().numpy(), a.astype(np.float64) @ b.astype(np.float64).T) <= 1e-4
    assert GpuPrecisionDiagnostics.LastPlan().Operation == "TensorMatMulTransposed"
    # equals TensorMatMul on the materialised transpose
    assert mixed_err(out.cpu().numpy(), eng.TensorMatMul(dev(a), dev(np.ascontiguousarray(b.T))).cpu().numpy()) <= 1e-5
    # rank 3: transpose + batched TensorMatMul
    a3 = rnd((3, 20, 33), 9); b3 = rnd((3, 17, 33), 10)
    o3 = eng.TensorMatMulTransposed(dev(a3), dev(b3))
    assert tuple(o3.shape) == (3, 20, 17)
    assert mixed_err(o3.cpu().numpy(), np.einsum("bmk,bnk->bmn", a3.astype(np.float64), b3.astype(np.float64))) <= 1e-4
    # 16-bit tensors: widened on the device, fp32 product, one rounding back
    from _util import bits16, from_bits16
    ab, ar = round_to(a, "bf16"); bb, br = round_to(b, "bf16")
    o16 = eng.TensorMatMulTransposed(from_bits16(ab, torch.bfloat16), from_bits16(bb, torch.bfloat16))
    assert o16.dtype == torch.bfloat16
    assert mixed_err(oracle.bf16_to_f32(bits16(o16)), ar.astype(np.float64) @ br.astype(np.float64).T) <= 2e-2
    # argument rules
    with pytest.raises(ArgumentNullException):
        eng.TensorMatMulTransposed(None, dev(b))
    with pytest.raises(ArgumentException, match="K mismatch"):
        eng.TensorMatMulTransposed(dev(a), dev(rnd((n, k + 1), 1)))
    with pytest.raises(ArgumentException, match="rank >= 2"):
        eng.TensorMatMulTransposed(dev(a[0]), dev(b))
