"""Precision planning for the GEMM routes: the policy scope, the capability table this backend advertises and the planner that
turns (public element type, requested compute preference) into the storage / multiply / accumulate / output types of one call.

Mirrors src/AiDotNet.Tensors/Engines/Gpu/GpuPrecisionPolicy.cs: enums :13-84, ``GpuExecutionPolicy`` :91-121 and its scope
:127-155, ``GpuPrecisionCapability`` :160-190, ``GpuComputePlan`` :246-300, ``GpuPrecisionDiagnostics`` :305-322,
``GpuPrecisionPlanner.CreatePlan`` :331-381 (PreserveInputType -> exact capability or refusal; SpeedFirst -> requested format, else
``Throw`` or the safe fallbacks of :524-551; Auto keeps an explicitly reduced public type and maps everything else to Float32,
:511-522), and the HIP backend's capability table (src/AiDotNet.Tensors/Engines/Gpu/DirectGpuPrecisionCapabilities.cs:60-101:
fp32 for every GEMM operation, fp16 storage with fp32 accumulation and fp32 output for MatMul only).  Where the reference plans a
CPU route this build raises ``NotSupportedException``: there is no CPU path behind this backend.
"""
from __future__ import annotations

import contextvars
from dataclasses import dataclass
from enum import Enum
from typing import Callable, List, Optional

import torch

from .backend import ArgumentException, ArgumentNullException, NotSupportedException


class GpuAccuracyMode(Enum):
    SpeedFirst = 0
    PreserveInputType = 1


class GpuComputePreference(Enum):
    Auto = 0
    Float64 = 1
    Float32 = 2
    TensorFloat32 = 3
    BFloat16 = 4
    Float16 = 5
    Float8E4M3 = 6
    Float8E5M2 = 7


class GpuPrecisionFallbackBehavior(Enum):
    UseHigherPrecision = 0
    Throw = 1


class GpuScalarType(Enum):
    Generic = 0
    Float64 = 1
    Float32 = 2
    TensorFloat32 = 3
    BFloat16 = 4
    Float16 = 5
    Float8E4M3 = 6
    Float8E5M2 = 7


class GpuPrecisionOperation(Enum):
    General = 0
    Elementwise = 1
    Add = 2
    Relu = 3
    Gelu = 4
    MatMul = 5
    MatMulTransposed = 6
    BatchMatMul = 7
    Convolution = 8
    Reduction = 9


class GpuPrecisionImplementation(Enum):
    Native = 0
    VendorLibrary = 1
    Composite = 2
    Packed = 3
    Emulated = 4


class GpuExecutionRoute(Enum):
    Gpu = 0
    Cpu = 1


@dataclass(frozen=True)
class GpuExecutionPolicy:
    AccuracyMode: GpuAccuracyMode = GpuAccuracyMode.SpeedFirst
    ComputePreference: GpuComputePreference = GpuComputePreference.Auto
    FallbackBehavior: GpuPrecisionFallbackBehavior = GpuPrecisionFallbackBehavior.UseHigherPrecision


GpuExecutionPolicy.Default = GpuExecutionPolicy()
GpuExecutionPolicy.Preserve = GpuExecutionPolicy(GpuAccuracyMode.PreserveInputType)

_current_scope: contextvars.ContextVar = contextvars.ContextVar("aidotnet_mi355_policy_scope", default=None)


class GpuExecutionPolicyScope:
    """``with GpuExecutionPolicyScope(policy):`` — the policy of the calls inside, restored on exit; scopes nest."""

    def __init__(self, policy: GpuExecutionPolicy):
        if policy is None:
            raise ArgumentNullException("policy")
        self.Policy = policy
        self._previous = _current_scope.get()
        self._disposed = False
        _current_scope.set(self)

    @staticmethod
    def Current() -> Optional["GpuExecutionPolicyScope"]:
        return _current_scope.get()

    @staticmethod
    def CurrentPolicy() -> GpuExecutionPolicy:
        s = _current_scope.get()
        return s.Policy if s is not None else GpuExecutionPolicy.Default

    def Dispose(self) -> None:
        if not self._disposed:
            self._disposed = True
            _current_scope.set(self._previous)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.Dispose()
        return False


@dataclass(frozen=True)
class GpuPrecisionCapability:
    InputStorage: GpuScalarType
    MultiplyType: GpuScalarType
    AccumulatorType: GpuScalarType
    OutputStorage: GpuScalarType
    Implementation: GpuPrecisionImplementation
    ReducesStorageBytes: bool
    ComputeFormat: Optional[GpuScalarType] = None

    def __post_init__(self):
        if self.ComputeFormat is None:
            object.__setattr__(self, "ComputeFormat", self.InputStorage)


@dataclass(frozen=True)
class GpuComputePlan:
    Route: GpuExecutionRoute
    Backend: str
    Operation: str
    PublicType: GpuScalarType
    RequestedPreference: GpuComputePreference
    ComputeFormat: GpuScalarType
    InputStorage: GpuScalarType
    MultiplyType: GpuScalarType
    AccumulatorType: GpuScalarType
    OutputStorage: GpuScalarType
    Implementation: Optional[GpuPrecisionImplementation]
    ReducesStorageBytes: bool
    FallbackReason: Optional[str]


class GpuPrecisionDiagnostics:
    """The plan of the last executed call on this context, and an observer list (GpuPrecisionPolicy.cs:305-322)."""
    _last: contextvars.ContextVar = contextvars.ContextVar("aidotnet_mi355_last_plan", default=None)
    PlanExecuted: List[Callable[[GpuComputePlan], None]] = []

    @classmethod
    def LastPlan(cls) -> Optional[GpuComputePlan]:
        return cls._last.get()

    @classmethod
    def Clear(cls) -> None:
        cls._last.set(None)

    @classmethod
    def Publish(cls, plan: GpuComputePlan) -> None:
        cls._last.set(plan)
        for observer in list(cls.PlanExecuted):
            observer(plan)


_F32, _F16, _BF16 = GpuScalarType.Float32, GpuScalarType.Float16, GpuScalarType.BFloat16
_FP32_GEMM = GpuPrecisionCapability(_F32, _F32, _F32, _F32, GpuPrecisionImplementation.Native, False)


def mi355_capabilities(operation: GpuPrecisionOperation) -> List[GpuPrecisionCapability]:
    """What this backend executes: fp32 for MatMul / MatMulTransposed / BatchMatMul; for MatMul also fp16 and bf16 storage,
    multiplied on the matrix cores in the storage type, accumulated in fp32, fp32 output, half the operand bytes
    (the shape of the HIP backend's table, DirectGpuPrecisionCapabilities.cs:60-101, plus the bf16 row this backend adds)."""
    if operation == GpuPrecisionOperation.MatMul:
        return [_FP32_GEMM,
                GpuPrecisionCapability(_F16, _F16, _F32, _F32, GpuPrecisionImplementation.Native, True),
                GpuPrecisionCapability(_BF16, _BF16, _F32, _F32, GpuPrecisionImplementation.Native, True)]
    if operation in (GpuPrecisionOperation.MatMulTransposed, GpuPrecisionOperation.BatchMatMul):
        return [_FP32_GEMM]
    return []


_SCALAR_OF_DTYPE = {torch.float64: GpuScalarType.Float64, torch.float32: _F32, torch.float16: _F16, torch.bfloat16: _BF16}
_SCALAR_OF_PREFERENCE = {GpuComputePreference.Float64: GpuScalarType.Float64, GpuComputePreference.Float32: _F32,
                         GpuComputePreference.TensorFloat32: GpuScalarType.TensorFloat32, GpuComputePreference.BFloat16: _BF16,
                         GpuComputePreference.Float16: _F16, GpuComputePreference.Float8E4M3: GpuScalarType.Float8E4M3,
                         GpuComputePreference.Float8E5M2: GpuScalarType.Float8E5M2}
_REDUCED = (_F16, _BF16, GpuScalarType.Float8E4M3, GpuScalarType.Float8E5M2)
_WIDER = {GpuScalarType.Float64: (GpuScalarType.Float64,),
          _F32: (_F32, GpuScalarType.Float64),
          _BF16: (_BF16, _F32, GpuScalarType.Float64),
          _F16: (_F16, _F32, GpuScalarType.Float64),
          GpuScalarType.Float8E4M3: (GpuScalarType.Float8E4M3, _BF16, _F16, _F32, GpuScalarType.Float64),
          GpuScalarType.Float8E5M2: (GpuScalarType.Float8E5M2, _BF16, _F16, _F32, GpuScalarType.Float64),
          GpuScalarType.TensorFloat32: (GpuScalarType.TensorFloat32, _F32, GpuScalarType.Float64)}


def scalar_type_for(dtype) -> GpuScalarType:
    return _SCALAR_OF_DTYPE.get(dtype, GpuScalarType.Generic)


def _automatic_type_for(source: GpuScalarType) -> GpuScalarType:
    return source if source in _REDUCED else _F32


def _safe_fallbacks(requested: GpuScalarType):
    if requested in (GpuScalarType.Float8E4M3, GpuScalarType.Float8E5M2):
        return (_BF16, _F16, _F32)
    if requested in (_BF16, _F16, GpuScalarType.TensorFloat32, GpuScalarType.Generic):
        return (_F32,)
    return ()                       # Float64 has no higher fallback; Float32 needs none


def _does_not_narrow(source: GpuScalarType, physical: GpuScalarType) -> bool:
    return physical in _WIDER.get(source, (source,))


class GpuPrecisionPlanner:
    @staticmethod
    def CreatePlan(dtype, operation: GpuPrecisionOperation, operationName: str, backendName: str = "MI355X",
                   capabilities: Optional[List[GpuPrecisionCapability]] = None) -> GpuComputePlan:
        if not operationName or not operationName.strip():
            raise ArgumentException("Operation name required.")
        policy = GpuExecutionPolicyScope.CurrentPolicy()
        requested = policy.ComputePreference
        source = scalar_type_for(dtype)
        caps = mi355_capabilities(operation) if capabilities is None else capabilities

        def plan(cap: GpuPrecisionCapability, reason: Optional[str]) -> GpuComputePlan:
            return GpuComputePlan(GpuExecutionRoute.Gpu, backendName, operationName, source, requested, cap.ComputeFormat, cap.InputStorage,
                                  cap.MultiplyType, cap.AccumulatorType, cap.OutputStorage, cap.Implementation, cap.ReducesStorageBytes, reason)

        def find(fmt: GpuScalarType) -> Optional[GpuPrecisionCapability]:
            return next((c for c in caps if c.ComputeFormat == fmt), None)

        if policy.AccuracyMode == GpuAccuracyMode.PreserveInputType:
            exact = next((c for c in caps if c.ComputeFormat == source and c.InputStorage == source and _does_not_narrow(source, c.MultiplyType)
                          and _does_not_narrow(source, c.AccumulatorType) and _does_not_narrow(source, c.OutputStorage)), None)
            if exact is not None:
                return plan(exact, None)
            raise NotSupportedException("%s has no %s %s route required by PreserveInputType (the reference plans its CPU route here; "
                                        "this backend has none)." % (backendName, source.name, operation.name))
        desired = _automatic_type_for(source) if requested == GpuComputePreference.Auto else _SCALAR_OF_PREFERENCE[requested]
        selected = find(desired)
        if selected is not None:
            reason = ("SpeedFirst Auto converts public %s through %s." % (source.name, desired.name)
                      if requested == GpuComputePreference.Auto and source != desired else None)
            return plan(selected, reason)
        if policy.FallbackBehavior == GpuPrecisionFallbackBehavior.Throw:
            raise NotSupportedException("%s does not support requested %s for %s." % (backendName, desired.name, operationName))
        for fb in _safe_fallbacks(desired):
            selected = find(fb)
            if selected is not None:
                return plan(selected, "Requested %s is unavailable for %s; using %s." % (desired.name, operation.name, selected.ComputeFormat.name))
        raise NotSupportedException("%s exposes no eligible GPU precision for %s (the reference plans its CPU route here; this backend "
                                    "has none)." % (backendName, operation.name))
