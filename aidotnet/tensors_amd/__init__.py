"""MI355X-native GEMM and fused attention behind AiDotNet.Tensors' GPU-backend slot.

``Mi355Backend`` mirrors the backend-slot members on the hot path, ``Mi355Engine`` the operator
API above it; both need ``libaidotnet_mi355.so`` (``python -m aidotnet.tensors_amd.build``) and a
gfx950 device.  There is no fallback path.
"""
from ._lib import LIB_PATH, SIGNATURES, AttnDesc, load as load_library
from .backend import (ArgumentException, ArgumentNullException, ArgumentOutOfRangeException, GpuBuffer,
                      HipException, InvalidOperationException, Mi355Backend, NotSupportedException)
from .engine import Mi355Engine
from .precision import (GpuAccuracyMode, GpuComputePlan, GpuComputePreference, GpuExecutionPolicy, GpuExecutionPolicyScope,
                        GpuExecutionRoute, GpuPrecisionCapability, GpuPrecisionDiagnostics, GpuPrecisionFallbackBehavior,
                        GpuPrecisionImplementation, GpuPrecisionOperation, GpuPrecisionPlanner, GpuScalarType)

__all__ = ["Mi355Backend", "Mi355Engine", "GpuBuffer", "AttnDesc", "load_library", "LIB_PATH", "SIGNATURES",
           "ArgumentException", "ArgumentNullException", "ArgumentOutOfRangeException", "HipException",
           "InvalidOperationException", "NotSupportedException",
           "GpuAccuracyMode", "GpuComputePlan", "GpuComputePreference", "GpuExecutionPolicy", "GpuExecutionPolicyScope", "GpuExecutionRoute",
           "GpuPrecisionCapability", "GpuPrecisionDiagnostics", "GpuPrecisionFallbackBehavior", "GpuPrecisionImplementation",
           "GpuPrecisionOperation", "GpuPrecisionPlanner", "GpuScalarType"]
