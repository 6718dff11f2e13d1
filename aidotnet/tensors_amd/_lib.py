"""ctypes binding of ``libaidotnet_mi355.so`` (the C ABI declared in ``include/aidotnet_mi355.h``).

There is no fallback: if the shared library is missing or does not load, importing the
backend raises.  The Python layer above is the stand-in for the reference's C# P/Invoke
layer (``HipNativeBindings`` / ``HipBlasNative``).
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# the in-tree build; AIDOTNET_MI355_LIBRARY names another build of the same library (for comparing builds)
LIB_PATH = os.environ.get("AIDOTNET_MI355_LIBRARY") or os.path.join(HERE, "libaidotnet_mi355.so")

AIDN_OK = 0
AIDN_ERR_INVALID_ARGUMENT = 1001
AIDN_ERR_UNSUPPORTED = 1002
AIDN_ERR_NO_DEVICE = 1003
AIDN_ERR_OUT_OF_MEMORY = 1004
AIDN_ERR_WORKSPACE = 1005


class AttnDesc(ctypes.Structure):
    """``aidn_attn_desc`` of include/aidotnet_mi355.h (field order and types must match)."""
    _fields_ = [
        ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("Hkv", ctypes.c_int32),
        ("Sq", ctypes.c_int32), ("Sk", ctypes.c_int32), ("D", ctypes.c_int32),
        ("scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("causal_query_offset", ctypes.c_int32),
        ("softcap", ctypes.c_float),
        ("mask_mode", ctypes.c_int32),
        ("out_is_16bit", ctypes.c_int32),
        ("bias_batch_stride", ctypes.c_int64),
        ("q_strides", ctypes.c_int64 * 3),
        ("k_strides", ctypes.c_int64 * 3),
        ("v_strides", ctypes.c_int64 * 3),
        ("o_strides", ctypes.c_int64 * 3),
    ]


_vp = ctypes.c_void_p
_i = ctypes.c_int
_f = ctypes.c_float
_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_descp = ctypes.POINTER(AttnDesc)

# name -> (restype, argtypes); every symbol include/aidotnet_mi355.h declares
SIGNATURES = {
    "aidn_mi355_create": (_i, [_i, ctypes.POINTER(_vp)]),
    "aidn_mi355_destroy": (_i, [_vp]),
    "aidn_mi355_last_error": (ctypes.c_char_p, [_vp]),
    "aidn_mi355_version": (ctypes.c_char_p, []),
    "aidn_mi355_sync": (_i, [_vp, _vp]),
    "aidn_mi355_sgemm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _f, _f, _i]),
    "aidn_mi355_sgemm_batched": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _f]),
    "aidn_mi355_sgemm_bias_act": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f]),
    "aidn_mi355_hgemm_bias_act": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f]),
    "aidn_mi355_bf16gemm_bias_act": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f]),
    "aidn_mi355_mha_fwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aidn_mi355_mha_fwd_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aidn_mi355_mha_fwd_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aidn_mi355_paged_attn_decode_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "aidn_mi355_paged_attn_prefill_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f]),
    "aidn_mi355_paged_attn_decode_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "aidn_mi355_paged_attn_prefill_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f]),
    "aidn_mi355_paged_attn_decode_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "aidn_mi355_paged_attn_prefill_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f]),
    "aidn_mi355_rope_interleaved_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i]),
    "aidn_mi355_rope_interleaved_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i]),
    "aidn_mi355_rope_interleaved_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i]),
    "aidn_mi355_sgemm_f16weight": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f]),
    "aidn_mi355_hgemm_f32out": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "aidn_mi355_hgemm_f16out": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "aidn_mi355_bf16gemm_f32out": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "aidn_mi355_bf16gemm_bf16out": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "aidn_mi355_hgemm_rope": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i, _i, _i]),
    "aidn_mi355_bf16gemm_rope": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i, _i, _i]),
    "aidn_mi355_convert_f32_to_f16": (_i, [_vp, _vp, _vp, _vp, _i64]),
    "aidn_mi355_convert_f16_to_f32": (_i, [_vp, _vp, _vp, _vp, _i64]),
    "aidn_mi355_convert_f32_to_bf16": (_i, [_vp, _vp, _vp, _vp, _i64]),
    "aidn_mi355_convert_bf16_to_f32": (_i, [_vp, _vp, _vp, _vp, _i64]),
    "aidn_mi355_attn_fwd_f32": (_i, [_vp, _vp, _descp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "aidn_mi355_attn_fwd_f16": (_i, [_vp, _vp, _descp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "aidn_mi355_attn_fwd_bf16": (_i, [_vp, _vp, _descp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "aidn_mi355_attn_decode_f32": (_i, [_vp, _vp, _descp, _vp, _vp, _vp, _vp, _vp, _i]),
    "aidn_mi355_attn_decode_f16": (_i, [_vp, _vp, _descp, _vp, _vp, _vp, _vp, _vp, _i]),
    "aidn_mi355_attn_decode_bf16": (_i, [_vp, _vp, _descp, _vp, _vp, _vp, _vp, _vp, _i]),
    "aidn_mi355_attn_decode_bf16_noalloc": (_i, [_vp, _vp, _descp, _vp, _vp, _vp, _vp, _vp, _i]),
    "aidn_mi355_mha_pack_qkv": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i]),
    "aidn_mi355_mha_fwd_packed_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aidn_mi355_mha_fwd_packed_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aidn_mi355_mha_fwd_packed_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aidn_mi355_packed_b_bytes": (_u64, [_i, _i, _i, _i]),
    "aidn_mi355_pack_b": (_i, [_vp, _vp, _i, _vp, _i, _i, _i, _vp]),
    "aidn_mi355_gemm_packed_b": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f]),
    "aidn_mi355_reserve_workspace": (_i, [_vp, _vp, _u64]),
    "aidn_mi355_release_stream_workspace": (_i, [_vp, _vp]),
    "aidn_mi355_workspace_bytes": (_u64, [_vp, _vp]),
    "aidn_mi355_set_gemm_tile": (_i, [_vp, _i]),
    "aidn_mi355_set_attention_fast_path": (_i, [_vp, _i]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library and type every entry point.  Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m aidotnet.tensors_amd.build` "
                "(there is no CPU or PyTorch fallback)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)      # AttributeError if the export is missing
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
