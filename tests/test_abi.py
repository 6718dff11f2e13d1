"""CPU-side checks of the drop-in boundary: the shared library is built in-tree, loads, and exports
exactly the symbols include/aidotnet_mi355.h declares; the ctypes table and descriptor layout match
the header.  No compute call is made (no GPU here)."""
import ctypes
import os
import re
import subprocess

import pytest

import aidotnet.tensors_amd as pkg
from aidotnet.tensors_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aidotnet_mi355.h")


def _declared():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"AIDN_API\s+(?:const\s+char\*|int|uint64_t)\s+(aidn_mi355_\w+)\s*\(", text)))


def test_library_exists_in_tree():
    assert os.path.exists(_lib.LIB_PATH), "build with `python -m aidotnet.tensors_amd.build`"
    assert os.path.dirname(_lib.LIB_PATH).startswith(ROOT)


def test_header_declarations_are_all_exported_and_bound():
    declared = _declared()
    assert len(declared) >= 20
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(set(re.findall(r" T (aidn_mi355_\w+)", out)))
    assert exported == declared
    assert sorted(_lib.SIGNATURES) == declared
    lib = pkg.load_library()
    for name in declared:
        assert getattr(lib, name) is not None
    assert b"gfx950" in lib.aidn_mi355_version()


def test_header_cites_reference_interface_for_every_entry_point_group():
    text = open(HEADER).read()
    for needle in ("IDirectGpuBackend.cs", "IGpuHalfPrecisionBackend.cs", "HipBackend.cs", "CpuEngine.cs",
                   "BFloat16.cs", "HipAttentionKernels.cs"):
        assert needle in text


def test_descriptor_layout_matches_header():
    # struct of 6 int32, float, 2 int32, float, 2 int32, then int64 + 4 * int64[3]
    d = _lib.AttnDesc
    assert ctypes.sizeof(d) == 12 * 4 + 8 + 12 * 8
    assert d.bias_batch_stride.offset == 48
    assert d.q_strides.offset == 56 and d.o_strides.offset == 56 + 3 * 24
    text = open(HEADER).read()
    body = text[text.index("typedef struct aidn_attn_desc"):text.index("} aidn_attn_desc;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"\b(B|H|Hkv|Sq|Sk|D|scale|causal|causal_query_offset|softcap|mask_mode|out_is_16bit|bias_batch_stride|q_strides|k_strides|v_strides|o_strides)\b(?=[,;\[])", body)
    assert fields == [f[0] for f in d._fields_]


def test_backend_refuses_to_run_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(pkg.InvalidOperationException):
        pkg.Mi355Backend()


def test_no_product_module_imports_the_oracle():
    pkgdir = os.path.join(ROOT, "aidotnet")
    for dp, _, files in os.walk(pkgdir):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                src = open(os.path.join(dp, f), errors="replace").read()
                assert "import oracle" not in src and "liboracle" not in src and "from oracle" not in src, f


def test_build_rejects_kernels_that_spill():
    """The build parses hipcc's resource-usage remarks and refuses a kernel that needs scratch memory."""
    from aidotnet.tensors_amd.build import kernels_with_scratch
    remarks = """a.hip:1:1: remark: Function Name: _ZN4aidn3fooEv [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     VGPRs: 17 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:9:1: remark: Function Name: _ZN4aidn3barEv [-Rpass-analysis=kernel-resource-usage]
a.hip:9:1: remark:     ScratchSize [bytes/lane]: 576 [-Rpass-analysis=kernel-resource-usage]
"""
    assert kernels_with_scratch(remarks) == [("_ZN4aidn3barEv", 576)]
    assert kernels_with_scratch("") == []
