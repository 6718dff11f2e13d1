"""The C# binding files under bindings/csharp against include/aidotnet_mi355.h.

There is no .NET toolchain in this build image, so the binding is not compiled; this test holds it to the header instead:
every export has exactly one DllImport declaration with the same argument count, every argument and the result have the
blittable C# type the C type asks for, the descriptor struct has the header's fields in order, and every native call the backend
decorator makes exists with that many arguments.
"""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aidotnet_mi355.h")
NATIVE = os.path.join(ROOT, "bindings", "csharp", "Mi355Native.cs")
BACKEND = os.path.join(ROOT, "bindings", "csharp", "Mi355HipBackend.cs")
BF16 = os.path.join(ROOT, "bindings", "csharp", "IGpuBFloat16Backend.cs")


def _strip_c_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def _split_args(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "(<[":
            depth += 1
        elif ch in ")>]":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def header_exports():
    """name -> (return type, [argument C types]) for every AIDN_API prototype."""
    text = _strip_c_comments(open(HEADER).read())
    protos = {}
    for m in re.finditer(r"AIDN_API\s+([\w\s\*]+?)\s*\b(aidn_mi355_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        ret, name, args = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
        types = []
        if args and args != "void":
            for a in _split_args(args):
                a = a.strip()
                # drop the parameter name: the last identifier not preceded by '*' glued to it
                mm = re.match(r"^(.*?)(\b\w+)$", a)
                ctype = mm.group(1).strip() if mm and mm.group(1).strip() else a
                types.append(" ".join(ctype.replace("*", " * ").split()))
        protos[name] = (" ".join(ret.replace("*", " * ").split()), types)
    return protos


def csharp_imports():
    """name -> (return type, [argument C# types]) for every DllImport declaration."""
    text = re.sub(r"//.*", "", open(NATIVE).read())
    decls = {}
    for m in re.finditer(r"\[DllImport\([^\]]*\)\]\s*internal\s+static\s+extern\s+(\w+)\s+(\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        ret, name, args = m.group(1), m.group(2), " ".join(m.group(3).split())
        types = []
        for a in _split_args(args):
            parts = a.split()
            types.append(" ".join(parts[:-1]))      # everything but the parameter name
        assert name not in decls, "declared twice: " + name
        decls[name] = (ret, types)
    return decls


def expected_csharp(ctype, is_return=False):
    c = ctype.replace("const ", "").strip()
    if c == "void * *":
        return "out IntPtr"
    if c == "aidn_attn_desc *":
        return "ref AidnAttnDesc"
    if c.endswith("*"):
        return "IntPtr"                         # device pointers, the context, the stream, returned C strings
    return {"int": "int", "int32_t": "int", "int64_t": "long", "uint64_t": "ulong", "float": "float"}[c]


def test_every_export_is_bound_with_matching_blittable_types():
    exports, imports = header_exports(), csharp_imports()
    assert len(exports) >= 50
    missing = sorted(set(exports) - set(imports))
    extra = sorted(set(imports) - set(exports))
    assert not missing, "exports without a DllImport declaration: %s" % missing
    assert not extra, "DllImport declarations without an export: %s" % extra
    for name, (ret, args) in exports.items():
        cs_ret, cs_args = imports[name]
        assert cs_ret == expected_csharp(ret, True), "%s returns %s in C, %s in C#" % (name, ret, cs_ret)
        assert len(cs_args) == len(args), "%s takes %d arguments in C, %d in C#" % (name, len(args), len(cs_args))
        for i, (c, cs) in enumerate(zip(args, cs_args)):
            assert cs == expected_csharp(c), "%s argument %d: C %r wants %s, C# has %s" % (name, i, c, expected_csharp(c), cs)


def test_binding_matches_the_library_symbols():
    # the header is what tests/test_abi.py holds against the built library; here: the same names through the Python loader's table
    from aidotnet.tensors_amd import _lib
    assert set(csharp_imports()) == set(_lib.SIGNATURES)


def test_descriptor_struct_has_the_header_fields_in_order():
    text = _strip_c_comments(open(HEADER).read())
    body = re.search(r"typedef struct aidn_attn_desc \{(.*?)\} aidn_attn_desc;", text, flags=re.S).group(1)
    c_fields = []
    for line in body.split(";"):
        line = " ".join(line.split())
        if not line:
            continue
        ctype, names = line.split(" ", 1)
        for n in names.split(","):
            n = n.strip()
            mm = re.match(r"(\w+)\[(\d+)\]", n)
            c_fields += [ctype] * int(mm.group(2)) if mm else [ctype]
    cs = re.sub(r"//.*", "", open(NATIVE).read())
    sbody = re.search(r"struct AidnAttnDesc\s*\{(.*?)\}", cs, flags=re.S).group(1)
    cs_fields = []
    for line in sbody.split(";"):
        line = " ".join(line.split())
        if not line:
            continue
        mm = re.match(r"public (\w+) (.*)", line)
        cs_fields += [mm.group(1)] * len(mm.group(2).split(","))
    want = [{"int32_t": "int", "float": "float", "int64_t": "long"}[t] for t in c_fields]
    assert cs_fields == want
    assert "LayoutKind.Sequential" in cs
    # 12 four-byte fields then 13 eight-byte ones: no padding in either language
    assert want[:12].count("long") == 0 and all(t == "long" for t in want[12:]) and len(want) == 25


def test_backend_calls_only_declared_entry_points_with_the_declared_argument_count():
    imports = csharp_imports()
    text = re.sub(r"//.*", "", open(BACKEND).read())
    calls = 0
    for m in re.finditer(r"Mi355Native\.(aidn_mi355_\w+)\s*\(", text):
        name = m.group(1)
        assert name in imports, "backend calls undeclared " + name
        # the argument list up to the matching parenthesis
        i, depth = m.end(), 1
        while depth:
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        args = _split_args(text[m.end():i - 1])
        assert len(args) == len(imports[name][1]), "%s called with %d arguments, declared with %d" % (name, len(args), len(imports[name][1]))
        calls += 1
    assert calls >= 25


def test_backend_overrides_the_members_of_the_path():
    text = open(BACKEND).read()
    for member in ("Gemm", "MatMulTransposed", "BatchedGemm", "GemmBias", "GemmBiasRelu", "GemmBiasGelu", "GemmBiasSigmoid", "GemmBiasTanh",
                   "GemmBiasSwish", "GemmBiasLeakyRelu", "ScaledDotProductAttention", "FlashAttentionV2", "FlashAttention", "RopeInterleaved",
                   "PagedAttentionDecode", "PagedAttentionDecodeGqa", "PagedAttentionPrefill", "PagedAttentionPrefillGqa", "ConvertToFp16",
                   "ConvertToFp32", "Synchronize"):
        assert re.search(r"public override [\w<>\?]+ %s\(" % member, text), "no override of " + member
    for member in ("Hgemm", "GemmFp16In32fOut", "Bf16Gemm", "GemmBf16In32fOut", "FlashDecode", "FlashAttentionReducedPrecision",
                   "DecodeAttentionReducedPrecision", "GetPrecisionCapabilities"):
        assert re.search(r"public [\w<>\?]+ %s\(" % member, text), "no member " + member
    # the bottom-right causal rule, the two mask modes, grouped-query heads and the decode strides are spelled out, not sketched
    assert "CausalQueryOffset = seqK - seqQ" in text and "MaskMode = mask == null ? 0 : (mask.Size >= wElems ? 2 : 1)" in text
    assert "KStride2 = (long)kvHeads * headDim" in text and "..." not in text
    # every member of the bf16 interface is implemented by the decorator
    iface = open(BF16).read()
    for m in re.finditer(r"^\s+(?:void|bool) (\w+)[ \(]", iface, flags=re.M):
        assert re.search(r"public (?:void|bool) %s\b" % m.group(1), text), "decorator lacks " + m.group(1)
