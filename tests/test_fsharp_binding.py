"""CPU: static cross-check of the F# glue (deepnet_amd/fsharp/Hip/*.fs, source only: no .NET SDK here) against the C header it
binds and against the reference interface it implements.

  * every DllImport of HipNative.fs names a symbol include/tensor_hip.h declares, with the same number of arguments, each of the
    matching kind (descriptor by reference, pointer, pointer by reference, int32, int32 by reference, size_t, array of descriptor
    pointers, byte buffer);
  * its DnhTensor struct has the header's fields in the header's order at the header's offsets (152 bytes);
  * its Status and DType enums carry the header's values;
  * the op codes HipBackend.fs passes (unary 0..21, binary 0..10, compare 0..5, reduce 0..6, arg-reduce 0..1) are the header's
    enum values for the member of that name;
  * HipBackend.fs implements every abstract member of ITensorBackend<'T> (Tensor/Tensor/TensorBackend.fs:64-146; the member list is
    the committed fixture tests/golden/itensorbackend_members.json) with the reference's argument count.
"""
import ctypes as C
import json
import os
import re

import pytest

from deepnet_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "tensor_hip.h")).read()
NATIVE = open(os.path.join(ROOT, "deepnet_amd", "fsharp", "Hip", "HipNative.fs")).read()
BACKEND = open(os.path.join(ROOT, "deepnet_amd", "fsharp", "Hip", "HipBackend.fs")).read()


def _strip_c_comments(text):
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def c_kind(param):
    """Kind of one C parameter declaration."""
    p = re.sub(r"\s+", " ", param.strip())
    ty = p.rsplit(" ", 1)[0] if " " in p else p     # drop the parameter name
    if p.endswith("*"):
        ty = p
    ty = ty.replace(" *", "*")
    table = {
        "const DnhTensor*": "desc", "const DnhTensor* const*": "descarray",
        "void*": "ptr", "const void*": "ptr", "void**": "ptrref",
        "int32_t": "i32", "int32_t*": "i32ref", "size_t": "size", "int64_t": "i64", "size_t*": "sizeref",
        "char*": "bytes", "const char*": "bytes", "float*": "f32ref",
        "DnhDeviceInfo*": "structref", "DnhPoolStats*": "structref",
    }
    assert ty in table, f"unclassified C parameter '{param}' (type '{ty}')"
    return table[ty]


def header_functions():
    text = _strip_c_comments(HEADER)
    out = {}
    for m in re.finditer(r"int32_t\s+(dnh_\w+)\s*\(([^)]*)\)\s*;", text):
        params = m.group(2).strip()
        kinds = [] if params in ("", "void") else [c_kind(p) for p in params.split(",")]
        out[m.group(1)] = kinds
    return out


def fs_kind(param):
    p = param.strip()
    ty = p.rsplit(" ", 1)[0].strip()
    table = {"DnhTensor&": "desc", "nativeint[]": "descarray", "nativeint": "ptr", "nativeint&": "ptrref", "int": "i32", "int&": "i32ref",
             "unativeint": "size", "byte[]": "bytes", "int64": "i64", "unativeint&": "sizeref"}
    assert ty in table, f"unclassified F# parameter '{param}'"
    return table[ty]


def fs_imports():
    out = []
    pat = re.compile(r"\[<DllImport\(Lib, CallingConvention=CallingConvention\.Cdecl(?:, EntryPoint=\"(\w+)\")?\)>\]\s*extern int (\w+) \(([^)]*)\)")
    for m in pat.finditer(NATIVE):
        params = m.group(3).strip()
        out.append({"name": m.group(2), "entry": m.group(1) or m.group(2), "kinds": [] if not params else [fs_kind(p) for p in params.split(",")]})
    return out


def test_every_dllimport_matches_a_declared_entry_point():
    decl = header_functions()
    imports = fs_imports()
    assert len(imports) >= 35
    assert NATIVE.count("DllImport(") == len(imports), "a DllImport line was not parsed"
    for imp in imports:
        assert imp["entry"] in decl, f"{imp['name']} binds {imp['entry']}, which include/tensor_hip.h does not declare"
        want, got = decl[imp["entry"]], imp["kinds"]
        assert len(want) == len(got), (imp["name"], want, got)
        for k, (w, g) in enumerate(zip(want, got)):
            # an alias that passes NULL for optional descriptors (dnh_batched_svd_values) declares them as plain pointers
            ok = w == g or (imp["name"] != imp["entry"] and w == "desc" and g == "ptr")
            assert ok, f"{imp['name']} argument {k}: header has {w}, F# has {g}"
    # every product entry point the backend needs is bound
    bound = {imp["entry"] for imp in imports}
    for op in list(abi.OP_SIGNATURES) + list(abi.LAPACK_OP_SIGNATURES):
        assert "dnh_" + op in bound, f"dnh_{op} has no DllImport"


def test_library_exports_what_the_dllimports_name():
    from deepnet_amd import native
    lib = native.load()
    for imp in fs_imports():
        assert hasattr(lib, imp["entry"])


def test_descriptor_struct_has_the_headers_fields():
    body = NATIVE[NATIVE.index("type internal DnhTensor ="):NATIVE.index("member this.SetShape")]
    fields = re.findall(r"val mutable (\w+):\s*(\w+)", body)
    size = {"nativeint": 8, "int64": 8, "int32": 4}
    want_names = ["Base", "Offset", "NDims", "DType"] + [f"Shape{i}" for i in range(8)] + [f"Stride{i}" for i in range(8)]
    assert [f[0] for f in fields] == want_names
    assert "LayoutKind.Sequential" in NATIVE[:NATIVE.index("type internal DnhTensor =")].rsplit("[<Struct", 1)[1]
    # sequential layout with natural alignment
    off, offsets = 0, {}
    for name, ty in fields:
        s = size[ty]
        off = (off + s - 1) // s * s
        offsets[name] = off
        off += s
    total = (off + 7) // 8 * 8
    T = abi.DnhTensor                     # tests/test_abi.py checks this ctypes struct against the header as gcc compiles it
    assert total == C.sizeof(T) == 152
    assert offsets["Base"] == T.base.offset and offsets["Offset"] == T.offset.offset
    assert offsets["NDims"] == T.ndims.offset and offsets["DType"] == T.dtype.offset
    assert offsets["Shape0"] == T.shape.offset and offsets["Stride0"] == T.stride.offset
    assert offsets["Shape7"] == T.shape.offset + 56 and offsets["Stride7"] == T.stride.offset + 56
    assert dict(fields)["Base"] == "nativeint" and dict(fields)["NDims"] == "int32" and dict(fields)["DType"] == "int32"
    # the header's own text: 4 scalar fields + two arrays of DNH_MAX_DIMS = 8
    struct = _strip_c_comments(HEADER)
    struct = struct[struct.index("typedef struct DnhTensor {"):struct.index("} DnhTensor;")]
    assert [n for _, n in re.findall(r"([\w\*]+)\s+(\w+)(?:\[DNH_MAX_DIMS\])?;", struct)] == ["base", "offset", "ndims", "dtype", "shape", "stride"]
    assert "#define DNH_MAX_DIMS 8" in HEADER


def header_enum(name):
    text = _strip_c_comments(HEADER)
    body = text[text.index(f"typedef enum {name} {{") + len(f"typedef enum {name} {{"):text.index(f"}} {name};")]
    vals, nxt = {}, 0
    for item in body.split(","):
        item = item.strip()
        if not item:
            continue
        if "=" in item:
            k, v = [x.strip() for x in item.split("=")]
            nxt = int(v)
        else:
            k = item
        vals[k] = nxt
        nxt += 1
    return vals


def _norm(s):
    return re.sub(r"^(DNH_ERR_|DNH_)", "", s).replace("_", "").lower()


def fs_enum(name):
    body = NATIVE[NATIVE.index(f"type internal {name} ="):]
    body = body[:body.index("\n\n")]
    return {k: int(v) for k, v in re.findall(r"\|\s*(\w+)\s*=\s*(\d+)", body)}


def test_status_and_dtype_enums_carry_the_headers_values():
    hs = {_norm(k): v for k, v in header_enum("DnhStatus").items()}
    fs = {k.lower(): v for k, v in fs_enum("Status").items()}
    assert fs == hs
    hd = {_norm(k): v for k, v in header_enum("DnhDType").items() if k != "DNH_DTYPE_COUNT"}
    fd = {k.lower(): v for k, v in fs_enum("DType").items()}
    assert fd == hd
    # the Python mirror too
    assert abi.DNH_F64 == hd["f64"] and abi.DNH_U16 == hd["u16"] and abi.DNH_ERR_NO_CONVERGENCE == hs["noconvergence"]


@pytest.mark.parametrize("helper,enum,suffix", [
    ("unary", "DnhUnaryOp", ""), ("binary", "DnhBinaryOp", ""), ("compare", "DnhCompareOp", ""),
    ("reduce", "DnhReduceOp", "LastAxis"), ("argReduce", "DnhArgReduceOp", "LastAxis"),
])
def test_op_codes_in_the_backend_are_the_headers_enum_values(helper, enum, suffix):
    want = {_norm(k): v for k, v in header_enum(enum).items() if not k.endswith("_COUNT")}
    got = {}
    for name, code in re.findall(r"member this\.(\w+) \([^)]*\) = " + helper + r" (\d+) ", BACKEND):
        key = name[:-len(suffix)] if suffix and name.endswith(suffix) else name
        got[key.lower()] = int(code)
    assert got == want, (sorted(set(want) ^ set(got)), {k: (want.get(k), got.get(k)) for k in want if want.get(k) != got.get(k)})


def test_backend_implements_every_member_of_the_reference_interface():
    fixture = json.load(open(os.path.join(ROOT, "tests", "golden", "itensorbackend_members.json")))
    members = fixture["members"]
    assert len(members) == 69
    body = BACKEND[BACKEND.index("interface ITensorBackend<'T> with"):BACKEND.index("and internal HipTransfer")]
    impl = {}
    for m in re.finditer(r"^\s+member this\.(\w+)\s*(\(([^)]*)\))?", body, flags=re.M):
        args = m.group(3)
        impl[m.group(1)] = None if args is None else (0 if not args.strip() else len([a for a in _split_top(args)]))
    for mem in members:
        assert mem["name"] in impl, f"HipBackend.fs lacks ITensorBackend.{mem['name']}"
        if mem["property"]:
            assert "with get idx" in body and "and set idx value" in body
        else:
            assert impl[mem["name"]] == mem["args"], (mem["name"], impl[mem["name"]], mem["args"])
    extra = set(impl) - {m["name"] for m in members}
    assert not extra, f"members the reference interface does not have: {extra}"


def _split_top(args):
    """Splits an F# tuple pattern at top-level commas (type annotations may hold commas inside angle brackets or parentheses)."""
    depth, cur, out = 0, "", []
    for ch in args:
        if ch in "(<":
            depth += 1
        elif ch in ")>":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    out.append(cur)
    return out
