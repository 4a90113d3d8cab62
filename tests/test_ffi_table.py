"""The Deno FFI symbol table checked in beside the header (include/karume_hip.ffi.ts) names
every function the header declares, with the arity and the FFI types the C prototypes imply.
Pure text processing: neither Deno nor a GPU is needed."""
import os
import re

import helpers
from karume_amd import _ffi

HEADER = os.path.join(helpers.ROOT, "include", "karume_hip.h")
TABLE = os.path.join(helpers.ROOT, "include", "karume_hip.ffi.ts")

# C parameter / result type -> Deno FFI type.  Opaque handles travel as "pointer"; host arrays
# and out-parameters are TypedArrays on the Deno side ("buffer"); device addresses are u64.
HANDLES = {"krm_ctx*", "krm_event*", "krm_graph*", "void*"}
SCALARS = {"int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64", "size_t": "usize",
           "float": "f32", "krm_buf": "u64"}


def ffi_type(ctype: str, is_result: bool = False, name: str = "") -> str:
    ctype = re.sub(r"\s+", " ", ctype.strip())
    ctype = re.sub(r"\s*\*", "*", ctype)
    bare = ctype.replace("const ", "")
    if name == "host":          # host memory handed over for the duration of the call
        return "buffer"
    if bare in SCALARS:
        return SCALARS[bare]
    if bare == "char*" and is_result:
        return "pointer"
    if bare in HANDLES:
        return "pointer"
    if bare.endswith("*"):
        return "buffer"
    raise AssertionError(f"no FFI type for C type '{ctype}'")


def header_prototypes():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    protos = {}
    for result, name, params in re.findall(
            r"([A-Za-z_][\w\s\*]*?)\b(krm_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        if "typedef" in result:
            continue
        args = []
        params = params.strip()
        if params and params != "void":
            for param in params.split(","):
                param = param.strip()
                ctype, pname = re.match(r"(.*?)([A-Za-z_]\w*)$", param).groups()
                args.append(ffi_type(ctype, name=pname))
        protos[name] = (args, ffi_type(result, is_result=True))
    return protos


def table_entries():
    text = open(TABLE).read()
    entries = {}
    for name, params, result in re.findall(
            r"(krm_[a-z0-9_]+):\s*\{\s*parameters:\s*\[([^\]]*)\],\s*result:\s*\"(\w+)\"", text):
        args = re.findall(r"\"(\w+)\"", params)
        entries[name] = (args, result)
    return entries


def test_ffi_table_matches_the_header():
    protos, table = header_prototypes(), table_entries()
    assert len(protos) >= 50
    assert set(protos) == set(_ffi.PROTOTYPES), "header and ctypes table disagree"
    assert set(table) == set(protos), sorted(set(table) ^ set(protos))
    for name, (args, result) in protos.items():
        assert table[name][0] == args, (name, table[name][0], args)
        assert table[name][1] == result, (name, table[name][1], result)


def test_ctypes_table_has_the_header_arity():
    protos = header_prototypes()
    for name, (args, _result) in protos.items():
        assert len(_ffi.PROTOTYPES[name][1]) == len(args), name
