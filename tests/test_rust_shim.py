"""The Rust binding under rust/ cannot be compiled here (no cargo): keep it in step with include/knhip.h by text.
Every `pub fn knhip_*` of kn-hip-sys must be declared in the header with the same number of parameters, the repr(C)
structs must have the header's fields in order, and the operation / dtype codes of the serialiser must be the
header's."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _read(*parts):
    with open(os.path.join(ROOT, *parts)) as f:
        return f.read()


def _header():
    return re.sub(r"/\*.*?\*/", "", _read("include", "knhip.h"), flags=re.S)


def _c_functions():
    out = {}
    for name, params in re.findall(r"\b(knhip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", _header(), flags=re.S):
        params = params.strip()
        out[name] = 0 if params in ("", "void") else len(params.split(","))
    return out


def _rust_functions():
    text = re.sub(r"//.*", "", _read("rust", "kn-hip-sys", "src", "lib.rs"))
    out = {}
    for name, params in re.findall(r"pub fn (knhip_[a-z0-9_]+)\s*\(([^)]*)\)", text, flags=re.S):
        out[name] = len([p for p in params.split(",") if p.strip()])
    return out


def test_every_bound_function_matches_the_header():
    c, rust = _c_functions(), _rust_functions()
    assert len(rust) >= 45
    assert not [n for n in rust if n not in c], "bound in Rust but not declared in knhip.h"
    assert {n: c[n] for n in rust} == rust
    # the whole runtime and executor tiers are bound; only builder / query / layout-test entry points may be left out
    unbound = [n for n in c if n not in rust and not n.startswith(("knhip_graph_", "knhip_optimizer_"))]
    assert sorted(unbound) == ["knhip_executor_new", "knhip_executor_step_source"]


def _c_struct_fields(name):
    body = re.search(r"typedef struct \{([^}]*)\} " + name + ";", _header(), flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(","):
            fields.append(re.sub(r"\[.*\]", "", part.strip().split()[-1].lstrip("*")))
    return fields


def _rust_struct_fields(name):
    text = _read("rust", "kn-hip-sys", "src", "lib.rs")
    body = re.search(r"pub struct " + name + r" \{([^}]*)\}", text, flags=re.S).group(1)
    return re.findall(r"pub ([a-z0-9_]+):", body)


def test_repr_c_structs_have_the_fields_of_the_header():
    for name in ("knhip_mem_usage", "knhip_profile", "knhip_matmul_args", "knhip_executor_options", "knhip_tensor"):
        assert _rust_struct_fields(name) == _c_struct_fields(name), name


def test_the_python_struct_has_the_fields_of_the_header_too():
    from kyanite_amd._lib import ExecutorOptionsT, MatmulArgsT, TensorT
    for name, struct in (("knhip_executor_options", ExecutorOptionsT), ("knhip_matmul_args", MatmulArgsT), ("knhip_tensor", TensorT)):
        assert [f for f, _ in struct._fields_] == _c_struct_fields(name), name


def test_device_tensor_and_autokernels_of_the_rust_crate_call_what_the_header_declares():
    """every knhip_* name used by kn-hip-eval is bound in kn-hip-sys, and the reference's public methods are there"""
    rust = _rust_functions()
    for module in ("device_tensor.rs", "autokernel.rs", "shape.rs", "executor.rs"):
        text = _read("rust", "kn-hip-eval", "src", module)
        for name in set(re.findall(r"\b(knhip_[a-z0-9_]+)\s*\(", text)):
            assert name in rust, f"{module} calls {name}, which kn-hip-sys does not bind"
    tensor = _read("rust", "kn-hip-eval", "src", "device_tensor.rs")
    for method in ("alloc_simple", "deep_clone", "copy_simple_from_host", "copy_simple_to_host", "copy_from", "copy_from_host_staged",
                   "copy_to_host_staged", "permute", "view", "broadcast", "slice", "index", "flip", "repeat_unary", "to_mat_mul_arg"):
        assert re.search(r"pub (unsafe )?fn " + method + r"\b", tensor), method
    kernels = _read("rust", "kn-hip-eval", "src", "autokernel.rs")
    for kernel in ("ScalarKernel", "ReduceKernel", "SoftmaxKernel", "LayernormKernel", "GatherKernel"):
        assert f"pub struct {kernel}" in kernels and re.search(r"impl " + kernel + r" \{.*?pub unsafe fn run", kernels, flags=re.S), kernel
    executor = _read("rust", "kn-hip-eval", "src", "executor.rs")
    assert "pub device_inputs: Vec<DeviceTensor>" in executor and "pub device_outputs: Vec<DeviceTensor>" in executor


def test_codes_of_the_rust_serialiser_are_the_header_codes():
    header = _header()
    enums = {}
    for body in re.findall(r"enum\s*\{([^}]*)\}", header, flags=re.S):
        for item in body.split(","):
            m = re.match(r"\s*(KNHIP_[A-Z0-9_]+)\s*=\s*(\d+)", item)
            if m:
                enums[m.group(1)] = int(m.group(2))
    ser = _read("rust", "kn-hip-eval", "src", "serialize.rs")
    for rust_name, code in re.findall(r"DType::([A-Za-z0-9]+) => (\d+),", ser):
        assert enums["KNHIP_" + rust_name.upper()] == int(code)
    for rust_name, code in re.findall(r"UnaryOp::([A-Za-z]+)(?:\(to\))? => \((\d+),", ser):
        key = {"ValueCast": "VALUE_CAST", "BitCast": "BIT_CAST"}.get(rust_name, rust_name.upper())
        assert enums["KNHIP_UNARY_" + key] == int(code)
    for rust_name, code in re.findall(r"BinaryOp::([A-Za-z]+) => (\d+),", ser):
        assert enums["KNHIP_BINARY_" + rust_name.upper()] == int(code)
    for rust_name, code in re.findall(r"ReduceOp::([A-Za-z]+) => (\d+),", ser):
        assert enums["KNHIP_REDUCE_" + rust_name.upper()] == int(code)
    # operation tags in the order of the match arms
    tags = re.findall(r"Operation::([A-Za-z]+) \{[^}]*\} => \{\s*w\.u8\((\d+)\);", ser)
    assert len(tags) == 16
    for rust_name, code in tags:
        assert enums["KNHIP_OP_" + {"MatMul": "MATMUL"}.get(rust_name, rust_name.upper())] == int(code)
    sys_lib = _read("rust", "kn-hip-sys", "src", "lib.rs")
    for name, value in re.findall(r"pub const (KNHIP_[A-Z0-9_]+): c_int = (\d+);", sys_lib):
        if name in enums:
            assert enums[name] == int(value), name
    for name in ("KNHIP_OK", "KNHIP_ERROR", "KNHIP_BUFFER_TOO_SMALL"):
        value = re.search(r"#define " + name + r" (\d+)", header).group(1)
        assert re.search(r"pub const " + name + r": c_int = " + value + ";", sys_lib), name


def test_the_blob_the_rust_serialiser_describes_is_the_one_the_library_reads():
    """The layout comment of serialize.rs and the reader in csrc/serialize.cpp agree on magic and version; a blob
    written field by field the way serialize_graph does it deserialises into the same graph."""
    import struct

    import numpy as np

    from kyanite_amd import BATCH, Graph, UnaryOp

    g = Graph()
    x = g.input([BATCH, 3])
    w = g.constant([2, 3], np.arange(6, dtype=np.float32))
    y = g.softmax(g.unary(UnaryOp.EXP, x), 1)
    g.output(y)
    g.output(w)
    expected = g.to_bytes()

    def size(factor, exp):
        return struct.pack("<QI", factor, exp)

    no_id = struct.pack("<I", 0)
    blob = b"KNHG" + struct.pack("<II", 1, 4)
    blob += struct.pack("<BI", 0, 2) + size(1, 1) + size(3, 0) + struct.pack("<BI", 0, 0) + no_id            # Input 0
    data = np.arange(6, dtype=np.float32).tobytes()
    blob += struct.pack("<BI", 0, 2) + size(2, 0) + size(3, 0) + struct.pack("<BQ", 1, len(data)) + data + no_id  # Constant
    blob += struct.pack("<BI", 0, 2) + size(1, 1) + size(3, 0) + struct.pack("<BIBB", 11, 0, 4, 0) + no_id   # Unary exp
    blob += struct.pack("<BI", 0, 2) + size(1, 1) + size(3, 0) + struct.pack("<BII", 13, 2, 1) + no_id       # Softmax
    blob += struct.pack("<II", 1, 0) + struct.pack("<III", 2, 3, 1)
    assert blob == expected
    assert Graph.from_bytes(blob).to_bytes() == expected
