"""The C ABI library loads and exports every symbol that include/knhip.h declares (no compute calls)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    with open(os.path.join(ROOT, "include", "knhip.h")) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(knhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from kyanite_amd import LIB_PATH
    lib = ctypes.CDLL(LIB_PATH)
    names = declared_symbols()
    assert len(names) > 70
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in knhip.h but not exported: {missing}"


def test_python_binding_covers_the_header():
    from kyanite_amd import _lib
    bound = set(_lib.SIGNATURES) | set(_lib.SPECIAL)
    assert set(declared_symbols()) == bound


def test_error_reporting_does_not_throw_across_the_abi():
    from kyanite_amd._lib import lib
    out = ctypes.c_void_p()
    status = lib.knhip_graph_deserialize((ctypes.c_uint8 * 4)(1, 2, 3, 4), 4, ctypes.byref(out))
    assert status != 0
    assert b"truncated" in lib.knhip_last_error() or b"magic" in lib.knhip_last_error()
    n = ctypes.c_int(-1)
    assert lib.knhip_device_count(ctypes.byref(n)) == 0 and n.value >= 0


def test_oracle_is_not_linked_into_the_product():
    """The shipped library must not contain or load the oracle."""
    from kyanite_amd import LIB_PATH
    with open(LIB_PATH, "rb") as f:
        blob = f.read()
    assert b"kn_oracle_eval" not in blob and b"liboracle" not in blob
    for root, _, files in os.walk(os.path.join(ROOT, "kyanite_amd")):
        for name in files:
            if name.endswith((".py", ".cpp", ".h", ".hip")):
                with open(os.path.join(root, name)) as f:
                    assert "oracle" not in f.read().lower(), f"{name} mentions the oracle"


def test_one_kernel_plans_pass_the_launch_argument_check():
    """A plan that runs as one generated kernel is only built when the compiled kernel expects exactly the bytes of
    launch arguments that the executor passes (pointer table by value, completion word, launch number): read from the
    code object's metadata when the executor is made, with or without a device. Every small case of the graph tests goes
    through the same check; here the count is spelled out for the tiny MLP: 8 operands of 3 steps."""
    import re

    from kyanite_amd import HipExecutor
    from kyanite_amd.configs import build_tiny_mlp

    graph, _ = build_tiny_mlp(seed=0, batch=8)
    ex = HipExecutor(0, graph, 8, plan_only=True)
    source = ex.fused_source()
    assert source, "the tiny MLP plans as one kernel"
    slots = int(re.search(r"struct KnFusedPtrs \{ void \*p\[(\d+)\]; \};", source).group(1))
    assert slots == sum(len(re.findall(r"\bf32\[", ex.step_str(i).split("operands:")[1])) for i in range(ex.step_count())) == 8
