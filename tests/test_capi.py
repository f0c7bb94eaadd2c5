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
