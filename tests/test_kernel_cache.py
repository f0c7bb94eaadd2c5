"""The on-disk cache of compiled kernels (csrc/rtc.cpp; the role of kn-cuda-eval/src/autokernel/common.rs:14-46, which
only caches in memory): a cache file that is damaged, cut short or written in another layout is never loaded; it is
replaced by a fresh compilation. Runs without a GPU (plan-only executors compile, they do not launch)."""
import json
import os
import struct
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import json, sys
import numpy as np
sys.path.insert(0, %r)
from kyanite_amd import Graph, HipDevice, HipExecutor, compile_stats, DType
from kyanite_amd.graph import UnaryOp
g = Graph()
x = g.input([8, 16], DType.F32)
y = g.softmax(g.unary(UnaryOp.EXP, x), 1)
z = g.layernorm(g.add(x, y), 1, 1e-5)
g.output(y)
g.output(z)
ex = HipExecutor(0, g, 0, plan_only=True, step_by_step=True)
print(json.dumps(compile_stats()))
"""


def run_child(cache_dir):
    env = dict(os.environ, KNHIP_CACHE_DIR=cache_dir)
    out = subprocess.run([sys.executable, "-c", CHILD % ROOT], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    stats = json.loads(out.stdout.strip().splitlines()[-1])
    return stats["compiled"], stats["disk_hits"]


def cache_files(cache_dir):
    return sorted(os.path.join(cache_dir, f) for f in os.listdir(cache_dir) if f.endswith(".hsaco"))


def test_damaged_cache_files_are_rebuilt(tmp_path):
    cache_dir = str(tmp_path / "kcache")
    compiled, disk_hits = run_child(cache_dir)
    files = cache_files(cache_dir)
    assert compiled == len(files) >= 3 and disk_hits == 0
    for f in files:
        blob = open(f, "rb").read()
        magic, layout, header_bytes, key, check, code_bytes, code_hash = struct.unpack("<8sIIQQQQ", blob[:48])
        assert magic == b"KNHSACO\0" and header_bytes == 48 and code_bytes == len(blob) - 48
        assert "%016x" % key == os.path.basename(f)[:16]
        assert blob[48:52] == b"\x7fELF"

    # an intact cache serves every kernel
    assert run_child(cache_dir) == (0, len(files))

    originals = [open(f, "rb").read() for f in files]
    # one byte of the code object flipped, a file cut short, and a bare code object without the header
    damaged = bytearray(originals[0])
    damaged[len(damaged) // 2] ^= 0x40
    open(files[0], "wb").write(bytes(damaged))
    open(files[1], "wb").write(originals[1][: len(originals[1]) // 2])
    open(files[2], "wb").write(originals[2][48:])
    compiled, disk_hits = run_child(cache_dir)
    assert (compiled, disk_hits) == (3, len(files) - 3)
    # hipRTC is deterministic for one source and one set of options: the rebuilt files equal the first ones
    assert [open(f, "rb").read() for f in files] == originals

    # a file that belongs to another source (same name, other second hash) is not trusted either
    other = bytearray(originals[0])
    other[24] ^= 1
    open(files[0], "wb").write(bytes(other))
    assert run_child(cache_dir) == (1, len(files) - 1)
    assert not [f for f in os.listdir(cache_dir) if ".tmp" in f]
