"""The command line contract of bench.py that needs no GPU: more than one GPU is refused with a message, and the
workload names are the five configurations."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout) and "--gpus 2" in (r.stderr + r.stdout)


def test_help_lists_the_workloads():
    r = run("--help")
    assert r.returncode == 0
    for name in ("all", "bandwidth", "mlp", "resnet", "llama", "unet"):
        assert name in r.stdout


def test_build_check_graph_still_covers_every_kernel_family():
    # the graph that `__graft_entry__.build()` plans after compiling; new fusions must not silently remove a family
    sys.path.insert(0, ROOT)
    import __graft_entry__

    steps, kinds = __graft_entry__.check_kernel_families()
    assert steps >= 7 and len(kinds) == 7
