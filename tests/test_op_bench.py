"""`python -m kyanite_amd.op_bench`: every case of the families without weights plans and compiles without a device and
names the kernels it got; on a device a family runs and reports a time per case."""
import pytest

from kyanite_amd import op_bench


def test_plans_without_a_device(capsys):
    assert op_bench.main(["-p", "reduce", "rows", "elementwise", "gather", "activations", "attention"]) == 0
    text = capsys.readouterr().out
    assert text.count("MatMul attention") == 8 and text.count("[128 queries share each block of keys]") == 5
    assert "fold of 1024 partial results" in text and "columns TX=32 TY=8" in text and "transposed tiles 64x64" in text
    assert "rank=2 vec=8 unroll=4" in text  # embedding rows of halves: 16 bytes per thread


def test_rejects_an_unknown_family():
    with pytest.raises(SystemExit):
        op_bench.main(["-p", "sorting"])


@pytest.mark.gpu
def test_times_a_family(hip_device, capsys):
    assert op_bench.main(["-d", str(hip_device.index), "-n", "2", "reduce"]) == 0
    lines = [line for line in capsys.readouterr().out.splitlines() if " us " in line]
    assert len(lines) == 8 and all("TB/s" in line for line in lines)
