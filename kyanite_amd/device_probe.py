"""`python -m kyanite_amd.device_probe [device]`: what the matrix cores sustain on this device, and at which clock.

A register-only loop of independent f16 MFMAs (no memory traffic) with small integers and with N(0, 1) values in the
operands. The second rate is the ceiling for matmul / convolution kernels on real data."""
import sys
from ctypes import byref, c_double

from ._lib import check, lib


PROBE_NORMAL, PROBE_F32, PROBE_RECTIFIED = 1, 2, 4


def mfma_probe(device=0, normal_data=True, iterations=100000, f32=False, rectified=False):
    """(TFLOP/s, shader clock in MHz) of the register-only MFMA loop: f16 or f32 instruction, operands small integers
    or N(0, 1), the B operands optionally max(x, 0) like activations behind a relu."""
    mode = (PROBE_NORMAL if normal_data else 0) | (PROBE_F32 if f32 else 0) | (PROBE_RECTIFIED if rectified else 0)
    tflops, mhz = c_double(), c_double()
    check(lib.knhip_device_mfma_probe(int(device), mode, int(iterations), byref(tflops), byref(mhz)))
    return tflops.value, mhz.value


def main(argv):
    device = int(argv[1]) if len(argv) > 1 else 0
    for f32, peak in ((False, 2500.0), (True, 157.3)):
        for normal, rectified, name in ((False, False, "small integers             "), (True, False, "N(0, 1) values             "),
                                        (True, True, "N(0, 1), B operands relu'd ")):
            tflops, mhz = mfma_probe(device, normal, 100000 if not f32 else 30000, f32, rectified)
            print(f"{'f32' if f32 else 'f16'} MFMA, register only, {name}: {tflops:7.1f} TFLOP/s ({tflops / peak:.3f} of {peak:g}) at {mhz:6.0f} MHz")


if __name__ == "__main__":
    main(sys.argv)
