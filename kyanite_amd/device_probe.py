"""`python -m kyanite_amd.device_probe [device]`: what the matrix cores sustain on this device, and at which clock.

A register-only loop of independent f16 MFMAs (no memory traffic) with small integers and with N(0, 1) values in the
operands. The second rate is the ceiling for matmul / convolution kernels on real data."""
import sys
from ctypes import byref, c_double

from ._lib import check, lib


def mfma_probe(device=0, normal_data=True, iterations=100000):
    """(TFLOP/s, shader clock in MHz) of the register-only f16 MFMA loop."""
    tflops, mhz = c_double(), c_double()
    check(lib.knhip_device_mfma_probe(int(device), 1 if normal_data else 0, int(iterations), byref(tflops), byref(mhz)))
    return tflops.value, mhz.value


def main(argv):
    device = int(argv[1]) if len(argv) > 1 else 0
    for normal, name in ((False, "small integers"), (True, "N(0, 1) values ")):
        tflops, mhz = mfma_probe(device, normal)
        print(f"f16 MFMA, register only, {name}: {tflops:7.1f} TFLOP/s ({tflops / 2500:.3f} of 2500) at {mhz:6.0f} MHz")


if __name__ == "__main__":
    main(sys.argv)
