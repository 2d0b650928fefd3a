"""Shared helpers of the test-suite: scene construction for both the oracle and the HIP library,
and the ctypes view of the host build of the kernel bodies (tests/hostsim)."""
import ctypes as C
import os
import subprocess

import numpy as np

from oracle import oracle as O
from sphericalrf_amd import scene

HERE = os.path.dirname(os.path.abspath(__file__))

from oracle.support import oracle_params, build_scene, random_network_output  # noqa: F401  (shared with bench.py and the smoke check)


class HostSim:
    def __init__(self, lib):
        self.lib = lib
        lib.hs_elem.restype = C.c_float
        lib.hs_elem.argtypes = [C.c_int, C.c_float, C.c_float]
        lib.hs_float_to_half.restype = C.c_uint16
        lib.hs_float_to_half.argtypes = [C.c_float]
        lib.hs_half_to_float.restype = C.c_float
        lib.hs_half_to_float.argtypes = [C.c_uint16]
        lib.hs_morton3d.restype = C.c_uint32
        lib.hs_morton3d.argtypes = [C.c_uint32] * 3
        lib.hs_morton3d_invert.restype = C.c_uint32
        lib.hs_morton3d_invert.argtypes = [C.c_uint32]
        lib.hs_ld_random_val.restype = C.c_float
        lib.hs_ld_random_val.argtypes = [C.c_uint32] * 3


def load_hostsim():
    d = os.path.join(HERE, "hostsim")
    subprocess.run(["make", "-C", d], check=True, stdout=subprocess.DEVNULL)
    return HostSim(C.CDLL(os.path.join(d, "libhostsim.so")))


def ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)
