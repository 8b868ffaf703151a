"""ctypes wrapper of oracle/brute.c (test infrastructure, see oracle/__init__.py)."""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_DIR, "libbrute.so")


def build():
    subprocess.check_call(["make", "-C", _DIR, "-s"])


def _lib():
    if not os.path.exists(_LIB):
        build()
    lib = ctypes.CDLL(_LIB)
    lib.brute_sf_offset.restype = ctypes.c_int64
    lib.brute_sf_offset.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
    return lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def fp8_blockwise(a_codes, b_codes, sa, sb, problem_sizes, expert_offsets):
    a_codes = np.ascontiguousarray(a_codes, dtype=np.uint8)
    b_codes = np.ascontiguousarray(b_codes, dtype=np.uint8)
    sa = np.ascontiguousarray(sa, dtype=np.float32)
    sb = np.ascontiguousarray(sb, dtype=np.float32)
    ps = np.ascontiguousarray(problem_sizes, dtype=np.int32)
    eo = np.ascontiguousarray(expert_offsets, dtype=np.int32)
    out = np.full((a_codes.shape[0], b_codes.shape[1]), np.nan, dtype=np.float64)
    _lib().brute_fp8_blockwise(_p(a_codes), _p(b_codes), _p(sa), _p(sb), _p(ps), _p(eo), len(ps), _p(out))
    return out


def mxfp8(a_codes, b_codes, sfa, sfb, problem_sizes, expert_offsets, blockscale_offsets):
    a_codes = np.ascontiguousarray(a_codes, dtype=np.uint8)
    b_codes = np.ascontiguousarray(b_codes, dtype=np.uint8)
    sfa = np.ascontiguousarray(sfa, dtype=np.uint8)
    sfb = np.ascontiguousarray(sfb, dtype=np.uint8)
    ps = np.ascontiguousarray(problem_sizes, dtype=np.int32)
    eo = np.ascontiguousarray(expert_offsets, dtype=np.int32)
    bso = np.ascontiguousarray(blockscale_offsets, dtype=np.int32)
    out = np.full((a_codes.shape[0], b_codes.shape[1]), np.nan, dtype=np.float64)
    _lib().brute_mxfp8(_p(a_codes), _p(b_codes), _p(sfa), _p(sfb), _p(ps), _p(eo), _p(bso), len(ps), _p(out))
    return out


def sf_offset(r, c, k):
    return int(_lib().brute_sf_offset(int(r), int(c), int(k)))
