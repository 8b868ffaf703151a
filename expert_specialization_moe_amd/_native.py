"""Loads the in-tree native libraries and exposes the C ABI through ctypes.

``lib`` is ``libesmoe.so`` (include/esmoe.h) with argument types declared;
loading ``_C.so`` registers ``torch.ops.expert_specialization.*``.
"""
import ctypes
import os

import torch  # noqa: F401  torch's HIP runtime must be in the process first

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libesmoe.so")
BINDING_PATH = os.path.join(_PKG, "_C.so")


def _missing(path):
    return ImportError(
        f"{path} is missing: build the native libraries first with "
        "`python expert_specialization_moe_amd/build.py` (there is no non-native fallback)"
    )


if not os.path.exists(LIB_PATH):
    raise _missing(LIB_PATH)
if not os.path.exists(BINDING_PATH):
    raise _missing(BINDING_PATH)

lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
torch.ops.load_library(BINDING_PATH)

_vp = ctypes.c_void_p
_i = ctypes.c_int
_sz = ctypes.c_size_t

lib.esmoe_gemm_workspace_bytes.restype = _sz
lib.esmoe_gemm_workspace_bytes.argtypes = [_i]
lib.esmoe_stream_workspace.restype = _i
lib.esmoe_stream_workspace.argtypes = [_vp, ctypes.POINTER(_vp), ctypes.POINTER(_sz)]
lib.esmoe_fp8_blockwise_grouped_mm.restype = _i
lib.esmoe_fp8_blockwise_grouped_mm.argtypes = [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz, _vp]
lib.esmoe_fp8_blockwise_grouped_mm_static.restype = _i
lib.esmoe_fp8_blockwise_grouped_mm_static.argtypes = [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]
lib.esmoe_mxfp8_grouped_mm.restype = _i
lib.esmoe_mxfp8_grouped_mm.argtypes = [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz, _vp]
lib.esmoe_mxfp8_grouped_quant.restype = _i
lib.esmoe_mxfp8_grouped_quant.argtypes = [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]
lib.esmoe_fp8_blockwise_grouped_mm_swiglu_quant.restype = _i
lib.esmoe_fp8_blockwise_grouped_mm_swiglu_quant.argtypes = [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp,
                                                            ctypes.c_size_t, _vp]
lib.esmoe_mxfp8_grouped_mm_swiglu_quant.restype = _i
lib.esmoe_mxfp8_grouped_mm_swiglu_quant.argtypes = [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp,
                                                    ctypes.c_size_t, _vp]
lib.esmoe_swiglu_mxfp8_grouped_quant.restype = _i
lib.esmoe_swiglu_mxfp8_grouped_quant.argtypes = [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]
lib.esmoe_mxfp8_quant_weight.restype = _i
lib.esmoe_mxfp8_quant_weight.argtypes = [_vp, _i, _vp, _vp, ctypes.c_long, _i, _vp]
lib.esmoe_fp8_quant_act_1x128.restype = _i
lib.esmoe_fp8_quant_act_1x128.argtypes = [_vp, _i, _vp, _vp, ctypes.c_long, _i, _vp]
lib.esmoe_fp8_quant_weight_128x128.restype = _i
lib.esmoe_fp8_quant_weight_128x128.argtypes = [_vp, _i, _vp, _vp, ctypes.c_long, _i, _vp]
lib.esmoe_route_workspace_bytes.restype = _sz
lib.esmoe_route_workspace_bytes.argtypes = [ctypes.c_long, _i]
lib.esmoe_route_metadata.restype = _i
lib.esmoe_route_metadata.argtypes = [_vp, ctypes.c_long, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _sz, _vp]
lib.esmoe_permute_rows.restype = _i
lib.esmoe_permute_rows.argtypes = [_vp, _vp, ctypes.c_long, _i, ctypes.c_long, _vp, _vp]
lib.esmoe_swiglu_quant_1x128.restype = _i
lib.esmoe_swiglu_quant_1x128.argtypes = [_vp, _i, _vp, _vp, ctypes.c_long, _i, _vp]
lib.esmoe_last_error.restype = ctypes.c_char_p
lib.esmoe_last_error.argtypes = []
lib.esmoe_version.restype = ctypes.c_char_p
lib.esmoe_version.argtypes = []
lib.esmoe_host_schedule.restype = _i
lib.esmoe_host_schedule.argtypes = [_vp, _i, _i, _i, _i, _vp]
lib.esmoe_host_decode_heavy.restype = _i
lib.esmoe_host_decode_heavy.argtypes = [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp]
lib.esmoe_host_decode_light.restype = _i
lib.esmoe_host_decode_light.argtypes = [_vp, _vp, _i, _i, _i, _i, _i, _vp]


def last_error():
    return lib.esmoe_last_error().decode()
