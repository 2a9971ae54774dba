"""Loader of the native code built by ``python -m geo_amd.build``.

Nothing here falls back to Python or CPU code: if a library is missing the import fails
with the command that builds it.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os
import sys
import sysconfig

import torch  # noqa: F401  loads the HIP runtime the libraries bind to

HERE = os.path.dirname(os.path.abspath(__file__))
LIBDIR = os.path.join(HERE, "lib")
_BUILD_HINT = "build the native code first: python -m geo_amd.build"


class ConvDesc(ctypes.Structure):
    """geo_sc_conv_desc of include/geo_sc.h"""
    _fields_ = [(n, ctypes.c_int32) for n in (
        "n", "c_in", "w_in", "h_in", "c_out", "w_k", "h_k", "pad_w", "pad_h", "bit_length",
        "total_width", "load_width", "load_wait_w", "load_wait_a", "accumulate", "z_unit", "generator", "seed")]


class Options(ctypes.Structure):
    """geo_sc_options of include/geo_sc.h"""
    _fields_ = [("struct_bytes", ctypes.c_size_t), ("forward_stream_bytes", ctypes.c_size_t),
                ("backward_groups_per_round", ctypes.c_int32), ("forward_single_stream", ctypes.c_int32)]


# every symbol include/geo_sc.h declares: name -> (restype, argtypes)
_P = ctypes.c_void_p
_SZ = ctypes.POINTER(ctypes.c_size_t)
_D = ctypes.POINTER(ConvDesc)
_O = ctypes.POINTER(Options)
C_API = {
    "geo_sc_init": (ctypes.c_int, []),
    "geo_sc_stream_table_copy": (ctypes.c_int, [ctypes.c_int, _P, ctypes.c_size_t, _SZ]),
    "geo_sc_static_workspace_bytes": (ctypes.c_size_t, []),
    "geo_sc_conv2d_add_partial_workspace_size_ex": (ctypes.c_int, [_D, _O, _SZ]),
    "geo_sc_conv2d_add_partial_forward_chunk": (ctypes.c_int, [_D, _O, ctypes.POINTER(ctypes.c_int)]),
    "geo_sc_conv2d_add_partial_forward_ex": (ctypes.c_int, [_D, _O, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    "geo_sc_conv2d_add_partial_backward_workspace_size_ex": (ctypes.c_int, [_D, _O, _SZ]),
    "geo_sc_conv2d_add_partial_backward_ex": (ctypes.c_int, [_D, _O, _P, _P, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    "geo_sc_version": (ctypes.c_int, []),
    "geo_sc_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "geo_sc_conv2d_add_partial_workspace_size": (ctypes.c_int, [_D, _SZ]),
    "geo_sc_conv2d_add_partial_forward": (ctypes.c_int, [_D, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    "geo_sc_conv2d_add_partial_from_streams": (ctypes.c_int, [_D, _P, _P, _P, _P]),
    "geo_sc_stream_tables_size": (ctypes.c_int, [ctypes.c_int, _SZ]),
    "geo_sc_act_streams": (ctypes.c_int, [_D, _P, _P, _P, _P]),
    "geo_sc_weight_streams": (ctypes.c_int, [_D, _P, _P, _P, _P]),
    "geo_sc_act_streams_q7": (ctypes.c_int, [_D, _P, _P, _P, _P]),
    "geo_sc_act_stream_words": (ctypes.c_int, [_D, _SZ]),
    "geo_sc_act_stream_layout": (ctypes.c_int, [_D, ctypes.POINTER(ctypes.c_int)]),
    "geo_sc_conv2d_add_partial_backward_workspace_size": (ctypes.c_int, [_D, _SZ]),
    "geo_sc_conv2d_add_partial_backward": (ctypes.c_int, [_D, _P, _P, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    "geo_sc_weight_stream_words": (ctypes.c_int, [_D, _SZ]),
    "geo_sc_layer_epilogue": (ctypes.c_int, [_P] + [ctypes.c_int] * 5 + [_P, _P, ctypes.c_int, _P, _P, _P]),
    "geo_sc_layer_tail_backward_workspace_size": (ctypes.c_int, [ctypes.c_int] * 4 + [_SZ]),
    "geo_sc_layer_tail_backward": (ctypes.c_int, [_P, _P] + [ctypes.c_int] * 5 + [_P] * 5 + [ctypes.c_int] + [_P] * 4 +
                                   [ctypes.c_size_t, _P]),
    "geo_sc_count_stats_workspace_size": (ctypes.c_int, [ctypes.c_int] * 4 + [_SZ]),
    "geo_sc_count_stats": (ctypes.c_int, [_P] + [ctypes.c_int] * 5 + [_P, _P, _P, ctypes.c_size_t, _P]),
    "geo_sc_bn_fixed_affine": (ctypes.c_int, [_P] * 4 + [ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_longlong] +
                               [_P] * 7),
    "geo_sc_bn_fixed_from_counts": (ctypes.c_int, [_P] + [ctypes.c_int] * 5 + [_P, _P, ctypes.c_float, ctypes.c_float] +
                                    [_P] * 9 + [ctypes.c_size_t, _P]),
    "geo_sc_quantize_many": (ctypes.c_int, [ctypes.c_int, _P, _P, _P, ctypes.c_int, _P]),
    "geo_sc_copy_back_clamp": (ctypes.c_int, [ctypes.c_int, _P, _P, _P, _P, ctypes.c_float, ctypes.c_float, _P]),
    "geo_sc_conv2d_add_partial_forward_q7": (ctypes.c_int, [_D, _P, _P, _P, _P, ctypes.c_size_t, _P]),
    "geo_sc_quantize": (ctypes.c_int, [_P, _P, ctypes.c_size_t, ctypes.c_int, _P]),
    "geo_sc_weight_streams_finish": (ctypes.c_int, [_D, _P, _P]),
    "geo_sc_weight_streams_check": (ctypes.c_int, [_D, _P, _P]),
    "geo_sc_conv2d_add_partial_forward_static": (ctypes.c_int, [_D, _P, _P, _P, _P]),
}

_lib = None
_probe = None
_modules = {}


def lib_path() -> str:
    return os.path.join(LIBDIR, "libgeo_sc.so")


def lib() -> ctypes.CDLL:
    """libgeo_sc.so with argument types set."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.isfile(path):
            raise ImportError(f"{path} not found; {_BUILD_HINT}")
        L = ctypes.CDLL(path)
        for name, (res, args) in C_API.items():
            fn = getattr(L, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def probe_lib() -> ctypes.CDLL:
    """libgeo_sc_probe.so: the benchmark's issue-rate probe (csrc/sc_probe.hip), not part of the C ABI."""
    global _probe
    if _probe is None:
        path = os.path.join(LIBDIR, "libgeo_sc_probe.so")
        if not os.path.isfile(path):
            raise ImportError(f"{path} not found; {_BUILD_HINT}")
        L = ctypes.CDLL(path)
        L.geo_sc_probe_and_or_rate.restype = ctypes.c_int
        L.geo_sc_probe_and_or_rate.argtypes = [ctypes.c_int, _P, ctypes.c_size_t, ctypes.POINTER(ctypes.c_double), _P]
        L.geo_sc_probe_mfma_slices.restype = ctypes.c_int
        L.geo_sc_probe_mfma_slices.argtypes = [ctypes.c_int] * 4 + [_P, ctypes.c_size_t, _P, ctypes.c_size_t, _P, _P]
        _probe = L
    return _probe


def module(name: str):
    """The PyTorch extension module ``sc_extension_cuda`` or ``sc_extension``."""
    if name not in _modules:
        path = os.path.join(LIBDIR, name + sysconfig.get_config_var("EXT_SUFFIX"))
        if not os.path.isfile(path):
            raise ImportError(f"{path} not found; {_BUILD_HINT}")
        spec = importlib.util.spec_from_file_location(name, path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _modules[name] = mod
    return _modules[name]


def register_reference_module_names():
    """Make ``import sc_extension`` / ``import sc_extension_cuda`` resolve to this build, the
    way the reference's utils_functional.py imports them (utils_functional.py:11-12)."""
    for name in ("sc_extension", "sc_extension_cuda"):
        sys.modules[name] = module(name)
