"""ctypes front-end of the CPU oracle (``sc_oracle.c``) and loader of the compiled
reference (``oracle/_ref``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
``cpu_baseline`` leg of ``bench.py``.  The shipped GPU path never imports this module.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(HERE, "libsc_oracle.so")
_lib = None

SUPPORTED_LENGTHS = (8, 16, 32, 64, 128, 256)
# Progressive loading parameters that leave every code untouched; total_width is what the
# reference's Python always passes (utils_functional.py:28, :497).
NEUTRAL = dict(total_width=7, load_width=8, load_wait_w=1, load_wait_a=1)


def lib():
    """Load (building if nothing is built yet) ``libsc_oracle.so``."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.isfile(_LIB_PATH):
        from . import build_oracle  # type: ignore
        build_oracle.build_oracle()
    L = ctypes.CDLL(_LIB_PATH)
    i = ctypes.c_int
    fp = ctypes.POINTER(ctypes.c_float)
    up = ctypes.POINTER(ctypes.c_uint32)
    ip = ctypes.POINTER(ctypes.c_int32)
    L.sco_lfsr_step.argtypes = [i, i]
    L.sco_lfsr_step.restype = i
    L.sco_nbits_for_length.argtypes = [i]
    L.sco_nbits_for_length.restype = i
    for name in ("sco_code_act", "sco_code_wpos", "sco_code_wneg"):
        getattr(L, name).argtypes = [ctypes.c_float, i]
        getattr(L, name).restype = i
    L.sco_stream_of.argtypes = [i, i, i, i, i, i, up]
    L.sco_stream_of.restype = i
    L.sco_weight_streams.argtypes = [fp, i, i, i, i, i, i, i, i, up, up]
    L.sco_weight_streams.restype = i
    L.sco_act_streams.argtypes = [fp, i, i, i, i, i, i, i, up]
    L.sco_act_streams.restype = i
    L.sco_conv2d_add_partial.argtypes = [fp, fp, ip] + [i] * 16
    L.sco_conv2d_add_partial.restype = i
    L.sco_conv2d_modes.argtypes = [fp, fp, ip] + [i] * 16
    L.sco_conv2d_modes.restype = i
    L.sco_conv2d_general.argtypes = [fp, fp, ip] + [i] * 17 + [ctypes.c_uint64]
    L.sco_conv2d_general.restype = i
    L.sco_philox4x32_10.argtypes = [up, up, up]
    L.sco_philox4x32_10.restype = None
    L.sco_random_stream_words.argtypes = [i, i, i, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_uint64, up]
    L.sco_random_stream_words.restype = None
    L.sco_max_threads.argtypes = []
    L.sco_max_threads.restype = i
    _lib = L
    return L


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def lfsr_step(n_bits: int, state: int) -> int:
    return lib().sco_lfsr_step(n_bits, state)


def nbits_for_length(L: int) -> int:
    return lib().sco_nbits_for_length(L)


def code_act(x: float, L: int) -> int:
    return lib().sco_code_act(float(np.float32(x)), L)


def code_wpos(w: float, L: int) -> int:
    return lib().sco_code_wpos(float(np.float32(w)), L)


def code_wneg(w: float, L: int) -> int:
    return lib().sco_code_wneg(float(np.float32(w)), L)


def stream_of(code: int, seed: int, L: int, total_width=7, load_width=8, load_wait=1):
    """(words[P] uint32, final LFSR state) of one value."""
    P = (L + 31) // 32
    words = np.zeros(P, dtype=np.uint32)
    s = lib().sco_stream_of(code, seed, L, total_width, load_width, load_wait, _ptr(words, ctypes.c_uint32))
    if s < 0:
        raise ValueError(f"unsupported stream length {L}")
    return words, s


def weight_streams(w, L: int, total_width=7, load_width=8, load_wait=1):
    """(wpos, wneg), each uint32 [P][H][Cin][W][Cout]."""
    w = _f32(w)
    Cout, Cin, W, H = w.shape
    P = (L + 31) // 32
    wpos = np.zeros((P, H, Cin, W, Cout), dtype=np.uint32)
    wneg = np.zeros_like(wpos)
    rc = lib().sco_weight_streams(_ptr(w, ctypes.c_float), Cout, Cin, W, H, L, total_width, load_width, load_wait,
                                  _ptr(wpos, ctypes.c_uint32), _ptr(wneg, ctypes.c_uint32))
    if rc != 0:
        raise ValueError(f"unsupported stream length {L}")
    return wpos, wneg


def act_streams(x_item_padded, L: int, total_width=7, load_width=8, load_wait=1):
    """uint32 [P][Cin][Wi][Hi] for ONE already padded batch item (Cin, Wi, Hi)."""
    x = _f32(x_item_padded)
    Cin, Wi, Hi = x.shape
    P = (L + 31) // 32
    out = np.zeros((P, Cin, Wi, Hi), dtype=np.uint32)
    rc = lib().sco_act_streams(_ptr(x, ctypes.c_float), Cin, Wi, Hi, L, total_width, load_width, load_wait,
                               _ptr(out, ctypes.c_uint32))
    if rc != 0:
        raise ValueError(f"unsupported stream length {L}")
    return out


def conv2d_add_partial(x, w, L: int, padding=(0, 0), total_width=7, load_width=8, load_wait_w=1, load_wait_a=1,
                       fast=True, n_threads=0):
    """int32 (N,Cout,Wo,Ho).  ``padding=(p0,p1)`` follows the reference: p0 pads the last
    dim, p1 the one before it (sc.cpp:298)."""
    x = _f32(x)
    w = _f32(w)
    N, Cin, Wx, Hx = x.shape
    Cout, Cin2, W, H = w.shape
    if Cin != Cin2:
        raise ValueError("channel mismatch")
    pad_h, pad_w = int(padding[0]), int(padding[1])
    Wo = Wx + 2 * pad_w - W + 1
    Ho = Hx + 2 * pad_h - H + 1
    y = np.zeros((N, Cout, max(Wo, 0), max(Ho, 0)), dtype=np.int32)
    rc = lib().sco_conv2d_add_partial(_ptr(x, ctypes.c_float), _ptr(w, ctypes.c_float), _ptr(y, ctypes.c_int32),
                                      N, Cin, Wx, Hx, Cout, W, H, pad_w, pad_h, L, total_width, load_width,
                                      load_wait_w, load_wait_a, int(bool(fast)), int(n_threads))
    if rc != 0:
        raise ValueError("unsupported stream length or bad arguments")
    return y


MODES = {"y": 0, "z": 1, "yz": 2}


def conv2d_modes(x, w, L: int, padding=(0, 0), mode="y", z_unit=1, total_width=7, load_width=8, load_wait_w=1,
                 load_wait_a=1):
    """int32 (N,Cout,Wo,Ho) for accumulation mode "y" | "z" | "yz" (scalar loops: small shapes).
    "z"/"yz" follow the reference's CUDA source text only (no executable reference)."""
    x = _f32(x)
    w = _f32(w)
    N, Cin, Wx, Hx = x.shape
    Cout, _, W, H = w.shape
    pad_h, pad_w = int(padding[0]), int(padding[1])
    Wo = Wx + 2 * pad_w - W + 1
    Ho = Hx + 2 * pad_h - H + 1
    y = np.zeros((N, Cout, max(Wo, 0), max(Ho, 0)), dtype=np.int32)
    rc = lib().sco_conv2d_modes(_ptr(x, ctypes.c_float), _ptr(w, ctypes.c_float), _ptr(y, ctypes.c_int32), N, Cin, Wx,
                                Hx, Cout, W, H, pad_w, pad_h, L, total_width, load_width, load_wait_w, load_wait_a,
                                MODES[mode], int(z_unit))
    if rc != 0:
        raise ValueError("unsupported stream length or bad arguments")
    return y


GENERATORS = {"lfsr": 0, "acc": 1, "rand": 2}
MODES_ALL = {"y": 0, "z": 1, "yz": 2, "full": 3}


def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    out = np.zeros(4, dtype=np.uint32)
    lib().sco_philox4x32_10(_ptr(c, ctypes.c_uint32), _ptr(k, ctypes.c_uint32), _ptr(out, ctypes.c_uint32))
    return out


def random_stream(code: int, L: int, generator: str, tag: int, index: int, seed: int):
    """words[P] uint32 of one value's random stream (generator "acc" or "rand")."""
    words = np.zeros((L + 31) // 32, dtype=np.uint32)
    lib().sco_random_stream_words(int(code), L, GENERATORS[generator], tag, index, seed, _ptr(words, ctypes.c_uint32))
    return words


def conv2d_general(x, w, L: int, padding=(0, 0), mode="y", z_unit=1, generator="lfsr", seed=0, total_width=7,
                   load_width=8, load_wait_w=1, load_wait_a=1):
    """int32 (N,Cout,Wo,Ho) for any accumulation mode ("y" | "z" | "yz" | "full") and generator
    ("lfsr" | "acc" | "rand"); scalar loops, small shapes."""
    x = _f32(x)
    w = _f32(w)
    N, Cin, Wx, Hx = x.shape
    Cout, _, W, H = w.shape
    pad_h, pad_w = int(padding[0]), int(padding[1])
    Wo = Wx + 2 * pad_w - W + 1
    Ho = Hx + 2 * pad_h - H + 1
    y = np.zeros((N, Cout, max(Wo, 0), max(Ho, 0)), dtype=np.int32)
    rc = lib().sco_conv2d_general(_ptr(x, ctypes.c_float), _ptr(w, ctypes.c_float), _ptr(y, ctypes.c_int32), N, Cin,
                                  Wx, Hx, Cout, W, H, pad_w, pad_h, L, total_width, load_width, load_wait_w,
                                  load_wait_a, MODES_ALL[mode], int(z_unit), GENERATORS[generator], int(seed))
    if rc != 0:
        raise ValueError("unsupported stream length or bad arguments")
    return y


def max_threads() -> int:
    return lib().sco_max_threads()


# ---------------------------------------------------------------------------------------
# The compiled reference (oracle/_ref): sc.cpp built unmodified by build_oracle.build_ref
# ---------------------------------------------------------------------------------------
def _cpu_flags():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


def ref_variants_usable():
    """ISA variants of the compiled reference that exist on disk and that this CPU can run,
    widest first."""
    flags = _cpu_flags()
    out = []
    for name, need in (("avx512", "avx512f"), ("avx2", "avx2"), ("scalar", None)):
        path = os.path.join(HERE, "_ref", f"sc_extension_ref_{name}.so")
        if os.path.isfile(path) and (need is None or need in flags):
            out.append(name)
    return out


_ref_cache = {}


def load_ref(variant: str | None = None):
    """Import the compiled reference module (exports ``conv2d_add_partial_new``), or return
    None when none is built/usable here."""
    usable = ref_variants_usable()
    if variant is None:
        if not usable:
            return None
        variant = usable[0]
    elif variant not in usable:
        return None
    if variant in _ref_cache:
        return _ref_cache[variant]
    import torch  # noqa: F401  (the module links against libtorch)

    name = f"sc_extension_ref_{variant}"
    path = os.path.join(HERE, "_ref", name + ".so")
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _ref_cache[variant] = mod
    return mod
