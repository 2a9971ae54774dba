"""Python callers of the C ABI in ``include/geo_sc.h`` (ctypes, raw device pointers).

torch is used for device memory and the current stream only; every function below is one
C call.  These are what the GPU parity tests and the benchmark drive.
"""
from __future__ import annotations

import ctypes

import torch

from . import _native
from ._native import ConvDesc, Options

NEUTRAL_LOADING = dict(total_width=7, load_width=8, load_wait_w=1, load_wait_a=1)


class GeoScError(RuntimeError):
    def __init__(self, status: int, what: str):
        self.status = status
        text = _native.lib().geo_sc_status_string(status).decode()
        super().__init__(f"{what}: {text} (status {status})")


def _check(status: int, what: str):
    if status != 0:
        raise GeoScError(status, what)


# enum geo_sc_accumulate
ACCUMULATE = {"y": 0, "z": 1, "yz": 2, "full": 3}
# enum geo_sc_generator
GENERATOR = {"lfsr": 0, "acc": 1, "rand": 2}


def make_desc(x_shape, w_shape, bit_length, padding=(0, 0), total_width=7, load_width=8, load_wait_w=1,
              load_wait_a=1, accumulate="y", z_unit=1, generator="lfsr", seed=0) -> ConvDesc:
    """``padding=(p0, p1)`` follows the reference: p0 pads the last dim, p1 the one before.
    ``accumulate``: "y" (OR over c_in and w_k, add over h_k), "z" (OR over the kernel window, add
    over c_in) or "yz" (OR over ``z_unit`` channels and w_k, add over h_k and channel groups)."""
    n, c_in, w_in, h_in = (int(v) for v in x_shape)
    c_out, c_in2, w_k, h_k = (int(v) for v in w_shape)
    if c_in != c_in2:
        raise ValueError(f"channel mismatch: {c_in} vs {c_in2}")
    return ConvDesc(n, c_in, w_in, h_in, c_out, w_k, h_k, int(padding[1]), int(padding[0]), int(bit_length),
                    int(total_width), int(load_width), int(load_wait_w), int(load_wait_a),
                    ACCUMULATE[accumulate] if isinstance(accumulate, str) else int(accumulate), int(z_unit),
                    GENERATOR[generator] if isinstance(generator, str) else int(generator),
                    ctypes.c_int32(int(seed) & 0xffffffff).value)


def make_options(forward_stream_bytes=0, backward_groups_per_round=0, forward_single_stream=False) -> Options:
    """geo_sc_options: the budget (bytes) of the forward's activation stream buffer - a batch whose streams
    exceed it runs in chunks of items - and the cap on the add groups per round of backward launches;
    0 leaves a field at the library's default.  forward_single_stream keeps a cut batch on the caller's stream
    (by default its odd chunks run on a second stream of the library)."""
    return Options(ctypes.sizeof(Options), int(forward_stream_bytes), int(backward_groups_per_round),
                   1 if forward_single_stream else 0)


def _opt_ptr(options):
    return ctypes.byref(options) if options is not None else None


def _stream_ptr(stream=None):
    s = stream if stream is not None else torch.cuda.current_stream()
    return ctypes.c_void_p(s.cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def version() -> int:
    return _native.lib().geo_sc_version()


def workspace_size(desc: ConvDesc, options: Options = None) -> int:
    out = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_conv2d_add_partial_workspace_size_ex(ctypes.byref(desc), _opt_ptr(options),
                                                                     ctypes.byref(out)), "workspace query")
    return out.value


def forward_chunk(desc: ConvDesc, options: Options = None) -> int:
    """Batch items per chunk of the forward (geo_sc_conv2d_add_partial_forward_chunk)."""
    out = ctypes.c_int(0)
    _check(_native.lib().geo_sc_conv2d_add_partial_forward_chunk(ctypes.byref(desc), _opt_ptr(options),
                                                                 ctypes.byref(out)), "chunk query")
    return out.value


def output_shape(desc: ConvDesc):
    return (desc.n, desc.c_out, desc.w_in + 2 * desc.pad_w - desc.w_k + 1, desc.h_in + 2 * desc.pad_h - desc.h_k + 1)


def _require_gpu_f32(t, name):
    if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
        raise ValueError(f"{name} must be a contiguous float32 GPU tensor")


def conv2d_add_partial_forward(x, w, bit_length, padding=(0, 0), total_width=7, load_width=8, load_wait_w=1,
                               load_wait_a=1, out=None, workspace=None, stream=None, desc=None, accumulate="y",
                               z_unit=1, generator="lfsr", seed=0, options=None):
    """int32 (N, Cout, Wo, Ho) GPU tensor via geo_sc_conv2d_add_partial_forward_ex."""
    _require_gpu_f32(x, "x")
    _require_gpu_f32(w, "w")
    if desc is None:
        desc = make_desc(x.shape, w.shape, bit_length, padding, total_width, load_width, load_wait_w, load_wait_a,
                         accumulate, z_unit, generator, seed)
    if workspace is None:
        workspace = torch.empty(workspace_size(desc, options), dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty(output_shape(desc), dtype=torch.int32, device=x.device)
    _check(_native.lib().geo_sc_conv2d_add_partial_forward_ex(ctypes.byref(desc), _opt_ptr(options), _ptr(x), _ptr(w),
                                                              _ptr(out), _ptr(workspace), workspace.numel(),
                                                              _stream_ptr(stream)),
           "geo_sc_conv2d_add_partial_forward")
    return out


def static_workspace_bytes() -> int:
    """Size of the library's static device workspace (geo_sc_static_workspace_bytes)."""
    return int(_native.lib().geo_sc_static_workspace_bytes())


def init():
    """geo_sc_init: per-device lookups of the library on the current device (call before a stream capture)."""
    _check(_native.lib().geo_sc_init(), "geo_sc_init")


def conv2d_add_partial_forward_static(x, w, out, desc: ConvDesc, stream=None):
    """geo_sc_conv2d_add_partial_forward_static: the forward on the library's static device workspace;
    allocates nothing (``out`` is the caller's int32 tensor of output_shape(desc)).  The workspace is the
    current device's: all three tensors must live there."""
    _require_gpu_f32(x, "x")
    _require_gpu_f32(w, "w")
    cur = torch.cuda.current_device()
    if not (x.device.index == cur and w.device.index == cur and out.device.index == cur):
        raise ValueError("x, w and out must be on the current device (the static workspace is per device)")
    if not (out.is_cuda and out.dtype == torch.int32 and out.is_contiguous()
            and tuple(out.shape) == output_shape(desc)):
        raise ValueError("out must be a contiguous int32 GPU tensor of the output's shape")
    _check(_native.lib().geo_sc_conv2d_add_partial_forward_static(ctypes.byref(desc), _ptr(x), _ptr(w), _ptr(out),
                                                                  _stream_ptr(stream)),
           "geo_sc_conv2d_add_partial_forward_static")
    return out


def conv2d_add_partial_forward_q7(x_q7, w, bit_length, padding=(0, 0), total_width=7, load_width=8, load_wait_w=1,
                                  load_wait_a=1, out=None, workspace=None, stream=None, accumulate="y", z_unit=1):
    """The forward for activations given as uint8 integers k = round(x * 128), k <= 127
    (geo_sc_conv2d_add_partial_forward_q7): same counts as the fp32 entry point on k / 128."""
    if not (x_q7.is_cuda and x_q7.dtype == torch.uint8 and x_q7.is_contiguous()):
        raise ValueError("x_q7 must be a contiguous uint8 GPU tensor")
    _require_gpu_f32(w, "w")
    desc = make_desc(x_q7.shape, w.shape, bit_length, padding, total_width, load_width, load_wait_w, load_wait_a,
                     accumulate, z_unit)
    if workspace is None:
        workspace = torch.empty(workspace_size(desc), dtype=torch.uint8, device=w.device)
    if out is None:
        out = torch.empty(output_shape(desc), dtype=torch.int32, device=w.device)
    _check(_native.lib().geo_sc_conv2d_add_partial_forward_q7(ctypes.byref(desc), _ptr(x_q7), _ptr(w), _ptr(out),
                                                              _ptr(workspace), workspace.numel(),
                                                              _stream_ptr(stream)),
           "geo_sc_conv2d_add_partial_forward_q7")
    return out


# enum geo_sc_epilogue_flags
EPI_RELU, EPI_POOL2, EPI_HARDTANH01, EPI_QUANT7 = 1, 2, 4, 8


def layer_epilogue(counts, bit_length, w_n, b_n, relu=False, pool=True, hardtanh=True, quant7=True, want_act=True,
                   want_q7=False, stream=None):
    """geo_sc_layer_epilogue: int32 counts (N, C, W, H) -> (fp32 activation or None, uint8 7-bit
    integers or None), each (N, C, W', H'): count / L, per-channel w_n, b_n, then the selected
    relu / AvgPool2d(2) / Hardtanh(0, 1) / 7-bit quantisation."""
    if not (counts.is_cuda and counts.dtype == torch.int32 and counts.is_contiguous() and counts.dim() == 4):
        raise ValueError("counts must be a contiguous int32 GPU tensor (N, C, W, H)")
    n, c, w, h = counts.shape
    w_n = w_n.to(counts.device, torch.float32).contiguous()
    b_n = b_n.to(counts.device, torch.float32).contiguous()
    if w_n.numel() != c or b_n.numel() != c:
        raise ValueError("w_n and b_n need one entry per channel")
    flags = (EPI_RELU if relu else 0) | (EPI_POOL2 if pool else 0) | (EPI_HARDTANH01 if hardtanh else 0) | \
        (EPI_QUANT7 if quant7 else 0)
    shape = (n, c, w // 2, h // 2) if pool else (n, c, w, h)
    act = torch.empty(shape, dtype=torch.float32, device=counts.device) if want_act else None
    q7 = torch.empty(shape, dtype=torch.uint8, device=counts.device) if want_q7 else None
    _check(_native.lib().geo_sc_layer_epilogue(_ptr(counts), n, c, w, h, int(bit_length), _ptr(w_n), _ptr(b_n), flags,
                                               _ptr(act), _ptr(q7), _stream_ptr(stream)), "geo_sc_layer_epilogue")
    return act, q7


def layer_tail_backward(counts, grad_out, bit_length, w_n, b_n, mean, invstd, gamma=None, relu=False, pool=True,
                        hardtanh=True, stream=None):
    """geo_sc_layer_tail_backward: (grad_y, grad_gamma, grad_beta) of the training-mode layer tail
    (batch norm on the batch statistics, relu, AvgPool2d(2), Hardtanh(0, 1))."""
    n, c, w, h = counts.shape
    dev = counts.device
    f = lambda t: t.to(dev, torch.float32).contiguous()
    grad_out, w_n, b_n, mean, invstd = f(grad_out), f(w_n), f(b_n), f(mean), f(invstd)
    gamma = None if gamma is None else f(gamma)
    exp = (n, c, w // 2, h // 2) if pool else (n, c, w, h)
    if tuple(grad_out.shape) != exp:
        raise ValueError(f"grad_out has shape {tuple(grad_out.shape)}, expected {exp}")
    flags = (EPI_RELU if relu else 0) | (EPI_POOL2 if pool else 0) | (EPI_HARDTANH01 if hardtanh else 0)
    nbytes = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_layer_tail_backward_workspace_size(n, c, w, h, ctypes.byref(nbytes)), "tail workspace")
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
    grad_y = torch.empty((n, c, w, h), dtype=torch.float32, device=dev)
    gg = torch.empty(c, dtype=torch.float32, device=dev)
    gb = torch.empty(c, dtype=torch.float32, device=dev)
    _check(_native.lib().geo_sc_layer_tail_backward(_ptr(counts), _ptr(grad_out), n, c, w, h, int(bit_length), _ptr(w_n),
                                                    _ptr(b_n), _ptr(mean), _ptr(invstd), _ptr(gamma), flags,
                                                    _ptr(grad_y), _ptr(gg), _ptr(gb), _ptr(ws), ws.numel(),
                                                    _stream_ptr(stream)), "geo_sc_layer_tail_backward")
    return grad_y, gg, gb


def count_stats(counts, bit_length, stream=None):
    """geo_sc_count_stats: per-channel mean and biased variance of ``counts / bit_length`` over batch and
    positions, from exact integer sums.  ``counts``: contiguous int32 GPU tensor (n, c, w, h) or (n, c)."""
    if not (counts.is_cuda and counts.dtype == torch.int32 and counts.is_contiguous() and counts.dim() in (2, 4)):
        raise ValueError("counts must be a contiguous int32 GPU tensor (n, c, w, h) or (n, c)")
    n, c = counts.shape[:2]
    w, h = (counts.shape[2], counts.shape[3]) if counts.dim() == 4 else (1, 1)
    need = ctypes.c_size_t()
    _check(_native.lib().geo_sc_count_stats_workspace_size(n, c, w, h, ctypes.byref(need)),
           "geo_sc_count_stats_workspace_size")
    ws = torch.empty(max(need.value, 8), dtype=torch.uint8, device=counts.device)
    mean = torch.empty(c, dtype=torch.float32, device=counts.device)
    var = torch.empty(c, dtype=torch.float32, device=counts.device)
    _check(_native.lib().geo_sc_count_stats(_ptr(counts), n, c, w, h, int(bit_length), _ptr(mean), _ptr(var), _ptr(ws),
                                            ws.numel(), _stream_ptr(stream)), "geo_sc_count_stats")
    return mean, var


def bn_fixed_affine(mean, var, gamma, beta, eps, elements_per_channel, running_mean=None, running_var=None,
                    eps_grad=1e-5, stream=None):
    """geo_sc_bn_fixed_affine: (w_n, b_n, invstd, scale) of a fixed-point batch norm from channel
    statistics; updates running_mean / running_var in place when given."""
    c = mean.numel()
    dev = mean.device
    for t in (mean, var, gamma, beta, running_mean, running_var):
        if t is not None and not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == c):
            raise ValueError("statistics and parameters must be contiguous float32 GPU tensors of one size")
    w_n = torch.empty(c, dtype=torch.float32, device=dev)
    b_n = torch.empty(c, dtype=torch.float32, device=dev)
    invstd = torch.empty(c, dtype=torch.float32, device=dev)
    scale = torch.empty((), dtype=torch.float32, device=dev)
    _check(_native.lib().geo_sc_bn_fixed_affine(_ptr(mean), _ptr(var), _ptr(gamma), _ptr(beta), c, float(eps),
                                                float(eps_grad), int(elements_per_channel), _ptr(running_mean),
                                                _ptr(running_var), _ptr(w_n), _ptr(b_n), _ptr(invstd), _ptr(scale),
                                                _stream_ptr(stream)), "geo_sc_bn_fixed_affine")
    return w_n, b_n, invstd, scale


def bn_fixed_from_counts(counts, bit_length, gamma, beta, eps, running_mean=None, running_var=None, eps_grad=1e-5,
                         stream=None):
    """geo_sc_bn_fixed_from_counts: (mean, var, w_n, b_n, invstd, scale) of a fixed-point batch norm on the batch
    statistics of ``counts / bit_length`` (exact integer sums), updating running_mean / running_var in place
    when given: count_stats + bn_fixed_affine in two launches."""
    if not (counts.is_cuda and counts.dtype == torch.int32 and counts.is_contiguous() and counts.dim() in (2, 4)):
        raise ValueError("counts must be a contiguous int32 GPU tensor (n, c, w, h) or (n, c)")
    n, c = counts.shape[:2]
    w, h = (counts.shape[2], counts.shape[3]) if counts.dim() == 4 else (1, 1)
    dev = counts.device
    for t in (gamma, beta, running_mean, running_var):
        if t is not None and not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == c):
            raise ValueError("parameters and running statistics must be contiguous float32 GPU tensors of c entries")
    need = ctypes.c_size_t()
    _check(_native.lib().geo_sc_count_stats_workspace_size(n, c, w, h, ctypes.byref(need)),
           "geo_sc_count_stats_workspace_size")
    ws = torch.empty(max(need.value, 8), dtype=torch.uint8, device=dev)
    out = torch.empty((5, c), dtype=torch.float32, device=dev)   # mean, var, w_n, b_n, invstd
    scale = torch.empty((), dtype=torch.float32, device=dev)
    mean, var, w_n, b_n, invstd = out[0], out[1], out[2], out[3], out[4]
    _check(_native.lib().geo_sc_bn_fixed_from_counts(_ptr(counts), n, c, w, h, int(bit_length), _ptr(gamma), _ptr(beta),
                                                     float(eps), float(eps_grad), _ptr(running_mean),
                                                     _ptr(running_var), _ptr(mean), _ptr(var), _ptr(w_n), _ptr(b_n),
                                                     _ptr(invstd), _ptr(scale), _ptr(ws), ws.numel(),
                                                     _stream_ptr(stream)), "geo_sc_bn_fixed_from_counts")
    return mean, var, w_n, b_n, invstd, scale


def quantize_many(tensors, prec, stream=None):
    """geo_sc_quantize_many: quantize() of every tensor of the list (contiguous fp32 GPU tensors) in one launch;
    returns the new tensors."""
    for t in tensors:
        _require_gpu_f32(t, "tensor")
    outs = [torch.empty_like(t) for t in tensors]
    n = len(tensors)
    if n:
        arr = ctypes.c_void_p * n
        sizes = (ctypes.c_size_t * n)(*[t.numel() for t in tensors])
        _check(_native.lib().geo_sc_quantize_many(n, arr(*[t.data_ptr() for t in tensors]),
                                                  arr(*[o.data_ptr() for o in outs]), sizes, int(prec),
                                                  _stream_ptr(stream)), "geo_sc_quantize_many")
    return outs


def copy_back_clamp(masters, params, orgs, lo, hi, stream=None):
    """geo_sc_copy_back_clamp: params[i] <- masters[i], and orgs[i] <- clamp(masters[i], lo, hi) where orgs[i] is
    not None, for all i in one launch (contiguous float32 GPU tensors of equal sizes per i)."""
    n = len(masters)
    if n == 0:
        return
    for m, p, o in zip(masters, params, orgs):
        for t in (m, p) + ((o,) if o is not None else ()):
            if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == m.numel()):
                raise ValueError("master copies, parameters and buffers must be contiguous float32 GPU tensors")
    arr = ctypes.c_void_p * n
    sizes = (ctypes.c_size_t * n)(*[m.numel() for m in masters])
    _check(_native.lib().geo_sc_copy_back_clamp(n, arr(*[m.data_ptr() for m in masters]),
                                                arr(*[p.data_ptr() for p in params]),
                                                arr(*[o.data_ptr() if o is not None else None for o in orgs]), sizes,
                                                float(lo), float(hi), _stream_ptr(stream)), "geo_sc_copy_back_clamp")


def quantize(x, prec, out=None, stream=None):
    """geo_sc_quantize: round(x * 2^prec) clamped to +-(2^prec - 1), over 2^prec, in one launch.
    ``x`` is a contiguous fp32 GPU tensor; ``out`` may be ``x`` itself."""
    _require_gpu_f32(x, "x")
    if out is None:
        out = torch.empty_like(x)
    elif not (out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and out.shape == x.shape):
        raise ValueError("out must be a contiguous fp32 GPU tensor of x's shape")
    _check(_native.lib().geo_sc_quantize(_ptr(x), _ptr(out), x.numel(), int(prec), _stream_ptr(stream)),
           "geo_sc_quantize")
    return out


def act_streams(x, desc: ConvDesc, stream=None):
    """int32-typed tensor of stream words (reinterpret as uint32), shaped as the library stores them:
    (N, P, Cin, Wi, Hi), or (P, Cin, Wi, Hi, N) for the geometries whose streams are batch-item-innermost
    (geo_sc_act_stream_layout: single-row outputs of 1/3/5-wide kernels with N >= 2).  ``x`` is fp32, or
    uint8 holding the 7-bit integers round(x * 128)."""
    q7 = x.dtype == torch.uint8
    if q7:
        if not (x.is_cuda and x.is_contiguous()):
            raise ValueError("x must be a contiguous GPU tensor")
    else:
        _require_gpu_f32(x, "x")
    n = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_act_stream_words(ctypes.byref(desc), ctypes.byref(n)), "act words")
    packs = (desc.bit_length + 31) // 32
    wi, hi = desc.w_in + 2 * desc.pad_w, desc.h_in + 2 * desc.pad_h
    inner = ctypes.c_int(0)
    _check(_native.lib().geo_sc_act_stream_layout(ctypes.byref(desc), ctypes.byref(inner)), "act layout")
    shape = (packs, desc.c_in, wi, hi, desc.n) if inner.value else (desc.n, packs, desc.c_in, wi, hi)
    out = torch.empty(shape, dtype=torch.int32, device=x.device)
    assert out.numel() == n.value
    fn = _native.lib().geo_sc_act_streams_q7 if q7 else _native.lib().geo_sc_act_streams
    _check(fn(ctypes.byref(desc), _ptr(x), _ptr(out), None, _stream_ptr(stream)), "geo_sc_act_streams")
    return out


def weight_streams(w, desc: ConvDesc, stream=None):
    """int32-typed tensor of stream words [P][H][Cin*W][ceil(Cout/16)][2][16] (the line order
    inside a pack depends on the accumulation mode; the shape is that of mode "y")."""
    _require_gpu_f32(w, "w")
    n = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_weight_stream_words(ctypes.byref(desc), ctypes.byref(n)), "weight words")
    packs = (desc.bit_length + 31) // 32
    shape = (packs, desc.h_k, desc.c_in * desc.w_k, (desc.c_out + 15) // 16, 2, 16)
    classic = packs * desc.h_k * desc.c_in * desc.w_k * ((desc.c_out + 15) // 16) * 32
    # the buffer may continue behind the two-rail lines (rail-packed copy for large y-mode launches);
    # the returned view shows the lines and keeps the whole buffer alive
    buf = torch.empty(n.value, dtype=torch.int32, device=w.device)
    assert n.value >= classic
    out = buf[:classic].view(shape)
    _check(_native.lib().geo_sc_weight_streams(ctypes.byref(desc), _ptr(w), _ptr(out), None, _stream_ptr(stream)),
           "geo_sc_weight_streams")
    return out


def weight_streams_from_lines(lines, desc: ConvDesc, stream=None):
    """A complete weight stream buffer from two-rail lines [P][H][K][ceil(Cout/16)][2][16] written by the
    caller (int32-typed GPU tensor): copies them into a buffer of geo_sc_weight_stream_words words and
    lets geo_sc_weight_streams_finish fill the rest.  Returns the view of the lines, as weight_streams()."""
    n = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_weight_stream_words(ctypes.byref(desc), ctypes.byref(n)), "weight words")
    if not (lines.is_cuda and lines.dtype == torch.int32 and lines.is_contiguous()) or lines.numel() > n.value:
        raise ValueError("lines must be a contiguous int32 GPU tensor of the two-rail layout")
    buf = torch.empty(n.value, dtype=torch.int32, device=lines.device)
    out = buf[:lines.numel()].view(lines.shape)
    out.copy_(lines)
    _check(_native.lib().geo_sc_weight_streams_finish(ctypes.byref(desc), _ptr(out), _stream_ptr(stream)),
           "geo_sc_weight_streams_finish")
    return out


def weight_streams_ok(wgt, desc: ConvDesc, stream=None) -> bool:
    """geo_sc_weight_streams_check on a buffer view as weight_streams() / weight_streams_from_lines()
    return it: False when a caller-written line has two non-zero rails for one channel.  Waits for the
    stream."""
    n = ctypes.c_size_t(0)
    # the descriptor on its own first: after this, GEO_SC_ERR_INVALID_ARGUMENT can only mean a flagged buffer
    _check(_native.lib().geo_sc_weight_stream_words(ctypes.byref(desc), ctypes.byref(n)), "weight words")
    rc = _native.lib().geo_sc_weight_streams_check(ctypes.byref(desc), _ptr(wgt), _stream_ptr(stream))
    if rc == 1:
        return False
    _check(rc, "geo_sc_weight_streams_check")
    return True


def skips_zero_rail(desc: ConvDesc) -> bool:
    """True when the forward of this geometry runs the kernel that processes only the non-zero rail
    of every weight (its weight stream buffer then carries the rail-packed copy)."""
    n = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_weight_stream_words(ctypes.byref(desc), ctypes.byref(n)), "weight words")
    packs = (desc.bit_length + 31) // 32
    return n.value > packs * desc.h_k * desc.c_in * desc.w_k * ((desc.c_out + 15) // 16) * 32


def conv2d_add_partial_from_streams(act, wgt, desc: ConvDesc, out=None, stream=None):
    """The AND/OR/popcount kernel alone on pre-generated streams (int32-typed words)."""
    if out is None:
        out = torch.empty(output_shape(desc), dtype=torch.int32, device=act.device)
    n = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_weight_stream_words(ctypes.byref(desc), ctypes.byref(n)), "weight words")
    if wgt.untyped_storage().nbytes() - wgt.storage_offset() * wgt.element_size() < 4 * n.value:
        raise ValueError("weight streams: the buffer behind this tensor is smaller than geo_sc_weight_stream_words "
                         "(take it from weight_streams())")
    _check(_native.lib().geo_sc_conv2d_add_partial_from_streams(ctypes.byref(desc), _ptr(act), _ptr(wgt), _ptr(out),
                                                                _stream_ptr(stream)),
           "geo_sc_conv2d_add_partial_from_streams")
    return out


def backward_workspace_size(desc: ConvDesc, options: Options = None) -> int:
    out = ctypes.c_size_t(0)
    _check(_native.lib().geo_sc_conv2d_add_partial_backward_workspace_size_ex(ctypes.byref(desc), _opt_ptr(options),
                                                                              ctypes.byref(out)),
           "backward workspace query")
    return out.value


def conv2d_add_partial_backward(x, w, grad_y, bit_length=128, padding=(0, 0), need_grad_x=True, need_grad_w=True,
                                workspace=None, stream=None, desc=None, accumulate="y", z_unit=1, options=None):
    """(grad_x, grad_w) of the surrogate via geo_sc_conv2d_add_partial_backward_ex; an output
    that is not needed is returned as None."""
    _require_gpu_f32(x, "x")
    _require_gpu_f32(w, "w")
    _require_gpu_f32(grad_y, "grad_y")
    if desc is None:
        desc = make_desc(x.shape, w.shape, bit_length, padding, accumulate=accumulate, z_unit=z_unit)
    if tuple(grad_y.shape) != output_shape(desc):
        raise ValueError(f"grad_y has shape {tuple(grad_y.shape)}, expected {output_shape(desc)}")
    if workspace is None:
        workspace = torch.empty(backward_workspace_size(desc, options), dtype=torch.uint8, device=x.device)
    gx = torch.empty_like(x) if need_grad_x else None
    gw = torch.empty_like(w) if need_grad_w else None
    _check(_native.lib().geo_sc_conv2d_add_partial_backward_ex(ctypes.byref(desc), _opt_ptr(options), _ptr(x), _ptr(w),
                                                               _ptr(grad_y), _ptr(gx), _ptr(gw), _ptr(workspace),
                                                               workspace.numel(), _stream_ptr(stream)),
           "geo_sc_conv2d_add_partial_backward")
    return gx, gw


def probe_and_or_rate(iters=20000, stream=None):
    """Sustained v_and_or_b32 rate (32-bit lane operations per second) of a memory-free loop,
    timed with events on the launch stream."""
    scratch = torch.zeros(128 + 4096 * 64 * 4, dtype=torch.uint8, device="cuda")
    ops = ctypes.c_double(0)

    def launch(n):
        _check(_native.probe_lib().geo_sc_probe_and_or_rate(n, _ptr(scratch), scratch.numel(), ctypes.byref(ops),
                                                      _stream_ptr(stream)), "geo_sc_probe_and_or_rate")
    launch(200)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    launch(iters)
    e1.record()
    torch.cuda.synchronize()
    return ops.value / (e0.elapsed_time(e1) * 1e-3)


# tile of the matrix-core probe (csrc/sc_probe.hip): 128 positions x 256 rail-columns, 384 members, operand rows of
# 384 fp4 values padded to 208 bytes
PROBE_MFMA_ROWS, PROBE_MFMA_COLS, PROBE_MFMA_K, PROBE_MFMA_ROW_BYTES = 128, 256, 384, 208


def probe_mfma_operands(n_a, n_b, seed=0, p_a=1 / 8, p_b=1 / 16):
    """Random 0 / 1 operand tiles of the probe as fp4 (1.0 = 0x2), uint8 GPU tensors (n, rows, 208)."""
    g = torch.Generator().manual_seed(seed)

    def tiles(n, rows, p):
        bits = (torch.rand((n, rows, PROBE_MFMA_K), generator=g) < p).to(torch.uint8)
        packed = bits[..., 0::2] * 0x2 + bits[..., 1::2] * 0x20
        out = torch.zeros((n, rows, PROBE_MFMA_ROW_BYTES), dtype=torch.uint8)
        out[..., :PROBE_MFMA_K // 2] = packed
        return out.cuda(), bits

    a, a_bits = tiles(n_a, PROBE_MFMA_ROWS, p_a)
    b, b_bits = tiles(n_b, PROBE_MFMA_COLS, p_b)
    return a, b, a_bits, b_bits


def probe_mfma_slices(mode, a, b, workgroups, slices, reload_sixteenths=16, out=None, stream=None):
    """geo_sc_probe_mfma_slices: `slices` (cycle, kernel row) slices of the forward as fp4 GEMM tiles per workgroup;
    returns the int32 counts (workgroups, 128, 256)."""
    if out is None:
        out = torch.empty((workgroups, PROBE_MFMA_ROWS, PROBE_MFMA_COLS), dtype=torch.int32, device="cuda")
    _check(_native.probe_lib().geo_sc_probe_mfma_slices(int(mode), int(reload_sixteenths), int(workgroups), int(slices),
                                                        _ptr(a), a.shape[0], _ptr(b), b.shape[0], _ptr(out),
                                                        _stream_ptr(stream)), "geo_sc_probe_mfma_slices")
    return out
