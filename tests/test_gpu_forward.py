"""GPU parity of the HIP forward path, driven through the C ABI (geo_amd.capi) and through
the PyTorch modules with the reference's names.  Everything is compared bit-for-bit with
the CPU oracle, the reference-kernel fixtures and the reference-kernel checksums."""
import ctypes
import hashlib

import numpy as np
import pytest
import torch

from geo_amd import workloads as wl

pytestmark = pytest.mark.gpu

LENGTHS = (8, 16, 32, 64, 128, 256)


@pytest.fixture(scope="module")
def capi():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from geo_amd import capi as m
    return m


@pytest.fixture(scope="module")
def so():
    from oracle import sc_oracle
    return sc_oracle


def gpu_forward(capi, x, w, L, pad, **kw):
    if isinstance(pad, int):
        pad = (pad, pad)
    xd = torch.as_tensor(x).float().contiguous().cuda()
    wd = torch.as_tensor(w).float().contiguous().cuda()
    y = capi.conv2d_add_partial_forward(xd, wd, L, pad, **kw)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def u32(t):
    return t.cpu().numpy().view(np.uint32)


# ------------------------------------------------------------------ stream generators
@pytest.mark.parametrize("L", LENGTHS)
@pytest.mark.parametrize("loading", [(7, 8, 1, 1), (7, 2, 2, 2), (7, 1, 3, 5), (7, 3, 40, 7)])
def test_activation_streams_match_oracle(capi, so, L, loading):
    tw, lw, ww, wa = loading
    x, _ = wl.make_inputs((3, 5, 7, 6), (2, 5, 3, 3), "prescribed", seed=L)
    x.view(-1)[::13] = 0.0
    x.view(-1)[5::17] = 1.0
    d = capi.make_desc(x.shape, (2, 5, 3, 3), L, (2, 1), tw, lw, ww, wa)
    got = u32(capi.act_streams(x.cuda(), d))
    xp = np.pad(x.numpy(), ((0, 0), (0, 0), (1, 1), (2, 2)))
    for n in range(x.shape[0]):
        exp = so.act_streams(xp[n], L, tw, lw, wa)
        assert np.array_equal(got[n], exp), (L, loading, n)


def test_activation_streams_item_innermost_layout(capi, so):
    """Outputs with a single row (here 3-wide input, 3-wide kernel, no padding) get their
    streams as [P][Cin][Wi][Hi][N]: same words, batch item innermost."""
    L = 64
    x, _ = wl.make_inputs((5, 4, 3, 6), (2, 4, 3, 3), "prescribed", seed=77)
    d = capi.make_desc(x.shape, (2, 4, 3, 3), L, (0, 0))
    got = u32(capi.act_streams(x.cuda(), d))
    assert got.shape == (2, 4, 3, 6, 5)
    for n in range(5):
        assert np.array_equal(got[..., n], so.act_streams(x[n].numpy(), L))


@pytest.mark.parametrize("L", LENGTHS)
@pytest.mark.parametrize("loading", [(7, 8, 1, 1), (7, 2, 2, 2), (7, 1, 3, 5)])
def test_weight_streams_match_oracle(capi, so, L, loading):
    tw, lw, ww, wa = loading
    _, w = wl.make_inputs((1, 6, 4, 4), (19, 6, 3, 2), "prescribed", seed=100 + L)
    w.view(-1)[::7] = 0.0
    d = capi.make_desc((1, 6, 4, 4), w.shape, L, (0, 0), tw, lw, ww, wa)
    got = u32(capi.weight_streams(w.cuda(), d))          # [P][H][K][cot][2][16]
    wpos, wneg = so.weight_streams(w.numpy(), L, tw, lw, ww)  # [P][H][Cin][W][Cout]
    P, H, Cin, W, Cout = wpos.shape
    got = got.reshape(P, H, Cin, W, -1, 2, 16)
    gp = got[..., 0, :].reshape(P, H, Cin, W, -1)
    gn = got[..., 1, :].reshape(P, H, Cin, W, -1)
    assert np.array_equal(gp[..., :Cout], wpos)
    assert np.array_equal(gn[..., :Cout], wneg)
    assert not gp[..., Cout:].any() and not gn[..., Cout:].any()   # c_out padding is zero


def test_conv_kernel_alone_on_oracle_streams(capi, so):
    """The AND/OR/popcount kernel fed with streams produced by the CPU oracle; the last wave
    is partly empty and starts in the third item."""
    L = 64
    x, w = wl.make_inputs((3, 5, 8, 7), (18, 5, 3, 3), "prescribed", seed=31)
    d = capi.make_desc(x.shape, w.shape, L, (1, 1))
    xp = np.pad(x.numpy(), ((0, 0), (0, 0), (1, 1), (1, 1)))
    act = np.stack([so.act_streams(xp[n], L) for n in range(x.shape[0])])           # [N][P][Cin][Wi][Hi]
    wpos, wneg = so.weight_streams(w.numpy(), L)                                     # [P][H][Cin][W][Cout]
    P, H, Cin, W, Cout = wpos.shape
    K, ncot = Cin * W, (Cout + 15) // 16
    pad_c = ncot * 16 - Cout
    tiled = np.zeros((P, H, K, ncot, 2, 16), dtype=np.uint32)
    tiled[..., 0, :] = np.pad(wpos.reshape(P, H, K, Cout), ((0, 0),) * 3 + ((0, pad_c),)).reshape(P, H, K, ncot, 16)
    tiled[..., 1, :] = np.pad(wneg.reshape(P, H, K, Cout), ((0, 0),) * 3 + ((0, pad_c),)).reshape(P, H, K, ncot, 16)
    wgt = capi.weight_streams_from_lines(torch.from_numpy(tiled.view(np.int32)).cuda(), d)
    y = capi.conv2d_add_partial_from_streams(torch.from_numpy(act.view(np.int32)).cuda(), wgt, d)
    exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, (1, 1))
    assert np.array_equal(y.cpu().numpy(), exp)


def test_caller_written_lines_with_two_rails_are_reported(capi):
    """The rail-packed copy holds one rail per (line, channel); geo_sc_weight_streams_finish records a
    line that has two and geo_sc_weight_streams_check reports it."""
    d = capi.make_desc((2, 4, 6, 6), (20, 4, 3, 3), 64, (1, 1))
    lines = torch.zeros((2, 3, 12, 2, 2, 16), dtype=torch.int32)
    lines[1, 2, 7, 1, 0, 3] = 0x00f0
    lines[0, 0, 0, 0, 1, 0] = 0x0001
    good = capi.weight_streams_from_lines(lines.cuda(), d)
    assert capi.weight_streams_ok(good, d)
    lines[1, 2, 7, 1, 1, 3] = 0x0100            # same line and channel, other rail
    bad = capi.weight_streams_from_lines(lines.cuda(), d)
    assert not capi.weight_streams_ok(bad, d)
    _, w = wl.make_inputs((2, 4, 6, 6), (20, 4, 3, 3), "prescribed", seed=5)
    assert capi.weight_streams_ok(capi.weight_streams(w.cuda(), d), d)   # generated buffers always pass
    # a kernel width without rail-packed copy has nothing to break
    d7 = capi.make_desc((1, 2, 9, 9), (3, 2, 7, 7), 16, (3, 3))
    _, w7 = wl.make_inputs((1, 2, 9, 9), (3, 2, 7, 7), "prescribed", seed=5)
    assert capi.weight_streams_ok(capi.weight_streams(w7.cuda(), d7), d7)


# ------------------------------------------------------------------ forward: fixtures
def test_forward_matches_reference_fixtures(capi, fixtures_small):
    for name, d in fixtures_small.items():
        y = gpu_forward(capi, d["x"], d["w"], d["L"], d["pad"])
        assert y.dtype == np.int32 and y.shape == d["y"].shape
        assert np.array_equal(y, d["y"]), name


@pytest.mark.parametrize("shape_x,shape_w,pad,L,mode", [
    ((3, 5, 9, 7), (6, 5, 3, 3), (1, 1), 64, "prescribed"),
    ((2, 4, 8, 8), (17, 4, 5, 5), (2, 2), 32, "prescribed"),     # two c_out tiles, one partial
    ((2, 3, 7, 9), (5, 3, 1, 1), (0, 0), 128, "kaiming"),        # 1x1
    ((2, 6, 5, 8), (4, 6, 2, 4), (1, 0), 256, "prescribed"),     # even kernel, asymmetric pad
    ((1, 2, 9, 9), (3, 2, 7, 7), (3, 3), 16, "prescribed"),      # run-time kernel width
    ((5, 16, 1, 8), (33, 16, 1, 8), (0, 0), 128, "prescribed"),  # SC-linear mapping
    ((2, 3, 11, 5), (4, 3, 3, 5), (0, 2), 8, "prescribed"),      # odd row count, L=8
    ((70, 2, 3, 3), (3, 2, 3, 3), (0, 0), 64, "sparse"),         # waves spanning items
    ((7, 5, 3, 9), (4, 5, 3, 3), (0, 0), 64, "prescribed"),      # single output row: lanes pair up batch items (odd N)
    ((3, 5, 5, 9), (4, 5, 5, 3), (0, 0), 32, "prescribed"),      # same with a 5-wide kernel
    ((9, 8, 1, 6), (3, 8, 1, 2), (0, 0), 128, "prescribed"),     # 1-wide kernel, channels in trips of 3 + tail
    ((5, 4, 4, 4), (3, 4, 4, 4), (0, 0), 32, "prescribed"),      # classifier-style layer, run-time width
    ((1, 1, 1, 1), (1, 1, 1, 1), (0, 0), 8, "prescribed"),       # smallest possible
    ((2, 10, 6, 6), (5, 10, 1, 1), (0, 0), 64, "kaiming"),       # 1x1 conv, 10 channels = 3 trips + 1
])
def test_forward_matches_oracle(capi, so, shape_x, shape_w, pad, L, mode):
    x, w = wl.make_inputs(shape_x, shape_w, mode, seed=L + shape_x[0])
    exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad)
    got = gpu_forward(capi, x, w, L, pad)
    assert np.array_equal(got, exp)


@pytest.mark.parametrize("shape_x,shape_w,pad,L", [
    ((300, 16, 1, 40), (20, 16, 1, 40), (0, 0), 128),   # 3 position tiles, second items past the end, 160 groups
    ((130, 7, 1, 9), (33, 7, 1, 9), (0, 0), 256),       # channel trips 3 2 2, 72 groups, three c_out tiles
    ((64, 4, 3, 12), (5, 4, 3, 5), (0, 0), 64),         # 3-wide kernel, output (1, 8): lanes span output columns
    ((2, 3, 1, 2), (1, 3, 1, 2), (0, 0), 32),           # fewer groups than waves in the workgroup
    ((257, 5, 5, 6), (17, 5, 5, 6), (0, 0), 16),        # 5-wide kernel, odd batch
    ((2000, 16, 1, 5), (1024, 16, 1, 5), (0, 0), 64),   # groups of 16, 64 c_out tiles: the LDS-staged workgroups
    ((4100, 16, 1, 2), (520, 16, 1, 2), (0, 0), 32),    # same with two groups only; 33 c_out tiles: not staged
])
def test_forward_item_innermost_streams_match_oracle(capi, so, shape_x, shape_w, pad, L):
    """Single-row outputs (the SC-linear mapping): the workgroup kernel whose waves split the (pack,
    kernel row) groups and add their partial sums in LDS."""
    mode = "kaiming" if L >= 128 else "prescribed" if shape_x[0] == 2 else "sparse"
    x, w = wl.make_inputs(shape_x, shape_w, mode, seed=L + shape_x[0])
    d = capi.make_desc(shape_x, shape_w, L, pad)
    assert capi.act_streams(x.cuda(), d).shape[-1] == shape_x[0]     # item-innermost geometry
    exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad)
    got = gpu_forward(capi, x, w, L, pad)
    assert np.array_equal(got, exp)
    assert np.abs(exp).sum() > 0


@pytest.mark.parametrize("shape_x,shape_w,L", [
    ((2000, 16, 1, 5), (1024, 16, 1, 5), 64),     # the LDS-staged workgroups
    ((130, 7, 1, 9), (33, 7, 1, 9), 128),         # the general workgroup kernel
])
def test_item_innermost_streams_with_loading_and_7bit_activations(capi, so, shape_x, shape_w, L):
    """The single-row kernels behind the other ways into the forward: progressive loading (weights and
    activations with different waits) and the uint8 entry point (activations k / 128)."""
    x, w = wl.make_inputs(shape_x, shape_w, "q7", seed=L)
    w = (w * 4).clamp(-0.99, 0.99).contiguous()
    kw = dict(total_width=7, load_width=2, load_wait_w=2, load_wait_a=3)
    exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, (0, 0), **kw)
    assert np.abs(exp).sum() > 0
    got = gpu_forward(capi, x, w, L, (0, 0), **kw)
    assert np.array_equal(got, exp)
    k = (x * 128).round().to(torch.uint8)
    got_q7 = capi.conv2d_add_partial_forward_q7(k.cuda(), w.cuda(), L, (0, 0), **kw)
    assert np.array_equal(got_q7.cpu().numpy(), exp)


@pytest.mark.parametrize("loading", [(7, 2, 2, 2), (7, 1, 4, 4), (7, 4, 3, 3), (7, 2, 1, 1)])
@pytest.mark.parametrize("L", [16, 64, 128])
def test_forward_progressive_loading_matches_oracle(capi, so, loading, L):
    """Pinned by the reference's GPU source text only (sc_cuda_kernel.cu:155-165): no CPU
    code in the reference executes progressive loading."""
    tw, lw, ww, wa = loading
    x, w = wl.make_inputs((2, 4, 6, 6), (5, 4, 3, 3), "prescribed", seed=7)
    kw = dict(total_width=tw, load_width=lw, load_wait_w=ww, load_wait_a=wa)
    exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, (1, 1), **kw)
    got = gpu_forward(capi, x, w, L, (1, 1), **kw)
    assert np.array_equal(got, exp)
    neutral = gpu_forward(capi, x, w, L, (1, 1))
    assert not np.array_equal(got, neutral) or L == 16


def _window(words_msb_first, first, count):
    """bits first .. first+count-1 (cycle numbers from 1) of a 128-cycle stream given as 4 uint32 words"""
    bits = [(int(words_msb_first[c // 32]) >> (31 - c % 32)) & 1 for c in range(128)]
    return bits[first - 1:first - 1 + count]


def test_progressive_loading_literal_known_answers(capi):
    """The hand-derived bits of tests/loading_vectors.py (from sc_cuda_kernel.cu:155-160, :681-685) on
    the GPU generators.  Activation element 0 has seed 1; the positive rail of input channel 60 and the
    negative rail of input channel 90 of a 1x1 kernel have seed 1 as well ((67 + 60) % 127 + 1,
    (37 + 90) % 127 + 1)."""
    from tests import loading_vectors as lv

    L = 128
    for (tw, lw, wait), first, table in lv.VECTORS:
        codes = sorted(table)
        # activations: one item per code, a single element each
        x = torch.tensor(codes, dtype=torch.float32).view(-1, 1, 1, 1) / L
        d = capi.make_desc(x.shape, (1, 1, 1, 1), L, (0, 0), tw, lw, 1, wait)
        # single-row output, several items: the words are stored batch-item-innermost, [P][1][1][1][N]
        got = u32(capi.act_streams(x.cuda(), d))
        assert got.shape == (4, 1, 1, 1, len(codes))
        got = got.reshape(4, len(codes)).T
        for i, code in enumerate(codes):
            assert _window(got[i], first, len(table[code])) == table[code], ("act", (tw, lw, wait), first, code)
        # weights: output channel i carries code i on the positive rail of channel 60 and on the
        # negative rail of channel 90
        w = torch.zeros((len(codes), 91, 1, 1))
        w[:, 60, 0, 0] = torch.tensor(codes, dtype=torch.float32) / L
        w[:, 90, 0, 0] = -torch.tensor(codes, dtype=torch.float32) / L
        d = capi.make_desc((1, 91, 1, 1), w.shape, L, (0, 0), tw, lw, wait, 1)
        lines = u32(capi.weight_streams(w.cuda(), d)).reshape(4, 1, 91, 1, 2, 16)   # [P][H][K][cot][rail][16]
        for i, code in enumerate(codes):
            assert _window(lines[:, 0, 60, 0, 0, i], first, len(table[code])) == table[code], ("w+", first, code)
            assert _window(lines[:, 0, 90, 0, 1, i], first, len(table[code])) == table[code], ("w-", first, code)
            assert not lines[:, 0, 60, 0, 1, i].any() and not lines[:, 0, 90, 0, 0, i].any()


# ------------------------------------------------------------------ forward: full sizes
@pytest.mark.parametrize("name", [
    "C1_prescribed_L64", "C3_sparse_L32", "C3_sparse_L128", "C3_sparse_L256", "C3_kaiming_L128",
    "C3_kaiming_L256", "C3_q7_L128", "C3_q7_L256", "C3_prescribed_L128", "C4_prescribed_L128",
    "C5_kaiming_L256", "C5_sparse_L256", "C5_prescribed_L256",
])
def test_forward_full_size_checksums(capi, checksums, name):
    """SHA-256 of the int32 output against the reference CPU kernel's, inputs regenerated
    from the seed."""
    c = checksums[name]
    x, w, pad, _ = wl.named(c["shape_name"], c["mode"])
    y = gpu_forward(capi, x, w, c["L"], pad)
    assert list(y.shape) == c["shape"]
    assert int(y.astype(np.int64).sum()) == c["sum"]
    assert int(np.abs(y.astype(np.int64)).sum()) == c["abs_sum"]
    assert hashlib.sha256(np.ascontiguousarray(y).tobytes()).hexdigest() == c["sha256"]


def test_forward_full_size_properties(capi):
    """Size-independent properties at the headline shape: identical seeds for every batch
    item, c_out equivariance, the |y| <= H*L bound, zero input -> zero output."""
    x, w, pad, L = wl.named("C3", "kaiming")
    y = gpu_forward(capi, x, w, L, pad)
    assert np.abs(y).max() <= 3 * L
    perm = torch.randperm(x.shape[0], generator=torch.Generator().manual_seed(1))
    yp = gpu_forward(capi, x[perm], w, L, pad)
    assert np.array_equal(yp, y[perm.numpy()])
    cperm = torch.randperm(w.shape[0], generator=torch.Generator().manual_seed(2))
    yc = gpu_forward(capi, x, w[cperm], L, pad)
    assert np.array_equal(yc, y[:, cperm.numpy()])
    assert not gpu_forward(capi, torch.zeros_like(x), w, L, pad).any()
    x2 = x.clone()
    x2[1:] = x[0]
    y2 = gpu_forward(capi, x2, w, L, pad)
    assert np.array_equal(y2[5], y2[0]) and np.array_equal(y2[0], y[0])


# ------------------------------------------------------------------ boundary behaviour
def test_c_abi_error_codes(capi):
    x = torch.zeros((1, 2, 4, 4), device="cuda")
    w = torch.zeros((3, 2, 3, 3), device="cuda")
    with pytest.raises(capi.GeoScError) as e:
        capi.conv2d_add_partial_forward(x, w, 100)
    assert e.value.status == 2
    with pytest.raises(capi.GeoScError) as e:
        capi.conv2d_add_partial_forward(x, torch.zeros((3, 2, 5, 5), device="cuda"), 64)
    assert e.value.status == 1
    with pytest.raises(capi.GeoScError) as e:
        capi.conv2d_add_partial_forward(x, w, 64, load_wait_w=0)
    assert e.value.status == 1
    with pytest.raises(capi.GeoScError) as e:
        capi.conv2d_add_partial_forward(x, w, 64, workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    assert e.value.status == 3


def test_torch_modules_with_reference_names(capi, so, fixtures_small):
    from geo_amd import _native
    sc_cuda = _native.module("sc_extension_cuda")
    sc_cpu_name = _native.module("sc_extension")
    d = fixtures_small["T2"]
    x, w = torch.from_numpy(d["x"]), torch.from_numpy(d["w"])
    pad = d["pad"]
    # GPU op, positional call exactly as utils_functional.py:497 makes it
    y = sc_cuda.conv2d_add_partial_variable_acc(x.cuda(), w.cuda(), d["L"], (pad, pad), (1, 1), 7, 8, 1, False, 2)
    assert y.is_cuda and y.dtype == torch.int32
    assert np.array_equal(y.cpu().numpy(), d["y"])
    # caller-side padding as the reference does it (utils_functional.py:496)
    xp = torch.nn.functional.pad(x, (pad, pad, pad, pad)).cuda()
    y2 = sc_cuda.conv2d_add_partial_variable_acc(xp, w.cuda(), d["L"], (0, 0), (1, 1), 7, 8, 1, False, 2)
    assert np.array_equal(y2.cpu().numpy(), d["y"])
    # non-contiguous input is made contiguous rather than mis-indexed
    xt = x.cuda().transpose(2, 3).contiguous().transpose(2, 3)
    y3 = sc_cuda.conv2d_add_partial_variable_acc(xt, w.cuda(), d["L"], (pad, pad), (1, 1), 7, 8, 1, False, 2)
    assert np.array_equal(y3.cpu().numpy(), d["y"])
    # progressive loading through the module
    y4 = sc_cuda.conv2d_add_partial_variable_acc(x.cuda(), w.cuda(), d["L"], (pad, pad), (1, 1), 7, 2, 2, False, 2)
    exp4 = so.conv2d_add_partial(d["x"], d["w"], d["L"], (pad, pad), 7, 2, 2, 2)
    assert np.array_equal(y4.cpu().numpy(), exp4)
    # host-tensor entry point (utils_functional.py:493): same kernels, result back on the host
    y5 = sc_cpu_name.conv2d_add_partial_new(x, w, d["L"], (pad, pad), (1, 1))
    assert not y5.is_cuda and np.array_equal(y5.numpy(), d["y"])
    # errors are raised, not undefined behaviour
    with pytest.raises(RuntimeError):
        sc_cuda.conv2d_add_partial_variable_acc(x.cuda(), w.cuda(), 100, (pad, pad), (1, 1), 7, 8, 1, False, 2)
    with pytest.raises(RuntimeError):
        sc_cuda.conv2d_or_acc(x.cuda(), w.cuda(), 100, (pad, pad), (1, 1), False)


def test_runs_on_the_current_stream_and_single_hip_runtime(capi, fixtures_small):
    d = fixtures_small["T3"]
    x, w = torch.from_numpy(d["x"]).cuda(), torch.from_numpy(d["w"]).cuda()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        y = capi.conv2d_add_partial_forward(x, w, d["L"], (d["pad"], d["pad"]))
    s.synchronize()
    assert np.array_equal(y.cpu().numpy(), d["y"])
    with open("/proc/self/maps") as f:
        hips = {line.split()[-1] for line in f if "libamdhip64" in line}
    assert len(hips) == 1, hips


# ------------------------------------------------------------------ classifier-type layers
THIN_CASES = [
    # few output positions, OR groups of at least 64 members: the member-parallel kernel
    ((6, 64, 4, 4), (10, 64, 4, 4), (0, 0)),       # the 4-layer CNN's classifier
    ((5, 40, 3, 3), (19, 40, 3, 3), (0, 0)),       # 120 members: ragged over the 64 lanes; two c_out tiles
    ((3, 128, 1, 1), (33, 128, 1, 1), (0, 0)),     # 1x1 classifier, three c_out tiles
    ((2, 70, 4, 5), (5, 70, 3, 3), (1, 1)),        # several output positions per item, padding
    ((2, 24, 5, 4), (7, 24, 2, 3), (1, 0)),        # even kernel extent
]


@pytest.mark.parametrize("case", range(len(THIN_CASES)))
@pytest.mark.parametrize("L", [8, 64, 256])
def test_classifier_layers_match_oracle(capi, so, case, L):
    sx, sw, pad = THIN_CASES[case]
    x, w = wl.make_inputs(sx, sw, "kaiming", seed=700 + case)
    w = (w * 3).contiguous()
    print(f"classifier case {sx} {sw} pad {pad} L {L}", flush=True)
    exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, 7, 2, 2, 2)
    assert L < 64 or np.abs(exp).sum() > 0   # short streams of small weights round to nothing
    assert np.array_equal(gpu_forward(capi, x, w, L, pad, total_width=7, load_width=2, load_wait_w=2, load_wait_a=2),
                          exp)
    for mode, zu in (("yz", 32), ("full", 1)):
        e2 = so.conv2d_general(x.numpy(), w.numpy(), L, pad, mode, zu)
        assert np.array_equal(gpu_forward(capi, x, w, L, pad, accumulate=mode, z_unit=zu), e2), mode
    # 7-bit integer activations take the same path
    k = (x * 128).round().clamp(0, 127).to(torch.uint8)
    a = capi.conv2d_add_partial_forward_q7(k.cuda(), w.cuda(), L, pad)
    assert np.array_equal(a.cpu().numpy(), so.conv2d_add_partial((k.float() / 128).numpy(), w.numpy(), L, pad))


@pytest.mark.parametrize("sx,sw,pad", [((4, 8, 1, 40), (21, 8, 1, 40), (0, 0)),     # linear mapping, 40 kernel rows
                                       ((2, 3, 4, 24), (5, 3, 2, 17), (1, 0)),      # ragged last chunk of 16 rows
                                       ((3, 2, 3, 16), (33, 2, 3, 16), (0, 0))])    # exactly one chunk, three c_out tiles
@pytest.mark.parametrize("L", [16, 128])
def test_long_kernels_use_the_row_chunked_weight_generator(capi, so, sx, sw, pad, L):
    x, w = wl.make_inputs(sx, sw, "prescribed", seed=900)
    w.view(-1)[::5] = 0.0
    d = capi.make_desc(sx, sw, L, pad, 7, 2, 2, 2)
    got = u32(capi.weight_streams(w.cuda(), d))                       # [P][H][K][cot][2][16]
    wpos, wneg = so.weight_streams(w.numpy(), L, 7, 2, 2)             # [P][H][Cin][W][Cout]
    P, H, Cin, W, Cout = wpos.shape
    ncot = (Cout + 15) // 16
    padc = ncot * 16 - Cout
    exp = np.zeros((P, H, Cin * W, ncot, 2, 16), dtype=np.uint32)
    exp[..., 0, :] = np.pad(wpos.reshape(P, H, Cin * W, Cout), ((0, 0),) * 3 + ((0, padc),)).reshape(P, H, Cin * W, ncot, 16)
    exp[..., 1, :] = np.pad(wneg.reshape(P, H, Cin * W, Cout), ((0, 0),) * 3 + ((0, padc),)).reshape(P, H, Cin * W, ncot, 16)
    assert np.array_equal(got, exp)
    assert np.array_equal(gpu_forward(capi, x, w, L, pad, total_width=7, load_width=2, load_wait_w=2, load_wait_a=2),
                          so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, 7, 2, 2, 2))


# ------------------------------------------------------------------ rail-skipping kernel
@pytest.mark.parametrize("shape_x,shape_w,pad,L,loading,gen", [
    ((128, 3, 33, 32), (50, 3, 3, 3), (1, 1), 32, (7, 8, 1, 1), "lfsr"),    # odd row count, partial c_out tile
    ((128, 3, 32, 32), (50, 3, 3, 3), (1, 1), 64, (7, 2, 2, 2), "lfsr"),    # progressive loading
    ((136, 2, 32, 31), (64, 2, 5, 5), (2, 2), 16, (7, 8, 1, 1), "lfsr"),    # 5-wide kernel, partly empty last wave
    ((128, 5, 32, 32), (49, 5, 1, 1), (0, 0), 128, (7, 8, 1, 1), "lfsr"),   # 1 x 1
    ((128, 4, 32, 32), (65, 4, 3, 2), (1, 0), 8, (7, 8, 1, 1), "lfsr"),     # L = 8, even kernel extent in dim 3
    ((128, 3, 32, 32), (50, 3, 3, 3), (1, 1), 64, (7, 8, 1, 1), "acc"),     # random generators: same kernel
    # 3-wide kernels with c_in % 8 == 0 and 4 or 8 c_out tiles: activation words staged through LDS
    ((128, 8, 33, 32), (50, 8, 3, 3), (1, 1), 32, (7, 8, 1, 1), "lfsr"),    # four c_out tiles (one position tile per workgroup), odd row count, partial c_out tile
    ((73, 16, 30, 31), (113, 16, 3, 3), (1, 1), 64, (7, 2, 2, 2), "lfsr"),  # eight c_out tiles, two packs, 531 position tiles (not a multiple of the four per workgroup), the last one ragged
    ((128, 8, 32, 32), (128, 8, 3, 2), (1, 0), 128, (7, 8, 1, 1), "lfsr"),  # two kernel rows, four packs
    ((144, 24, 32, 32), (64, 24, 3, 1), (0, 0), 16, (7, 8, 1, 1), "acc"),   # three chunks of channels per pass
])
def test_large_y_mode_launches_skip_the_zero_rail(capi, so, shape_x, shape_w, pad, L, loading, gen):
    """Launches of at least 4096 waves in y mode run the kernel that processes only the non-zero rail of
    every weight (register-indexed accumulators): bit-exact against the oracle, through the whole-op
    entry point, the uint8 entry point and the stage entry points."""
    x, w = wl.make_inputs(shape_x, shape_w, "q7", seed=shape_w[0])
    w = (w * 3).clamp(-1, 1).contiguous()
    w.view(-1)[::5] = 0.0                                  # zero weights: neither rail
    tw, lw, ww, wa = loading
    d = capi.make_desc(x.shape, w.shape, L, pad, tw, lw, ww, wa, generator=gen, seed=11)
    n_words = ctypes.c_size_t(0)
    from geo_amd import _native
    assert _native.lib().geo_sc_weight_stream_words(ctypes.byref(d), ctypes.byref(n_words)) == 0
    P, (Cout, Cin, W, H) = (L + 31) // 32, w.shape
    assert n_words.value > P * H * Cin * W * ((Cout + 15) // 16) * 32   # the buffer carries the rail-packed copy
    if gen == "lfsr":
        exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, tw, lw, ww, wa)
    else:
        exp = so.conv2d_general(x.numpy(), w.numpy(), L, pad, "y", 1, gen, 11)
    y = capi.conv2d_add_partial_forward(x.cuda(), w.cuda(), L, pad, tw, lw, ww, wa, generator=gen, seed=11)
    assert np.array_equal(y.cpu().numpy(), exp)
    y2 = capi.conv2d_add_partial_from_streams(capi.act_streams(x.cuda(), d), capi.weight_streams(w.cuda(), d), d)
    assert torch.equal(y2, y)
    if gen == "lfsr":
        xq = (x * 128).round().to(torch.uint8).cuda()
        y3 = capi.conv2d_add_partial_forward_q7(xq, w.cuda(), L, pad, tw, lw, ww, wa)
        assert torch.equal(y3, y)
    # a buffer without the rail-packed copy is refused by the Python binding
    with pytest.raises(ValueError):
        short = torch.zeros(P * H * Cin * W * ((Cout + 15) // 16) * 32, dtype=torch.int32, device="cuda")
        capi.conv2d_add_partial_from_streams(capi.act_streams(x.cuda(), d), short, d)


# ------------------------------------------------------------------ launches split over (pack, kernel row) pairs
@pytest.mark.parametrize("shape_x,shape_w,pad,L,loading", [
    ((256, 32, 8, 8), (64, 32, 5, 5), (2, 2), 64, (7, 2, 2, 2)),     # 5120 waves, one pair each: the pairs of a tile in one workgroup
    ((250, 32, 8, 8), (60, 32, 5, 5), (2, 2), 64, (7, 8, 1, 1)),     # the same with a ragged last tile and a partial c_out tile
    ((256, 32, 16, 16), (32, 32, 5, 5), (2, 2), 64, (7, 2, 2, 2)),   # 10240 waves: two rounds, one pair per wave with atomics
    ((200, 16, 8, 9), (48, 16, 3, 3), (1, 1), 256, (7, 8, 1, 1)),    # 24 pairs: more than a workgroup takes
    ((64, 32, 8, 8), (64, 32, 5, 5), (2, 2), 64, (7, 8, 1, 1)),      # 1280 waves: under a round, several pairs per wave
])
def test_split_launches_match_oracle(capi, so, shape_x, shape_w, pad, L, loading):
    """Small layers whose (pack, kernel row) passes are split over waves (the 4-layer CNN's second and third
    layer at batch 256): every form of the split launch against the oracle, bit for bit, twice in a row (the
    second call finds the first one's counts in y)."""
    x, w = wl.make_inputs(shape_x, shape_w, "q7", seed=shape_w[0] + L)
    w.view(-1)[::7] = 0.0
    tw, lw, ww, wa = loading
    exp = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, tw, lw, ww, wa)
    d = capi.make_desc(x.shape, w.shape, L, pad, tw, lw, ww, wa)
    y = torch.full(capi.output_shape(d), 12345, dtype=torch.int32, device="cuda")
    act, wgt = capi.act_streams(x.cuda(), d), capi.weight_streams(w.cuda(), d)
    for _ in range(2):
        capi.conv2d_add_partial_from_streams(act, wgt, d, out=y)
        assert np.array_equal(y.cpu().numpy(), exp)
    assert np.array_equal(capi.conv2d_add_partial_forward(x.cuda(), w.cuda(), L, pad, tw, lw, ww, wa).cpu().numpy(), exp)


# ------------------------------------------------------------------ batches cut into chunks
@pytest.mark.parametrize("shape_x,shape_w,pad,L,kw", [
    ((11, 6, 9, 8), (20, 6, 3, 3), (1, 1), 64, {}),                                   # position-major, 3-wide
    ((11, 6, 9, 8), (20, 6, 3, 3), (1, 1), 128, dict(total_width=7, load_width=2, load_wait_w=2, load_wait_a=2)),
    ((13, 16, 1, 24), (40, 16, 1, 24), (0, 0), 32, {}),                               # SC-linear mapping: item-innermost chunks,
                                                                                      # a last chunk of one item is position-major
    ((10, 64, 4, 4), (10, 64, 4, 4), (0, 0), 64, {}),                                 # classifier layer (lanes over OR members)
    ((9, 5, 8, 8), (7, 5, 3, 3), (1, 1), 32, dict(accumulate="z")),
    ((9, 8, 8, 8), (7, 8, 3, 3), (1, 1), 32, dict(accumulate="yz", z_unit=3)),
    ((9, 4, 8, 8), (18, 4, 3, 3), (1, 1), 64, dict(generator="acc", seed=5)),         # random sequences are numbered by the
    ((9, 4, 8, 8), (18, 4, 3, 3), (1, 1), 64, dict(generator="rand", seed=6, accumulate="full")),  # item's index in the batch
])
def test_forward_in_chunks_of_the_batch(capi, so, shape_x, shape_w, pad, L, kw):
    """geo_sc_options.forward_stream_bytes below the batch's activation streams: the forward generates and
    consumes the streams of a few items at a time (2 - 13 chunks here, the last one often shorter).  Same counts as the
    oracle and as the uncut call, bit for bit, whatever the cut."""
    x, w = wl.make_inputs(shape_x, shape_w, "q7", seed=shape_x[0] + L)
    w = (w * 3).clamp(-1, 1).contiguous()
    xd, wd = x.cuda(), w.cuda()
    d = capi.make_desc(x.shape, w.shape, L, pad, **kw)
    whole = capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d)
    assert capi.forward_chunk(d) == shape_x[0]
    if kw.get("generator", "lfsr") == "lfsr":
        mode = kw.get("accumulate", "y")
        loading = {k: v for k, v in kw.items() if k.startswith(("total", "load"))}
        exp = so.conv2d_modes(x.numpy(), w.numpy(), L, pad, mode, kw.get("z_unit", 1), **loading)
    else:
        exp = so.conv2d_general(x.numpy(), w.numpy(), L, pad, kw.get("accumulate", "y"), 1, kw["generator"], kw["seed"])
    assert np.array_equal(whole.cpu().numpy(), exp)
    item = 4 * ((L + 31) // 32) * shape_x[1] * (shape_x[2] + 2 * pad[1]) * (shape_x[3] + 2 * pad[0])
    seen = set()
    # (a cut batch uses the budget as two buffers, chunks alternating between them and, unless asked otherwise,
    # between the caller's stream and a second stream of the library)
    for items, single in ((2, False), (4, False), (4, True), (8, False), (12, True), (12, False)):
        opt = capi.make_options(forward_stream_bytes=items * item + 5, forward_single_stream=single)
        nc = capi.forward_chunk(d, opt)
        if items >= shape_x[0]:
            assert nc == shape_x[0]      # inside the budget: not cut
        else:
            assert (items // 2 + 1) // 2 <= nc <= items // 2
        seen.add(nc)
        if items < shape_x[0]:
            assert capi.workspace_size(d, opt) < capi.workspace_size(d)
        out = torch.full(capi.output_shape(d), -3, dtype=torch.int32, device="cuda")
        capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d, out=out, options=opt)
        assert torch.equal(out, whole), (items, nc, single)
    assert len(seen) >= 3
    # a workspace sized for chunks is refused by the call that would hold the whole batch
    small = torch.empty(capi.workspace_size(d, capi.make_options(forward_stream_bytes=item)), dtype=torch.uint8,
                        device="cuda")
    with pytest.raises(capi.GeoScError) as e:
        capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d, workspace=small)
    assert e.value.status == 3


def test_forward_uncut_at_the_resnet_shape(capi, checksums):
    """The default budget cuts the batch of the 64->64 3x3 layer at 56x56 (0.88 GB of streams) into chunks -
    test_forward_full_size_checksums runs that way; here the whole batch in one launch, same checksum, and the
    7-bit integer entry point through its chunks."""
    c = checksums["C5_kaiming_L256"]
    x, w, pad, _ = wl.named(c["shape_name"], c["mode"])
    xd, wd = x.cuda(), w.cuda()
    d = capi.make_desc(xd.shape, wd.shape, c["L"], (pad, pad))
    assert capi.forward_chunk(d) < 128 and capi.workspace_size(d) <= 300 << 20
    whole = capi.make_options(forward_stream_bytes=1 << 40)
    assert capi.forward_chunk(d, whole) == 128
    y = capi.conv2d_add_partial_forward(xd, wd, c["L"], (pad, pad), desc=d, options=whole).cpu().numpy()
    assert hashlib.sha256(np.ascontiguousarray(y).tobytes()).hexdigest() == c["sha256"]
    xq7, wq7, _, _ = wl.named("C5", "q7")
    k = (xq7 * 128).round().to(torch.uint8).cuda()
    a = capi.conv2d_add_partial_forward_q7(k, wq7.cuda(), 256, (pad, pad))
    b = capi.conv2d_add_partial_forward(xq7.cuda(), wq7.cuda(), 256, (pad, pad), options=whole)
    assert torch.equal(a, b) and int(a.abs().max()) > 0


def test_chunked_forward_in_a_hip_graph(capi):
    """A cut batch alternates between the caller's stream and a second stream of the library (forked and joined
    with events): captured after geo_sc_init, the whole fork-join becomes part of the graph.  Replayed three
    times, with eager calls (which overwrite the workspace) and synchronisations between the replays, every
    replay against the eager result."""
    L, pad = 64, (1, 1)
    x, w = wl.make_inputs((12, 6, 9, 8), (20, 6, 3, 3), "q7", seed=21)
    xd, wd = x.cuda(), w.cuda()
    d = capi.make_desc(x.shape, w.shape, L, pad)
    item = 4 * 2 * 6 * 11 * 10
    opt = capi.make_options(forward_stream_bytes=6 * item)       # chunks of three items: four chunks, two per stream
    assert capi.forward_chunk(d, opt) == 3
    ws = torch.empty(capi.workspace_size(d, opt), dtype=torch.uint8, device="cuda")
    ref = capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d)
    capi.init()
    out = torch.zeros_like(ref)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d, out=out, workspace=ws, options=opt)   # warm-up
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d, out=out, workspace=ws, options=opt)
    x2 = torch.rand_like(xd)
    for i in range(3):
        out.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref), i
        # eager work on the same workspace between the replays
        other = capi.conv2d_add_partial_forward(x2, wd, L, pad, desc=d, workspace=ws, options=opt)
        torch.cuda.synchronize()
        assert not torch.equal(other, ref)
