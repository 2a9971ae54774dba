"""Pins the CPU oracle (oracle/sc_oracle.c) before anything is compared against it:
golden outputs of the reference's compiled CPU kernel, closed forms, invariants and an
independent per-bit formulation."""
import hashlib

import numpy as np
import pytest

from geo_amd import workloads as wl
from oracle import sc_oracle as so
from tests import bitref

LENGTHS = (8, 16, 32, 64, 128, 256)


# ----------------------------------------------------------------------------- LFSR
@pytest.mark.parametrize("n,first", [
    (5, [2, 4, 9, 18, 5, 11, 22, 12]),
    (6, [2, 4, 8, 16, 33, 3, 6, 12]),
    (7, [2, 4, 8, 16, 32, 65, 3, 6]),
    (8, [2, 4, 8, 17, 35, 71, 142, 28]),
])
def test_lfsr_known_first_states(n, first):
    s, got = 1, []
    for _ in first:
        s = so.lfsr_step(n, s)
        got.append(s)
    assert got == first


@pytest.mark.parametrize("n", [3, 4, 5, 6, 7, 8])
def test_lfsr_is_maximal_and_matches_bit_formulation(n):
    seen, s = [], 1
    for _ in range((1 << n) - 1):
        assert so.lfsr_step(n, s) == bitref.step(n, s)
        s = so.lfsr_step(n, s)
        seen.append(s)
    assert s == 1                                  # period 2^n - 1
    assert sorted(seen) == list(range(1, 1 << n))  # every non-zero state once
    assert so.lfsr_step(n, 0) == 0                 # zero is the lock-up state


def test_length_to_width():
    assert [so.nbits_for_length(L) for L in LENGTHS] == [3, 4, 5, 6, 7, 8]
    assert so.nbits_for_length(100) == -1


# ----------------------------------------------------------------------------- codes
@pytest.mark.parametrize("L", LENGTHS)
def test_codes_closed_form(L):
    assert so.code_act(0.0, L) == 0
    assert so.code_act(-0.3, L) == 0
    assert so.code_act(1.0, L) == L - 1            # clamp to L-1
    assert so.code_act(7.5, L) == L - 1
    assert so.code_act(1.0 / L, L) == 1
    assert so.code_act(1.0 / L + 1e-4, L) == 2     # ceil
    assert so.code_act(0.5, L) == L // 2
    assert so.code_wpos(-0.4, L) == 0 and so.code_wneg(0.4, L) == 0
    assert so.code_wneg(-1.0, L) == L - 1 and so.code_wneg(-0.5, L) == L // 2
    assert so.code_wneg(-(1.0 / L + 1e-4), L) == 2  # ceil of the negated clamp
    rng = np.random.default_rng(0)
    for v in rng.uniform(-1.2, 1.2, 200).astype(np.float32):
        xa, wp, wn = bitref.codes(np.array([v]), np.array([v]), L)
        assert so.code_act(float(v), L) == xa[0]
        assert so.code_wpos(float(v), L) == wp[0]
        assert so.code_wneg(float(v), L) == wn[0]
        assert wp[0] == 0 or wn[0] == 0


# ----------------------------------------------------------------------------- streams
@pytest.mark.parametrize("L", LENGTHS)
def test_stream_popcount_invariant(L):
    """L steps = one full period (each state 1..L-1 once) plus the first state again, so
    popcount = #(states < code) + [code > first state] = max(code-1,0) + [code > step(seed)]."""
    n = so.nbits_for_length(L)
    for seed in (1, 2, L // 2, L - 1):
        for code in range(L):
            words, final = so.stream_of(code, seed, L)
            pop = sum(bin(int(x)).count("1") for x in words)
            assert pop == max(code - 1, 0) + (1 if code > so.lfsr_step(n, seed) else 0)
            assert final == so.lfsr_step(n, seed)   # period L-1, L steps
            if L < 32:
                assert int(words[0]) < (1 << L)


@pytest.mark.parametrize("L", LENGTHS)
def test_stream_bits_msb_first_and_match_bit_formulation(L):
    for code, seed in ((0, 1), (1, 1), (L // 3, 5), (L - 1, L - 1), (L // 2, 7 % (L - 1) + 1)):
        words, _ = so.stream_of(code, seed, L)
        bits = bitref.bits_of(code, seed, L)
        unit = min(L, 32)
        got = []
        for p in range(len(words)):
            for b in range(unit):
                got.append((int(words[p]) >> (unit - 1 - b)) & 1)
        assert got == list(bits)


def test_progressive_loading_widths_and_neutrality():
    L = 128
    # neutral when load_width >= total_width + 1, whatever the wait
    for code in (3, 77, 127):
        a, _ = so.stream_of(code, 9, L, 7, 8, 1)
        b, _ = so.stream_of(code, 9, L, 7, 8, 5)
        c, _ = so.stream_of(code, 9, L, 7, 100, 3)
        assert np.array_equal(a, b) and np.array_equal(a, c)
    # (total 7, unit 2, wait 2): widths 1,3,3,5,5,7,7,...
    widths = [min(7, (b // 2 + 1) * 2 - 1) for b in range(1, 9)]
    assert widths == [1, 3, 3, 5, 5, 7, 7, 7]
    for code, seed in ((0b1011011, 3), (0b0101010, 100), (127, 64)):
        words, _ = so.stream_of(code, seed, L, 7, 2, 2)
        assert list(_unpack(words, L)) == list(bitref.bits_of(code, seed, L, 7, 2, 2))
        # from cycle 6 on the stream equals the unmasked one
        full, _ = so.stream_of(code, seed, L, 7, 8, 1)
        assert list(_unpack(words, L))[5:] == list(_unpack(full, L))[5:]
    # hand-computed: code 0b1000000 survives width 1 (mask keeps the top bit only)
    n = 7
    s1 = so.lfsr_step(n, 3)
    words, _ = so.stream_of(0b1111111, 3, L, 7, 2, 2)
    assert _unpack(words, L)[0] == (1 if 0b1000000 > s1 else 0)


def test_progressive_loading_literal_known_answers():
    """Hand-derived bits (tests/loading_vectors.py, worked out from sc_cuda_kernel.cu:155-160 cycle by cycle)
    applied to the oracle's generator: fixes that the first cycle has cur_bit == 1, that the division
    by load_wait is an integer division, and that the register advances before the comparison."""
    from tests import loading_vectors as lv

    s, states = 1, {}
    for cycle in range(1, 83):
        s = so.lfsr_step(7, s)
        states[cycle] = s
    assert {c: states[c] for c in lv.STATES_FROM_SEED_1} == lv.STATES_FROM_SEED_1
    for (tw, lw, wait), first, table in lv.VECTORS:
        for code, bits in table.items():
            words, _ = so.stream_of(code, 1, 128, tw, lw, wait)
            got = _unpack(words, 128)[first - 1:first - 1 + len(bits)]
            assert got == bits, ((tw, lw, wait), first, code)


def _unpack(words, L):
    unit = min(L, 32)
    return [(int(words[p]) >> (unit - 1 - b)) & 1 for p in range(len(words)) for b in range(unit)]


def test_weight_and_activation_stream_layouts():
    L = 64
    x, w, pad, _ = wl.named("T3")
    wpos, wneg = so.weight_streams(w.numpy(), L)
    Cout, Cin, W, H = w.shape
    assert wpos.shape == (2, H, Cin, W, Cout)
    for (co, ci, u, v) in ((0, 0, 0, 0), (4, 3, 2, 4), (2, 1, 1, 3)):
        f = ci * W + u
        words, _ = so.stream_of(so.code_wpos(float(w[co, ci, u, v]), L), (67 + f) % (L - 1) + 1, L)
        assert np.array_equal(wpos[:, v, ci, u, co], words)
        words, _ = so.stream_of(so.code_wneg(float(w[co, ci, u, v]), L), (37 + f) % (L - 1) + 1, L)
        assert np.array_equal(wneg[:, v, ci, u, co], words)
    item = x[0].numpy()
    A = so.act_streams(item, L)
    Cin, Wi, Hi = item.shape
    for (ci, p, q) in ((0, 0, 0), (3, 7, 10), (2, 5, 1)):
        i = (ci * Wi + p) * Hi + q
        words, _ = so.stream_of(so.code_act(float(item[ci, p, q]), L), i % (L - 1) + 1, L)
        assert np.array_equal(A[:, ci, p, q], words)
    assert not so.act_streams(np.zeros_like(item), L).any()


# ----------------------------------------------------------------------------- whole op
def test_against_reference_fixtures(fixtures_small):
    assert len(fixtures_small) >= 17
    for name, d in fixtures_small.items():
        for fast in (True, False):
            y = so.conv2d_add_partial(d["x"], d["w"], d["L"], (d["pad"], d["pad"]), fast=fast)
            assert np.array_equal(y, d["y"]), (name, fast)


@pytest.mark.parametrize("name", ["C1_prescribed_L64", "C3_sparse_L32", "C3_kaiming_L128"])
def test_against_reference_checksums(checksums, name):
    c = checksums[name]
    x, w, pad, _ = wl.named(c["shape_name"], c["mode"])
    y = so.conv2d_add_partial(x.numpy(), w.numpy(), c["L"], (pad, pad))
    assert int(y.astype(np.int64).sum()) == c["sum"]
    assert hashlib.sha256(y.tobytes()).hexdigest() == c["sha256"]


@pytest.mark.parametrize("shape_x,shape_w,pad,L", [
    ((2, 2, 4, 5), (3, 2, 3, 2), (1, 0), 8),
    ((1, 3, 4, 4), (2, 3, 2, 3), (0, 1), 16),
    ((2, 2, 3, 3), (2, 2, 3, 3), (1, 1), 32),
    ((1, 2, 4, 3), (3, 2, 1, 1), (0, 0), 64),
])
def test_against_independent_per_bit_formulation(shape_x, shape_w, pad, L):
    x, w = wl.make_inputs(shape_x, shape_w, "prescribed", seed=21)
    yb = bitref.conv_bits(x.numpy(), w.numpy(), L, pad)
    for fast in (True, False):
        y = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, fast=fast)
        assert np.array_equal(y.astype(np.int64), yb)
    # progressive loading, spec text only: both restatements agree on it as well
    yb = bitref.conv_bits(x.numpy(), w.numpy(), L, pad, 7, 2, 2, 3)
    y = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, 7, 2, 2, 3)
    assert np.array_equal(y.astype(np.int64), yb)


def test_asymmetric_padding_convention_matches_compiled_reference():
    ref = so.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built here")
    import torch
    x, w = wl.make_inputs((2, 3, 6, 5), (4, 3, 3, 2), "prescribed", seed=4)
    for pad in ((2, 0), (0, 1), (1, 2)):
        yr = ref.conv2d_add_partial_new(x, w, 32, pad, (1, 1)).numpy()
        y = so.conv2d_add_partial(x.numpy(), w.numpy(), 32, pad)
        assert y.shape == yr.shape and np.array_equal(y, yr)
    assert torch.is_tensor(x)


def test_compiled_reference_variants_agree_with_oracle():
    variants = so.ref_variants_usable()
    if not variants:
        pytest.skip("oracle/_ref not built here")
    x, w = wl.make_inputs((3, 5, 9, 11), (7, 5, 3, 3), "kaiming", seed=8)
    y = so.conv2d_add_partial(x.numpy(), w.numpy(), 128, (1, 1))
    for v in variants:
        yr = so.load_ref(v).conv2d_add_partial_new(x, w, 128, (1, 1), (1, 1)).numpy()
        assert np.array_equal(y, yr), v


def test_special_cases_and_invariants():
    L = 64
    # Cin = W = 1: no OR at all -> y = sum_v popc(a & wp) - popc(a & wn)
    x, w = wl.make_inputs((1, 1, 1, 6), (2, 1, 1, 3), "prescribed", seed=2)
    y = so.conv2d_add_partial(x.numpy(), w.numpy(), L)
    A = so.act_streams(x[0].numpy(), L)
    wp, wn = so.weight_streams(w.numpy(), L)
    for co in range(2):
        for b in range(4):
            e = 0
            for v in range(3):
                for p in range(2):
                    e += bin(int(A[p, 0, 0, b + v] & wp[p, v, 0, 0, co])).count("1")
                    e -= bin(int(A[p, 0, 0, b + v] & wn[p, v, 0, 0, co])).count("1")
            assert y[0, co, 0, b] == e
    # |y| <= H * L, and batch items are independent with identical seeds
    x, w = wl.make_inputs((3, 4, 6, 6), (5, 4, 3, 3), "prescribed", seed=9)
    y = so.conv2d_add_partial(x.numpy(), w.numpy(), L, (1, 1))
    assert np.abs(y).max() <= 3 * L
    perm = [2, 0, 1]
    yp = so.conv2d_add_partial(x.numpy()[perm], w.numpy(), L, (1, 1))
    assert np.array_equal(yp, y[perm])
    # output-channel permutation equivariance (weight sequences do not depend on c_out)
    yc = so.conv2d_add_partial(x.numpy(), w.numpy()[[4, 3, 2, 1, 0]], L, (1, 1))
    assert np.array_equal(yc, y[:, [4, 3, 2, 1, 0]])
    # all-zero activations or weights give zero
    assert not so.conv2d_add_partial(np.zeros_like(x.numpy()), w.numpy(), L, (1, 1)).any()
    assert not so.conv2d_add_partial(x.numpy(), np.zeros_like(w.numpy()), L, (1, 1)).any()
    # full-scale positive inputs: only the positive rail fires
    xs = np.ones((1, 8, 3, 3), dtype=np.float32)
    ws = np.ones((1, 8, 3, 3), dtype=np.float32)
    ys = so.conv2d_add_partial(xs, ws, L)
    assert ys.shape == (1, 1, 1, 1) and 0 < ys[0, 0, 0, 0] <= 3 * L


def test_bad_arguments():
    x, w = wl.make_inputs((1, 1, 3, 3), (1, 1, 3, 3))
    with pytest.raises(ValueError):
        so.conv2d_add_partial(x.numpy(), w.numpy(), 100)
    with pytest.raises(ValueError):
        so.conv2d_add_partial(x.numpy(), w.numpy()[:, :, :, :], 64, load_wait_w=0)
    with pytest.raises(ValueError):
        so.conv2d_add_partial(x.numpy()[:, :, :2], w.numpy(), 64)


# ------------------------------------------------------------------ z / yz accumulation modes
# No executable reference exists for these (GPU-only ops of the reference); they are pinned by
# reductions to the y-mode path, which the compiled reference pins bit for bit.
def test_modes_y_is_the_pinned_path():
    x, w = wl.make_inputs((2, 5, 6, 7), (4, 5, 3, 2), "prescribed", seed=31)
    for L in (8, 64, 256):
        y = so.conv2d_add_partial(x.numpy(), w.numpy(), L, (1, 2), 7, 2, 2, 3)
        assert np.array_equal(so.conv2d_modes(x.numpy(), w.numpy(), L, (1, 2), "y", 1, 7, 2, 2, 3), y)
        # a single channel group is y-mode exactly (same groups, same seeds)
        for zu in (5, 9):
            assert np.array_equal(so.conv2d_modes(x.numpy(), w.numpy(), L, (1, 2), "yz", zu, 7, 2, 2, 3), y)


@pytest.mark.parametrize("zu", [1, 2, 3, 4])
@pytest.mark.parametrize("L", [16, 128])
def test_yz_decomposes_into_y_mode_over_channel_blocks(zu, L):
    """Seeds restart in every block of z_unit channels (weights: (c % zu)*W + u, activations:
    index inside the block), blocks are added: yz(x, w) == sum over blocks of y(x[block], w[block])."""
    x, w = wl.make_inputs((2, 7, 5, 6), (3, 7, 3, 3), "prescribed", seed=40 + zu)
    x, w = x.numpy(), w.numpy()
    got = so.conv2d_modes(x, w, L, (1, 1), "yz", zu, 7, 3, 2, 5)
    exp = 0
    for c0 in range(0, 7, zu):
        exp = exp + so.conv2d_add_partial(x[:, c0:c0 + zu], w[:, c0:c0 + zu], L, (1, 1), 7, 3, 2, 5)
    assert np.array_equal(got, exp)


def test_z_reduces_to_y_mode_where_the_window_is_one_dimensional():
    L = 32
    # H = 1, Cin = 1: OR over u with seed u, nothing to add
    x, w = wl.make_inputs((2, 1, 6, 5), (3, 1, 3, 1), "prescribed", seed=51)
    assert np.array_equal(so.conv2d_modes(x.numpy(), w.numpy(), L, (0, 1), "z"),
                          so.conv2d_add_partial(x.numpy(), w.numpy(), L, (0, 1)))
    # W = 1 on a signal with a single row: OR over v with seed v; the transposed problem is y-mode
    x, w = wl.make_inputs((2, 1, 1, 9), (3, 1, 1, 4), "prescribed", seed=52)
    yz = so.conv2d_modes(x.numpy(), w.numpy(), L, (0, 0), "z")
    yt = so.conv2d_add_partial(x.numpy().transpose(0, 1, 3, 2).copy(), w.numpy().transpose(0, 1, 3, 2).copy(), L)
    assert np.array_equal(yz, yt.transpose(0, 1, 3, 2))
    # channel planes of 7*k words with L = 8: activation seeds restart per channel, so z-mode is
    # the sum over channels of single-channel z-mode
    x, w = wl.make_inputs((2, 3, 7, 3), (2, 3, 3, 1), "prescribed", seed=53)
    x, w = x.numpy(), w.numpy()
    exp = 0
    for c in range(3):
        exp = exp + so.conv2d_add_partial(x[:, c:c + 1], w[:, c:c + 1], 8)
    assert np.array_equal(so.conv2d_modes(x, w, 8, (0, 0), "z"), exp)


def _z_window_as_y_mode(x1, w1, L, load):
    """Single-channel z-mode (joint OR over a W x H window, weight seed index u*H + v) restated as
    a y-mode problem: kernel column u becomes input channel u, kernel row index v becomes the
    dim-2 tap, one kernel row: x'[u, p', q'] = x[q' + u, p'], w'[co, u, v, 0] = w[co, 0, u, v].
    y-mode then ORs over (c' = u, u' = v) with weight seed index c' * W' + u' = u * H + v - z-mode's.
    The activation seed of x'[u, q, a] is u*Hi*Wo + q*Wo + a, z-mode's is (a + u)*Hi + q: equal
    modulo L - 1 (all that a seed depends on) when Hi = Wo = 1 (mod L - 1).
    Returns out[n, co, a, b]."""
    n, _, wi, hi = x1.shape
    c_out, _, W, H = w1.shape
    wo = wi - W + 1
    assert hi % (L - 1) == 1 and wo % (L - 1) == 1
    xt = np.empty((n, W, hi, wo), dtype=np.float32)
    for u in range(W):
        xt[:, u] = x1[:, 0, u:u + wo, :].transpose(0, 2, 1)
    wt = np.ascontiguousarray(w1[:, 0, :, :, None])          # (c_out, W, H, 1)
    yt = so.conv2d_add_partial(xt, wt, L, (0, 0), *load)       # (n, c_out, Ho, Wo)
    return yt.transpose(0, 1, 3, 2)


@pytest.mark.parametrize("L,W,H,k", [(8, 3, 3, 1), (8, 2, 5, 2), (16, 3, 2, 1), (32, 2, 3, 1), (8, 7, 2, 1)])
def test_z_two_dimensional_windows_reduce_to_y_mode(L, W, H, k):
    """General W x H windows of z-mode against the y-mode path that the compiled reference pins:
    sizes with Hi = Wo = 1 (mod L - 1) make the restated problem's seeds coincide exactly.  With
    W = L - 1 the channel planes hold a multiple of L - 1 words, so several channels decompose too
    (z adds over input channels; weight seeds do not depend on the channel)."""
    hi = wo = 1 + k * (L - 1)
    wi = wo + W - 1
    c_in = 3 if W == L - 1 else 1
    x, w = wl.make_inputs((2, c_in, wi, hi), (3, c_in, W, H), "prescribed", seed=80 + L + W)
    x, w = x.numpy(), (w.numpy() * 0.5).astype(np.float32)
    for load in [(7, 8, 1, 1), (7, 2, 2, 3)]:
        got = so.conv2d_modes(x, w, L, (0, 0), "z", 1, *load)
        exp = 0
        for c in range(c_in):
            exp = exp + _z_window_as_y_mode(x[:, c:c + 1], w[:, c:c + 1], L, load)
        assert got.any()
        assert np.array_equal(got, exp), (L, W, H, load)


@pytest.mark.parametrize("mode,zu", [("z", 1), ("yz", 2), ("yz", 3), ("y", 1)])
def test_modes_against_independent_per_bit_formulation(mode, zu):
    for (sx, sw, pad, L) in [((2, 3, 4, 5), (2, 3, 3, 2), (1, 0), 8), ((1, 5, 4, 4), (3, 5, 2, 3), (0, 1), 32)]:
        x, w = wl.make_inputs(sx, sw, "prescribed", seed=61)
        yb = bitref.conv_bits_modes(x.numpy(), w.numpy(), L, pad, mode, zu, 7, 2, 2, 3)
        y = so.conv2d_modes(x.numpy(), w.numpy(), L, pad, mode, zu, 7, 2, 2, 3)
        assert np.array_equal(y.astype(np.int64), yb), (mode, zu, sx)


def test_modes_bounds():
    x, w = wl.make_inputs((1, 6, 5, 5), (2, 6, 3, 3), "prescribed", seed=70)
    L = 64
    assert np.abs(so.conv2d_modes(x.numpy(), w.numpy(), L, (1, 1), "z")).max() <= 6 * L
    assert np.abs(so.conv2d_modes(x.numpy(), w.numpy(), L, (1, 1), "yz", 4)).max() <= 2 * 3 * L
    with pytest.raises(ValueError):
        so.conv2d_modes(x.numpy(), w.numpy(), L, (1, 1), "yz", 0)
