"""Pins the random stream generators of the oracle ("acc": exactly `code` ones, "rand": Bernoulli
bits): Philox4x32-10 known answers, the exact-count invariant, bit frequencies, and the closed-form
expectation of the layer output.  The reference's own bit sequences (cuRAND XORWOW per thread) are
not reproducible; these are the distributional facts its generators have."""
import numpy as np
import pytest

from geo_amd import workloads as wl
from oracle import sc_oracle as so

LENGTHS = (8, 16, 32, 64, 128, 256)


def unpack(words, L):
    unit = min(L, 32)
    return np.array([(int(w) >> (unit - 1 - b)) & 1 for w in words for b in range(unit)], dtype=np.int64)


def test_philox_known_answers():
    # Random123 known-answer vectors of philox4x32-10
    assert [hex(v) for v in so.philox4x32_10([0] * 4, [0] * 2)] == ["0x6627e8d5", "0xe169c58d", "0xbc57ac4c", "0x9b00dbd8"]
    assert [hex(v) for v in so.philox4x32_10([0xffffffff] * 4, [0xffffffff] * 2)] == [
        "0x408f276d", "0x41c83b0e", "0xa20bc7c6", "0x6d5451fd"]
    assert [hex(v) for v in so.philox4x32_10([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344],
                                             [0xa4093822, 0x299f31d0])] == [
        "0xd16cfe09", "0x94fdcceb", "0x5001e420", "0x24126ea1"]


@pytest.mark.parametrize("L", LENGTHS)
def test_acc_streams_have_exactly_code_ones(L):
    for code in range(L):
        for index in (0, 1, 12345678901):
            bits = unpack(so.random_stream(code, L, "acc", 0, index, 99), L)
            assert len(bits) == L and bits.sum() == code, (L, code, index)


@pytest.mark.parametrize("gen", ["acc", "rand"])
@pytest.mark.parametrize("L,code", [(8, 3), (64, 17), (128, 100), (256, 5)])
def test_bit_frequencies(gen, L, code):
    n = 3000
    acc = np.zeros(L)
    for index in range(n):
        acc += unpack(so.random_stream(code, L, gen, 1, index, 7), L)
    p = code / L
    sigma = np.sqrt(p * (1 - p) / n)
    # every bit position is one with probability code / L (5.5 sigma over <= 256 positions)
    assert np.abs(acc / n - p).max() < 5.5 * sigma
    # overall mean: exact for "acc", binomial for "rand"
    if gen == "acc":
        assert acc.sum() == n * code
    else:
        assert abs(acc.sum() / (n * L) - p) < 5 * sigma / np.sqrt(L)


def test_streams_depend_on_seed_tag_and_index():
    base = so.random_stream(40, 128, "rand", 0, 5, 1)
    assert not np.array_equal(base, so.random_stream(40, 128, "rand", 0, 6, 1))
    assert not np.array_equal(base, so.random_stream(40, 128, "rand", 1, 5, 1))
    assert not np.array_equal(base, so.random_stream(40, 128, "rand", 0, 5, 2))
    assert np.array_equal(base, so.random_stream(40, 128, "rand", 0, 5, 1))
    # pairs of "rand" streams are uncorrelated: P(a & b) = p^2
    n, L = 2000, 128
    both = sum(int((unpack(so.random_stream(64, L, "rand", 0, i, 3), L) &
                    unpack(so.random_stream(64, L, "rand", 1, i, 3), L)).sum()) for i in range(n))
    assert abs(both / (n * L) - 0.25) < 5 * np.sqrt(0.25 * 0.75 / (n * L))


def expected_counts(x, w, L, pad, mode):
    """E[y]: per stream bit, P(OR over the group of a & w) = 1 - prod(1 - pa * pw) for independent
    streams with marginals pa = code_a / L, pw = code_w / L; times L bits; summed over add groups."""
    xp = np.pad(x, ((0, 0), (0, 0), (pad[1], pad[1]), (pad[0], pad[0])))
    N, Cin, Wi, Hi = xp.shape
    Cout, _, W, H = w.shape
    Wo, Ho = Wi - W + 1, Hi - H + 1
    pa = np.ceil(np.clip(xp * np.float32(L), 0, L - 1)) / L
    pw = [np.ceil(np.clip(w * np.float32(L), 0, L - 1)) / L, np.ceil(-np.clip(w * np.float32(L), 1 - L, 0)) / L]
    e = np.zeros((N, Cout, Wo, Ho))
    groups = [range(H)] if mode == "full" else [[v] for v in range(H)]
    for rail, sgn in ((0, 1.0), (1, -1.0)):
        for vs in groups:
            keep = np.ones((N, Cout, Wo, Ho))
            for v in vs:
                for u in range(W):
                    patch = pa[:, :, u:u + Wo, v:v + Ho]                       # n c a b
                    keep *= np.prod(1 - patch[:, None] * pw[rail][None, :, :, u, v, None, None], axis=2)
            e += sgn * L * (1 - keep)
    return e


@pytest.mark.parametrize("gen,mode", [("acc", "y"), ("rand", "full"), ("rand", "y"), ("acc", "full")])
def test_layer_output_has_the_closed_form_expectation(gen, mode):
    L = 64
    x, w = wl.make_inputs((2, 3, 5, 5), (4, 3, 3, 3), "prescribed", seed=3)
    x, w = x.numpy(), (w.numpy() * 0.6).astype(np.float32)
    S = 120
    ys = np.stack([so.conv2d_general(x, w, L, (1, 1), mode, 1, gen, seed) for seed in range(S)]).astype(np.float64)
    e = expected_counts(x, w, L, (1, 1), mode)
    err = ys.mean(0) - e
    sem = ys.std(0, ddof=1) / np.sqrt(S) + 1e-9
    assert np.abs(err / sem).max() < 5.5, np.abs(err / sem).max()
    assert abs(err.mean()) < 0.2
    # different seeds give different outputs, the same seed the same output
    assert not np.array_equal(ys[0], ys[1])
    assert np.array_equal(ys[5], so.conv2d_general(x, w, L, (1, 1), mode, 1, gen, 5))


def test_full_or_with_lfsr_is_a_single_or_group():
    """mode "full" under the LFSR generator: OR over the whole window; with H = 1 it is y-mode."""
    x, w = wl.make_inputs((2, 3, 6, 5), (4, 3, 3, 1), "prescribed", seed=8)
    assert np.array_equal(so.conv2d_general(x.numpy(), w.numpy(), 32, (0, 1), "full"),
                          so.conv2d_add_partial(x.numpy(), w.numpy(), 32, (0, 1)))
    x, w = wl.make_inputs((1, 2, 5, 5), (3, 2, 3, 3), "prescribed", seed=9)
    y = so.conv2d_general(x.numpy(), w.numpy(), 64, (1, 1), "full")
    assert np.abs(y).max() <= 64
