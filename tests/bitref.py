"""An independent, unpacked per-bit formulation of the SC convolution used to pin the
oracle on tiny shapes.

It shares no code with ``oracle/sc_oracle.c``: streams are lists of 0/1 bits produced by a
bit-twiddling LFSR (shift/xor of tap bits, not the reference's ``/`` and ``%`` arithmetic),
and the accumulation is the reference's legacy formulation (utils_functional.py:590-600):
a dense integer convolution of one bit-plane per stream cycle and kernel row, passed
through sign() to model the OR, summed over cycles and rows.
"""
import numpy as np

TAPS = {3: (2, 1), 4: (3, 2), 5: (4, 2), 6: (5, 4), 7: (6, 5), 8: (7, 5, 4, 3)}


def step(n, s):
    fb = 0
    for t in TAPS[n]:
        fb ^= (s >> t) & 1
    return ((s << 1) & ((1 << n) - 1)) | fb


def nbits(L):
    return {8: 3, 16: 4, 32: 5, 64: 6, 128: 7, 256: 8}[L]


def loaded(code, cycle, tw, lw, wait):
    cw = min(tw, (cycle // wait + 1) * lw - 1)
    sh = tw - cw
    return (code >> sh) << sh


def bits_of(code, seed, L, tw=7, lw=8, wait=1):
    n = nbits(L)
    s = seed
    out = np.zeros(L, dtype=np.int64)
    for t in range(L):
        s = step(n, s)
        out[t] = 1 if loaded(code, t + 1, tw, lw, wait) > s else 0
    return out


def codes(x, w, L):
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    Lf = np.float32(L)
    xa = np.ceil(np.clip(x * Lf, 0, L - 1)).astype(np.int64)
    wp = np.ceil(np.clip(w * Lf, 0, L - 1)).astype(np.int64)
    wn = np.ceil(-np.clip(w * Lf, 1 - L, 0)).astype(np.int64)
    return xa, wp, wn


def conv_bits(x, w, L, pad=(0, 0), tw=7, lw=8, wait_w=1, wait_a=1):
    """int64 (N,Cout,Wo,Ho); pad=(p0,p1): p0 pads the last dim, p1 the one before."""
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    x = np.pad(x, ((0, 0), (0, 0), (pad[1], pad[1]), (pad[0], pad[0])))
    N, Cin, Wi, Hi = x.shape
    Cout, _, W, H = w.shape
    Wo, Ho = Wi - W + 1, Hi - H + 1
    xa, wp, wn = codes(x, w, L)
    abits = np.zeros((N, Cin, Wi, Hi, L), dtype=np.int64)
    for c in range(Cin):
        for p in range(Wi):
            for q in range(Hi):
                i = (c * Wi + p) * Hi + q
                seed = i % (L - 1) + 1
                for n in range(N):
                    abits[n, c, p, q] = bits_of(int(xa[n, c, p, q]), seed, L, tw, lw, wait_a)
    wpb = np.zeros((Cout, Cin, W, H, L), dtype=np.int64)
    wnb = np.zeros_like(wpb)
    for c in range(Cin):
        for u in range(W):
            f = c * W + u
            sp = (67 + f) % (L - 1) + 1
            sn = (37 + f) % (L - 1) + 1
            for co in range(Cout):
                for v in range(H):
                    wpb[co, c, u, v] = bits_of(int(wp[co, c, u, v]), sp, L, tw, lw, wait_w)
                    wnb[co, c, u, v] = bits_of(int(wn[co, c, u, v]), sn, L, tw, lw, wait_w)
    y = np.zeros((N, Cout, Wo, Ho), dtype=np.int64)
    for v in range(H):
        # dense integer correlation over (ci, u) for kernel row v, per cycle t
        sp = np.zeros((N, Cout, Wo, Ho, L), dtype=np.int64)
        sn = np.zeros_like(sp)
        for u in range(W):
            a = abits[:, :, u:u + Wo, v:v + Ho, :]  # (N,Cin,Wo,Ho,L)
            sp += np.einsum("ncabt,oct->noabt", a, wpb[:, :, u, v, :])
            sn += np.einsum("ncabt,oct->noabt", a, wnb[:, :, u, v, :])
        y += np.sign(sp).sum(-1) - np.sign(sn).sum(-1)
    return y


def conv_bits_modes(x, w, L, pad=(0, 0), mode="y", z_unit=1, tw=7, lw=8, wait_w=1, wait_a=1):
    """The accumulation modes of the reference's GPU kernels written as one dense tensor of
    product bits T[n,o,a,b,c,u,v,t] that is OR-ed (sign of a sum) over one set of axes and
    added over the rest.  "y": OR (c,u), add v (sc_cuda_kernel.cu:91-170); "z": OR (u,v), add c
    (:270-349); "yz": OR (c within a block of z_unit channels, u), add v and blocks (:176-268).
    Seed numbering per mode as in those kernels and their host code (:1080)."""
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    x = np.pad(x, ((0, 0), (0, 0), (pad[1], pad[1]), (pad[0], pad[0])))
    N, Cin, Wi, Hi = x.shape
    Cout, _, W, H = w.shape
    Wo, Ho = Wi - W + 1, Hi - H + 1
    zu = min(z_unit, Cin)
    xa, wp, wn = codes(x, w, L)
    abits = np.zeros((N, Cin, Wi, Hi, L), dtype=np.int64)
    for c in range(Cin):
        for p in range(Wi):
            for q in range(Hi):
                i = (c * Wi + p) * Hi + q
                if mode == "yz":
                    i %= zu * Wi * Hi
                for n in range(N):
                    abits[n, c, p, q] = bits_of(int(xa[n, c, p, q]), i % (L - 1) + 1, L, tw, lw, wait_a)
    wbits = np.zeros((2, Cout, Cin, W, H, L), dtype=np.int64)
    for c in range(Cin):
        for u in range(W):
            for v in range(H):
                f = {"y": c * W + u, "z": u * H + v, "yz": (c % zu) * W + u}[mode]
                for co in range(Cout):
                    wbits[0, co, c, u, v] = bits_of(int(wp[co, c, u, v]), (67 + f) % (L - 1) + 1, L, tw, lw, wait_w)
                    wbits[1, co, c, u, v] = bits_of(int(wn[co, c, u, v]), (37 + f) % (L - 1) + 1, L, tw, lw, wait_w)
    y = np.zeros((N, Cout, Wo, Ho), dtype=np.int64)
    for rail, sgn in ((0, 1), (1, -1)):
        T = np.zeros((N, Cout, Wo, Ho, Cin, W, H, L), dtype=np.int64)
        for u in range(W):
            for v in range(H):
                a = abits[:, :, u:u + Wo, v:v + Ho, :]                       # n c a b t
                T[:, :, :, :, :, u, v, :] = np.einsum("ncabt,oct->noabct", a, wbits[rail, :, :, u, v, :])
        if mode == "y":
            r = np.sign(T.sum(axis=(4, 5))).sum(axis=(4, 5))
        elif mode == "z":
            r = np.sign(T.sum(axis=(5, 6))).sum(axis=(4, 5))
        else:
            r = 0
            for c0 in range(0, Cin, zu):
                r = r + np.sign(T[:, :, :, :, c0:c0 + zu].sum(axis=(4, 5))).sum(axis=(4, 5))
        y += sgn * r
    return y
