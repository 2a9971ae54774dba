"""CPU oracle of the fused layer epilogue: TEST INFRASTRUCTURE, never on the product path.

Restates, in numpy float32 and one operation at a time, the op chain the reference runs between
two SC layers (network.py:165-170): count / L (utils_functional.py:632) -> value of
BatchNorm2d_fixed, ``x * w_n + b_n`` (utils_class.py:63) -> optional relu -> AvgPool2d(2) ->
Hardtanh(0, 1) -> quantize(., 7) (utils_functional.py:33-39, applied by the next layer,
utils_class.py:32).

Pinning status: pinned against the PyTorch ops themselves (F.avg_pool2d, F.hardtanh, torch.round;
tests/test_oracle_epilogue.py); the reference's Python modules are not imported.
"""
from __future__ import annotations

import numpy as np


def layer_epilogue(counts, bit_length, w_n, b_n, relu=False, pool=True, hardtanh=True, quant7=True):
    """(activation float32, 7-bit integers uint8 or None) for int32 counts (N, C, W, H)."""
    f = np.float32
    x = counts.astype(f) / f(bit_length)
    v = x * np.asarray(w_n, dtype=f).reshape(1, -1, 1, 1)
    v = v + np.asarray(b_n, dtype=f).reshape(1, -1, 1, 1)
    if relu:
        v = np.maximum(v, f(0))
    if pool:
        w2, h2 = v.shape[2] // 2, v.shape[3] // 2
        v = v[:, :, :2 * w2, :2 * h2]
        s = v[:, :, 0::2, 0::2] + v[:, :, 0::2, 1::2]
        s = s + v[:, :, 1::2, 0::2]
        s = s + v[:, :, 1::2, 1::2]
        v = s / f(4)
    if hardtanh:
        v = np.minimum(np.maximum(v, f(0)), f(1))
    q7 = None
    if quant7:
        k = np.clip(np.rint(v * f(128)), f(-127), f(127))
        v = k / f(128)
        if hardtanh:
            q7 = k.astype(np.uint8)
    return v.astype(f), q7
