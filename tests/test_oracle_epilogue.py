"""Pins oracle/epilogue.py against the PyTorch op chain it restates (CPU)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from geo_amd import utils_functional as uf
from oracle import epilogue


def _inputs(seed, shape=(3, 5, 8, 6), L=64, H=5):
    g = torch.Generator().manual_seed(seed)
    counts = torch.randint(-H * L, H * L + 1, shape, generator=g, dtype=torch.int32)
    # per-channel affine as BatchNorm2d_fixed produces it: 8-bit integers times a power-of-two scale
    w_n = torch.randint(-127, 128, (shape[1],), generator=g).float() / 128 * 4.0
    b_n = torch.randint(-127, 128, (shape[1],), generator=g).float() / 128 * 4.0
    return counts, w_n, b_n, L


def torch_chain(counts, L, w_n, b_n, relu, pool, hardtanh, quant7):
    x = counts.float() / L
    v = x * w_n.reshape(-1, 1, 1) + b_n.reshape(-1, 1, 1)
    if relu:
        v = F.relu(v)
    if pool:
        v = F.avg_pool2d(v, 2)
    if hardtanh:
        v = F.hardtanh(v, 0, 1)
    if quant7:
        v = uf.quantize(v, prec=7)
    return v


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("relu,pool,hardtanh,quant7", [(False, True, True, True), (True, True, True, True),
                                                       (False, False, False, False), (False, False, True, True),
                                                       (True, True, False, True)])
def test_matches_torch_ops(seed, relu, pool, hardtanh, quant7):
    counts, w_n, b_n, L = _inputs(seed)
    act, q7 = epilogue.layer_epilogue(counts.numpy(), L, w_n.numpy(), b_n.numpy(), relu, pool, hardtanh, quant7)
    exp = torch_chain(counts, L, w_n, b_n, relu, pool, hardtanh, quant7).numpy()
    assert act.dtype == np.float32 and act.shape == exp.shape
    assert np.array_equal(act, exp)
    if hardtanh and quant7:
        assert q7.dtype == np.uint8 and q7.max() <= 127
        assert np.array_equal(q7.astype(np.float32) / 128, act)
    else:
        assert q7 is None


def test_odd_extents_and_rounding():
    counts, w_n, b_n, L = _inputs(5, (2, 3, 7, 5))
    act, _ = epilogue.layer_epilogue(counts.numpy(), L, w_n.numpy(), b_n.numpy())
    assert act.shape == (2, 3, 3, 2)
    assert np.array_equal(act, torch_chain(counts, L, w_n, b_n, False, True, True, True).numpy())
    # ties round to even: 0.5/128 -> 0, 1.5/128 -> 2/128
    c = np.array([[[[1]], [[3]]]], dtype=np.int32)
    act, q7 = epilogue.layer_epilogue(c, 256, [1.0, 1.0], [0.0, 0.0], pool=False)
    assert q7.reshape(-1).tolist() == [0, 2]
