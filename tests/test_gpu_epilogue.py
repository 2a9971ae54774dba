"""GPU parity of the fused layer epilogue and of the 7-bit-integer activation input, through the
C ABI, against the CPU oracle and against the PyTorch op chain; and of the fused inference
forward of the 4-layer CNN against its module-by-module forward.  Bit-exact."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from geo_amd import workloads as wl

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from geo_amd import capi as m
    return m


def _inputs(seed, shape, L, H=5):
    g = torch.Generator().manual_seed(seed)
    counts = torch.randint(-H * L, H * L + 1, shape, generator=g, dtype=torch.int32)
    w_n = torch.randint(-127, 128, (shape[1],), generator=g).float() / 128 * 4.0
    b_n = torch.randint(-127, 128, (shape[1],), generator=g).float() / 128 * 4.0
    return counts, w_n, b_n


@pytest.mark.parametrize("shape,L", [((3, 5, 8, 6), 64), ((2, 3, 7, 5), 256), ((4, 32, 32, 32), 128),
                                     ((70, 10, 1, 1), 64)])
@pytest.mark.parametrize("relu,pool,hardtanh,quant7", [(False, True, True, True), (True, True, True, True),
                                                       (False, False, False, False), (False, False, True, True),
                                                       (True, True, False, True)])
def test_epilogue_matches_oracle(capi, shape, L, relu, pool, hardtanh, quant7):
    from oracle import epilogue
    if pool and min(shape[2:]) < 2:
        pytest.skip("nothing to pool")
    counts, w_n, b_n = _inputs(L + shape[0], shape, L)
    want_q7 = hardtanh and quant7
    act, q7 = capi.layer_epilogue(counts.cuda(), L, w_n, b_n, relu, pool, hardtanh, quant7, want_q7=want_q7)
    torch.cuda.synchronize()
    e_act, e_q7 = epilogue.layer_epilogue(counts.numpy(), L, w_n.numpy(), b_n.numpy(), relu, pool, hardtanh, quant7)
    assert np.array_equal(act.cpu().numpy(), e_act)
    if want_q7:
        assert np.array_equal(q7.cpu().numpy(), e_q7)
        only_q7 = capi.layer_epilogue(counts.cuda(), L, w_n, b_n, relu, pool, hardtanh, quant7, want_act=False,
                                      want_q7=True)
        assert only_q7[0] is None and torch.equal(only_q7[1], q7)


def test_epilogue_matches_torch_ops_on_real_counts(capi):
    """Counts of an SC layer, the affine of a BatchNorm2d_fixed in eval mode, and the op chain
    as the reference's network runs it (network.py:165-170)."""
    from geo_amd import utils_class, utils_functional as uf
    x, w = wl.make_inputs((8, 16, 12, 12), (24, 16, 5, 5), "q7", seed=3)
    counts = capi.conv2d_add_partial_forward(x.cuda(), w.cuda(), 64, (2, 2))
    bn = utils_class.BatchNorm2d_fixed(24).cuda().eval()
    with torch.no_grad():
        bn.running_mean.uniform_(-0.2, 0.2)
        bn.running_var.uniform_(0.05, 0.5)
        bn.weight.uniform_(0.5, 1.5)
        bn.bias.uniform_(-0.3, 0.3)
        ref = uf.quantize(F.hardtanh(F.avg_pool2d(bn(counts.float() / 64), 2), 0, 1), prec=7)
        w_n, b_n = utils_class._fixed_affine(bn, None, bn.running_mean, bn.running_var)
    act, q7 = capi.layer_epilogue(counts, 64, w_n, b_n, want_q7=True)
    assert torch.equal(act, ref)
    assert torch.equal(q7.float() / 128, ref)


@pytest.mark.parametrize("L", [8, 64, 128, 256])
@pytest.mark.parametrize("mode,zu", [("y", 1), ("z", 1), ("yz", 2)])
def test_q7_activations_give_the_fp32_counts(capi, L, mode, zu):
    g = torch.Generator().manual_seed(L)
    k = torch.randint(0, 128, (3, 5, 7, 6), generator=g, dtype=torch.uint8)
    _, w = wl.make_inputs((3, 5, 7, 6), (19, 5, 3, 3), "prescribed", seed=L)
    wd = w.cuda()
    for loading in ((7, 8, 1, 1), (7, 2, 2, 3)):
        a = capi.conv2d_add_partial_forward_q7(k.cuda(), wd, L, (1, 1), *loading, accumulate=mode, z_unit=zu)
        b = capi.conv2d_add_partial_forward((k.float() / 128).cuda(), wd, L, (1, 1), *loading, accumulate=mode,
                                            z_unit=zu)
        assert torch.equal(a, b)
    # single-row outputs use the batch-item-innermost stream layout
    k1 = torch.randint(0, 128, (6, 4, 3, 8), generator=g, dtype=torch.uint8)
    _, w1 = wl.make_inputs((6, 4, 3, 8), (5, 4, 3, 3), "prescribed", seed=1)
    assert torch.equal(capi.conv2d_add_partial_forward_q7(k1.cuda(), w1.cuda(), L),
                       capi.conv2d_add_partial_forward((k1.float() / 128).cuda(), w1.cuda(), L))


def test_epilogue_argument_errors(capi):
    counts, w_n, b_n = _inputs(0, (2, 3, 4, 4), 64)
    with pytest.raises(capi.GeoScError):
        capi.layer_epilogue(counts.cuda(), 100, w_n, b_n)
    with pytest.raises(capi.GeoScError):   # the 7-bit output needs the clamp and the quantisation
        capi.layer_epilogue(counts.cuda(), 64, w_n, b_n, hardtanh=False, want_q7=True)
    with pytest.raises(ValueError):
        capi.layer_epilogue(counts.cuda(), 64, w_n[:2], b_n)
    with pytest.raises(ValueError):
        capi.layer_epilogue(counts, 64, w_n, b_n)


@pytest.mark.parametrize("compute,relu", [("1d_bin", False), ("1d_bin", True), ("yz_bin", False)])
def test_fused_inference_forward_equals_module_forward(compute, relu):
    from geo_amd import network
    torch.manual_seed(0)
    model = network.CONV_tiny_add_partial(sc_compute=compute, relu=relu).cuda()
    model.err = [6, 6, 6, 6]
    with torch.no_grad():
        for bn in (model.bn1, model.bn2, model.bn3, model.bn4):
            bn.running_mean.uniform_(-0.1, 0.3)
            bn.running_var.uniform_(0.02, 0.3)
            bn.weight.uniform_(0.5, 1.5)
            bn.bias.uniform_(-0.2, 0.4)
    model.eval()
    x = torch.rand(16, 3, 32, 32, generator=torch.Generator().manual_seed(1)).cuda()
    with torch.no_grad():
        ref = model(x.clone())
    got = model.forward_fused(x.clone())
    assert got.shape == ref.shape == (16, 10)
    assert torch.equal(got, ref)
    # HIP-graph replays, with eager work and synchronisations between them, against eager results
    for seed in (2, 3, 4):
        xs = torch.rand(16, 3, 32, 32, generator=torch.Generator().manual_seed(seed)).cuda()
        with torch.no_grad():
            ref_s = model(xs.clone())
        torch.cuda.synchronize()
        assert torch.equal(model.forward_fused(xs, graph=True), ref_s), seed
    # another batch size records another graph
    xb = torch.rand(5, 3, 32, 32, generator=torch.Generator().manual_seed(9)).cuda()
    with torch.no_grad():
        ref_b = model(xb.clone())
    assert torch.equal(model.forward_fused(xb, graph=True), ref_b)
    # parameters changed: the cache is rebuilt after train()/eval()
    model.train()
    with torch.no_grad():
        model.conv2.weight_org.mul_(0.5)
    model.eval()
    with torch.no_grad():
        ref2 = model(x.clone())
    assert not torch.equal(ref2, ref)
    assert torch.equal(model.forward_fused(x.clone()), ref2)
    model.train()
    with pytest.raises(RuntimeError):
        model.forward_fused(x)


@pytest.mark.parametrize("c,affine", [(10, True), (32, True), (64, False), (512, True), (700, True)])
def test_bn_fixed_affine_matches_torch_ops(capi, c, affine):
    """geo_sc_bn_fixed_affine against BatchNorm2d_fixed's own per-channel arithmetic
    (utils_class.py:52-62) and F.batch_norm's running-statistics update."""
    from geo_amd import utils_class
    g = torch.Generator().manual_seed(c)
    bn = utils_class.BatchNorm2d_fixed(c, affine=affine).cuda()
    mean = (torch.rand(c, generator=g) - 0.3).cuda()
    var = (torch.rand(c, generator=g) * 0.5 + 0.01).cuda()
    if affine:
        with torch.no_grad():
            bn.weight.copy_(torch.rand(c, generator=g) + 0.5)
            bn.bias.copy_(torch.rand(c, generator=g) - 0.5)
    rm, rv = torch.rand(c, generator=g).cuda(), (torch.rand(c, generator=g) + 0.5).cuda()
    m = 4096
    exp_w, exp_b = utils_class._fixed_affine(bn, None, mean, var)
    exp_scale = bn.scale.clone()
    exp_rm = rm * 0.9 + mean * 0.1
    exp_rv = rv * 0.9 + (var * (m / (m - 1))) * 0.1
    w_n, b_n, invstd, scale = capi.bn_fixed_affine(mean, var, bn.weight.detach() if affine else None,
                                                   bn.bias.detach() if affine else None, bn.eps, m, rm, rv)
    exp_w = exp_w if torch.is_tensor(exp_w) else torch.full((c,), float(exp_w), device="cuda")
    assert torch.equal(scale, exp_scale)
    assert torch.equal(w_n, exp_w.expand(c)) and torch.equal(b_n, exp_b.expand(c))
    assert torch.allclose(invstd, torch.rsqrt(var + 1e-5), rtol=1e-6)
    assert torch.allclose(rm, exp_rm, rtol=1e-6, atol=1e-7) and torch.allclose(rv, exp_rv, rtol=1e-6, atol=1e-7)


def test_quantize_kernel_equals_the_torch_op_chain():
    """geo_sc_quantize against (x * 2^p).round().clamp(+-(2^p - 1)) / 2^p (utils_functional.py:33-39):
    bit for bit, including ties (half to even), the clamp ends, zeros' signs aside, and NaN."""
    from geo_amd import capi, utils_functional as uf
    g = torch.Generator().manual_seed(5)
    x = (torch.rand(100003, generator=g) * 4 - 2)
    x[:16] = torch.tensor([0.5 / 128, 1.5 / 128, 2.5 / 128, -0.5 / 128, -1.5 / 128, 127.5 / 128, 1.0, -1.0, 3.0, -3.0,
                           0.0, 126.5 / 128, 1e-9, -1e-9, float("inf"), float("-inf")])
    x[16] = float("nan")
    xd = x.cuda()
    for prec in (7, 8, 3):
        p2 = 2 ** prec
        ref = (xd * p2).round().clamp(-p2 + 1, p2 - 1) / p2
        got = capi.quantize(xd, prec)
        same = (got == ref) | (got.isnan() & ref.isnan())
        assert bool(same.all()), (prec, x[~same.cpu()][:5])
        # the functional entry takes the kernel for fp32 GPU tensors and the op chain elsewhere
        assert torch.equal(torch.nan_to_num(uf.quantize(xd, prec)), torch.nan_to_num(ref))
        assert torch.equal(torch.nan_to_num(uf.quantize(x, prec)), torch.nan_to_num(ref.cpu()))
    y = xd.clone()
    assert capi.quantize(y, 7, out=y) is y and torch.equal(torch.nan_to_num(y), torch.nan_to_num(capi.quantize(xd, 7)))
    assert capi.quantize(torch.empty(0, device="cuda"), 7).numel() == 0


def test_quantize_many_equals_quantize_per_tensor(capi):
    """geo_sc_quantize_many: every tensor of the list as geo_sc_quantize gives it (odd sizes, an empty one, more
    tensors than one launch takes)."""
    g = torch.Generator().manual_seed(11)
    sizes = [1, 3, 1000, 4097, 0, 25 * 32 * 32, 7] + [5] * 23
    xs = [(torch.rand(n, generator=g) * 4 - 2).cuda() for n in sizes]
    assert len(xs) == 30
    xs[2][:4] = torch.tensor([0.5 / 128, 1.5 / 128, -2.5 / 128, 127.5 / 128], device="cuda")   # ties
    for prec in (7, 3):
        got = capi.quantize_many(xs, prec)
        for x, q in zip(xs, got):
            assert q.shape == x.shape and torch.equal(q, capi.quantize(x, prec))
    assert capi.quantize_many([], 7) == []
    with pytest.raises(Exception):
        capi.quantize_many(xs, 0)   # precision out of range


def test_copy_back_clamp_equals_the_torch_ops(capi):
    """geo_sc_copy_back_clamp against the end of the reference's training step (utils_own.py:108-113):
    p.data <- master, weight_org <- master.clamp(-1, 0.999), for parameters with and without such a buffer."""
    g = torch.Generator().manual_seed(12)
    sizes = [25 * 3 * 32, 10, 4099, 64, 1]
    masters = [(torch.rand(n, generator=g) * 3 - 1.5).cuda() for n in sizes]
    masters[1][:4] = torch.tensor([-1.0, 0.999, 1.0, -1.0000001], device="cuda")
    params = [torch.full((n,), 7.0, device="cuda") for n in sizes]
    orgs = [torch.full((n,), 9.0, device="cuda") if i % 2 == 0 else None for i, n in enumerate(sizes)]
    capi.copy_back_clamp(masters, params, orgs, -1.0, 0.999)
    torch.cuda.synchronize()
    for m, p, o in zip(masters, params, orgs):
        assert torch.equal(p, m)
        if o is not None:
            assert torch.equal(o, m.clamp(-1.0, 0.999))
    capi.copy_back_clamp([], [], [], -1.0, 0.999)
    with pytest.raises(ValueError):
        capi.copy_back_clamp(masters[:1], [params[1]], [None], -1.0, 0.999)   # sizes differ
    # more tensors than one launch takes
    many_m = [(torch.rand(9, generator=g) * 3 - 1.5).cuda() for _ in range(30)]
    many_p, many_o = [torch.zeros(9, device="cuda") for _ in many_m], [torch.zeros(9, device="cuda") for _ in many_m]
    capi.copy_back_clamp(many_m, many_p, many_o, -1.0, 0.999)
    for m, p, o in zip(many_m, many_p, many_o):
        assert torch.equal(p, m) and torch.equal(o, m.clamp(-1.0, 0.999))


@pytest.mark.parametrize("shape,L", [((64, 32, 16, 16), 64), ((37, 10, 1, 1), 64), ((8, 700, 4, 4), 128), ((256, 64, 4, 4), 256)])
def test_bn_fixed_from_counts_is_statistics_plus_affine(capi, shape, L):
    """geo_sc_bn_fixed_from_counts = geo_sc_count_stats + geo_sc_bn_fixed_affine (two launches instead of three,
    the partial sums handed over in the workspace): the same bits in every output, and the exact statistics
    against float64 sums of the integers."""
    g = torch.Generator().manual_seed(shape[1])
    counts = torch.randint(-5 * L, 5 * L + 1, shape, generator=g, dtype=torch.int32).cuda()
    c = shape[1]
    gamma, beta = (torch.rand(c, generator=g) + 0.5).cuda(), (torch.rand(c, generator=g) - 0.5).cuda()
    rm0, rv0 = torch.rand(c, generator=g).cuda(), (torch.rand(c, generator=g) + 0.5).cuda()
    rm1, rv1 = rm0.clone(), rv0.clone()
    mean, var, w_n, b_n, invstd, scale = capi.bn_fixed_from_counts(counts, L, gamma, beta, 1e-5, rm1, rv1)
    m2, v2 = capi.count_stats(counts, L)
    n_per = counts.numel() // c
    rm2, rv2 = rm0.clone(), rv0.clone()
    w2, b2, i2, s2 = capi.bn_fixed_affine(m2, v2, gamma, beta, 1e-5, n_per, rm2, rv2)
    torch.cuda.synchronize()
    for a, b in ((mean, m2), (var, v2), (w_n, w2), (b_n, b2), (invstd, i2), (scale, s2), (rm1, rm2), (rv1, rv2)):
        assert torch.equal(a, b)
    # the statistics from the integers themselves: sums in int64 (exact), one division in float64
    ci = counts.cpu().long().permute(1, 0, 2, 3).reshape(c, -1)
    s1, s2 = ci.sum(1), (ci * ci).sum(1)
    exact_mean = (s1.double() / (n_per * L)).float()
    exact_var = ((n_per * s2 - s1 * s1).double() / (float(n_per) ** 2 * float(L) ** 2)).float()
    assert torch.equal(mean.cpu(), exact_mean)
    ulp = torch.abs(torch.nextafter(exact_var, torch.full_like(exact_var, float("inf"))) - exact_var)
    assert bool((torch.abs(var.cpu() - exact_var) <= ulp).all())
