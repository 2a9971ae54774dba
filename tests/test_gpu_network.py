"""The 4-layer SC CNN training step (batch 256, 3x32x32 synthetic images, stream length 64):
layer-by-layer bit-exact SC counts against the CPU oracle with neutral progressive loading,
whole-network gradients against autograd over the torch surrogate, and the step bookkeeping."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _model(load_unit, seed=0):
    from geo_amd import network
    torch.manual_seed(seed)
    m = network.CONV_tiny_add_partial().cuda()
    m.err = [6, 6, 6, 6]
    m.load_unit = [load_unit] * 4
    m.load_wait = [2, 2, 2, 2]
    return m


def _batch(n=256, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.rand((n, 3, 32, 32), generator=g).cuda(), torch.randint(10, (n,), generator=g).cuda()


@pytest.mark.parametrize("load_unit", [8, 2])
def test_layers_bit_exact_against_oracle(load_unit):
    """load_unit=8 leaves codes untouched (what the reference CPU kernel computes);
    load_unit=2, wait 2 is the training script's default and is pinned by the reference's GPU
    source text only."""
    from geo_amd import utils_functional as uf
    from oracle import sc_oracle
    model = _model(load_unit).train()
    x, _ = _batch(32)
    seen = []
    orig = uf.conv2d_generic

    def spy(activation, weight, padding, stride, **kw):
        out = orig(activation, weight, padding, stride, **kw)
        seen.append((activation.detach().cpu().numpy(), weight.detach().cpu().numpy(), tuple(padding), dict(kw),
                     out.detach().cpu().numpy()))
        return out

    uf.conv2d_generic = spy
    try:
        with torch.no_grad():
            model(x)
    finally:
        uf.conv2d_generic = orig
    assert len(seen) == 4
    for a, w, pad, kw, out in seen:
        L = kw["bit_length"]
        exp = sc_oracle.conv2d_add_partial(a, w, L, pad, 7, kw["load_unit"], kw["load_wait_w"], kw["load_wait_w"])
        assert np.array_equal(out, exp.astype(np.float32) / L)
        assert np.abs(exp).sum() > 0


def test_network_gradients_match_autograd_over_the_torch_surrogate():
    """Same forward values, two backward paths: the HIP backward kernels versus torch autograd
    through conv2d_or_bin_1d with the value overwritten (the reference's composition,
    utils_functional.py:611-634)."""
    import torch.nn.functional as F
    from geo_amd import capi, utils_functional as uf
    from oracle import surrogate
    x, t = _batch(64, seed=1)
    crit = torch.nn.CrossEntropyLoss()

    def grads(model):
        for p in model.parameters():
            p.grad = None
        (crit(model(x.clone()), t) * 128).backward()
        return [p.grad.detach().clone() for p in model.parameters()]

    model = _model(8, seed=3).train()
    g_hip = grads(model)

    def torch_surrogate(activation, weight, padding, stride, **kw):
        L = kw["bit_length"]
        counts = capi.conv2d_add_partial_forward(activation.detach().contiguous(), weight.detach().contiguous(), L,
                                                 tuple(padding), 7, kw["load_unit"], kw["load_wait_w"],
                                                 kw["load_wait_w"])
        act = F.pad(activation, (padding[0], padding[0], padding[1], padding[1]))
        pos, neg = surrogate.surrogate_rails(act, weight.clamp(0, 100), -(weight.clamp(-100, 0)))
        pos.data = counts.float() / L
        neg.data = torch.zeros_like(neg)
        return pos - neg

    orig = uf.conv2d_generic
    uf.conv2d_generic = torch_surrogate
    try:
        g_ref = grads(model)
    finally:
        uf.conv2d_generic = orig
    assert len(g_hip) == len(g_ref) == 12
    for a, b in zip(g_hip, g_ref):
        scale = b.abs().max().clamp_min(1e-20)
        # torch's own fp32 convolutions carry rounding of the same size as ours
        assert ((a - b).abs().max() / scale).item() <= 5e-5


def test_training_step_bookkeeping():
    from geo_amd import network
    model = _model(2).train()
    x, t = _batch(256)
    copies = network.make_param_copies(model)
    opt = torch.optim.Adam(copies, lr=2e-3)
    crit = torch.nn.CrossEntropyLoss()
    w_before = model.conv2.weight_org.clone()
    losses = [network.train_step(model, x.clone(), t, crit, opt, copies).item() for _ in range(3)]
    assert all(np.isfinite(losses))
    assert not torch.equal(model.conv2.weight_org, w_before)
    assert model.conv2.weight_org.max() <= 0.999 and model.conv2.weight_org.min() >= -1
    for master, p in zip(copies, model.parameters()):
        assert torch.equal(master.data, p.data)
    assert losses[-1] < losses[0] * 1.5


@pytest.mark.parametrize("compute,relu", [("1d_bin", False), ("1d_bin", True), ("yz_bin", False)])
def test_fused_training_blocks_match_module_chain(compute, relu):
    """fused_blocks=True: one autograd node per conv + batch norm + pool + hardtanh block.  Logits
    and running statistics equal the module-by-module forward; gradients agree to fp32 rounding."""
    from geo_amd import network

    def make():
        torch.manual_seed(0)
        m = network.CONV_tiny_add_partial(sc_compute=compute, relu=relu).cuda().train()
        m.err = [6, 6, 6, 6]
        with torch.no_grad():
            for bn in (m.bn1, m.bn2, m.bn3, m.bn4):
                bn.weight.uniform_(0.5, 1.5)
                bn.bias.uniform_(-0.2, 0.4)
        return m

    ref, fused = make(), make()
    fused.fused_blocks = True
    g = torch.Generator().manual_seed(1)
    x = torch.rand(32, 3, 32, 32, generator=g).cuda()
    t = torch.randint(10, (32,), generator=g).cuda()
    crit = torch.nn.CrossEntropyLoss()
    out_r = ref(x.clone())
    out_f = fused(x.clone())
    assert torch.equal(out_r, out_f)
    (crit(out_r, t) * 128).backward()
    (crit(out_f, t) * 128).backward()
    for (name, pr), (_, pf) in zip(ref.named_parameters(), fused.named_parameters()):
        assert pf.grad is not None, name
        err = (pf.grad - pr.grad).abs().max().item() / max(pr.grad.abs().max().item(), 1e-30)
        assert err < 5e-5, (name, err)
    for (name, br), (_, bf) in zip(ref.named_buffers(), fused.named_buffers()):
        if br is None:
            continue
        if br.dtype.is_floating_point:
            assert torch.allclose(br, bf, rtol=1e-5, atol=1e-7), name
        else:
            assert torch.equal(br, bf), name
    # eval mode takes the module path again
    fused.eval()
    ref.eval()
    with torch.no_grad():
        assert torch.allclose(fused(x.clone()), ref(x.clone()), atol=1e-5)


def test_tail_backward_matches_torch_autograd():
    """geo_sc_layer_tail_backward against torch autograd over batch_norm(training) -> relu ->
    avg_pool2d -> hardtanh with the forward values replaced by the fixed-point affine."""
    from geo_amd import capi, utils_class
    import torch.nn.functional as F
    for (shape, relu, pool, hardtanh) in [((8, 6, 8, 6), False, True, True), ((4, 5, 7, 5), True, True, True),
                                          ((16, 10, 1, 1), False, False, False), ((3, 4, 6, 6), True, False, True)]:
        L = 64
        g = torch.Generator().manual_seed(shape[0])
        counts = torch.randint(-3 * L, 3 * L + 1, shape, generator=g, dtype=torch.int32).cuda()
        bn = utils_class.BatchNorm2d_fixed(shape[1]).cuda().train()
        with torch.no_grad():
            bn.weight.uniform_(0.5, 1.5)
            bn.bias.uniform_(-0.2, 0.6)
        y = (counts.float() / L).requires_grad_(True)
        v = bn(y)
        if relu:
            v = F.relu(v)
        if pool:
            v = F.avg_pool2d(v, 2)
        if hardtanh:
            v = F.hardtanh(v, 0, 1)
        go = torch.randn(v.shape, generator=g).cuda()
        v.backward(go)
        yd = y.detach()
        mean, var = yd.mean((0, 2, 3)), yd.var((0, 2, 3), unbiased=False)
        w_n, b_n = utils_class._fixed_affine(bn, None, mean, var)
        gy, gg, gb = capi.layer_tail_backward(counts, go, L, w_n, b_n, mean, torch.rsqrt(var + 1e-5), bn.weight.detach(),
                                              relu, pool, hardtanh)
        for got, ref in ((gy, y.grad), (gg, bn.weight.grad), (gb, bn.bias.grad)):
            err = (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)
            assert err < 2e-5, (shape, err)


def test_count_stats_are_the_correctly_rounded_channel_statistics():
    """geo_sc_count_stats against float64 mean and biased variance of counts / L (utils_class.py:52-56):
    equal to the float64 result rounded to fp32, for whole-quad planes, ragged planes, an unaligned
    tensor, single-position layers and negative counts."""
    from geo_amd import capi
    for shape, L in [((32, 6, 8, 8), 64), ((5, 3, 7, 5), 32), ((256, 32, 16, 16), 64), ((16, 10, 1, 1), 128),
                     ((3, 70, 4, 4), 256)]:
        g = torch.Generator().manual_seed(shape[1])
        counts = torch.randint(-5 * L, 5 * L + 1, shape, generator=g, dtype=torch.int32).cuda()
        y = counts.double() / L
        dims = (0, 2, 3)
        ref_mean, ref_var = y.mean(dims), y.var(dims, unbiased=False)
        mean, var = capi.count_stats(counts, L)
        assert torch.equal(mean, ref_mean.float()), shape
        # the variance is a difference of two exact terms rounded once: within one fp32 step of the fp64 value
        assert torch.allclose(var.double(), ref_var, rtol=2e-7, atol=0), shape
        # a tensor that does not start on a 16-byte boundary takes the one-count loads: same bits
        off = torch.empty(counts.numel() + 1, dtype=torch.int32, device="cuda")[1:].view(shape)
        off.copy_(counts)
        m2, v2 = capi.count_stats(off, L)
        assert torch.equal(m2, mean) and torch.equal(v2, var), shape
    const = torch.full((4, 2, 4, 4), 37, dtype=torch.int32, device="cuda")
    mean, var = capi.count_stats(const, 64)
    assert torch.equal(mean, torch.full((2,), 37 / 64, device="cuda")) and torch.equal(var, torch.zeros(2, device="cuda"))


def test_fused_block_with_either_source_of_batch_statistics():
    """sc_conv_block with the statistics from the exact integer sums (default) and from PyTorch's float
    reductions (torch_stats=True): the same block output and running statistics to fp32 rounding."""
    from geo_amd import utils_class
    outs = []
    for torch_stats in (False, True):
        torch.manual_seed(3)
        conv = utils_class.Conv2d_Add_Partial(8, 12, 3, padding=1, bias=False).cuda()
        bn = utils_class.BatchNorm2d_fixed(12).cuda().train()
        x = torch.rand(16, 8, 8, 8, generator=torch.Generator().manual_seed(4)).cuda()
        out = utils_class.sc_conv_block(conv, bn, x, err=6, torch_stats=torch_stats)
        outs.append((out.detach().clone(), bn.running_mean.clone(), bn.running_var.clone()))
    assert torch.allclose(outs[0][0], outs[1][0], atol=1.0 / 128 + 1e-6)   # at most one step of the 7-bit output
    assert (outs[0][0] != outs[1][0]).float().mean().item() < 0.01
    assert torch.allclose(outs[0][1], outs[1][1], rtol=1e-5, atol=1e-7)
    assert torch.allclose(outs[0][2], outs[1][2], rtol=1e-5, atol=1e-7)


def test_fused_training_blocks_at_the_benchmarked_batch():
    """Batch 256 with the training script's loading defaults (load_unit 2, wait 2): the configuration the
    benchmark's training step runs.  With PyTorch's float reductions for the batch statistics
    (fused_torch_stats=True: what BatchNorm*_fixed itself computes, utils_class.py:52-56) the fused blocks give
    the module chain's logits and scale buffers bit for bit (running statistics to fp32 rounding) - for three sets of weights
    (the initial ones of three seeds, each after a training step of its own as well).  With the default
    statistics from exact integer sums the correctly rounded mean and variance can differ from PyTorch's in
    the last bit, which the 8-bit rounding of the affine hides except on a rounding boundary: the fraction of
    logits that differ is printed and bounded."""
    from geo_amd import network

    x, t = _batch(256)
    crit = torch.nn.CrossEntropyLoss()
    differing = []
    for seed in (0, 1, 2):
        chain = _model(2, seed).train()
        copies = network.make_param_copies(chain)
        opt = torch.optim.Adam(copies, lr=2e-3)
        for step in range(2):
            fused = {}
            for torch_stats in (False, True):
                m = _model(2, seed).train()
                m.load_state_dict(chain.state_dict(), strict=False)   # 'scale' is None until the first forward
                m.fused_blocks, m.fused_torch_stats = True, torch_stats
                fused[torch_stats] = m
            before = {k: v.clone() for k, v in chain.state_dict().items() if v is not None}
            ref = chain(x.clone()).detach().clone()
            got = fused[True](x.clone()).detach()
            assert torch.equal(got, ref), (seed, step)
            for (name, br), (_, bt) in zip(chain.named_buffers(), fused[True].named_buffers()):
                if br is None:
                    continue
                if name.endswith("scale"):
                    assert torch.equal(br, bt), (seed, step, name)
                elif name.endswith(("running_mean", "running_var")):
                    # F.batch_norm updates these from the mean and variance its own kernel reduces, not from
                    # the two reductions BatchNorm*_fixed takes its affine from: equal to fp32 rounding
                    assert torch.allclose(br, bt, rtol=2e-6, atol=1e-8), (seed, step, name)
            differing.append((fused[False](x.clone()).detach() != ref).float().mean().item())
            # next set of weights: one training step of the module chain from the state before this forward
            chain.load_state_dict(before, strict=False)
            network.train_step(chain, x.clone(), t, crit, opt, copies)
    print("fraction of logits that differ between exact and PyTorch batch statistics:", differing)
    assert max(differing) <= 0.05


@pytest.mark.parametrize("fused_adam", [False, True])
def test_training_step_replayed_from_a_hip_graph(fused_adam):
    """network.GraphedTrainStep against the eager step on the same sequence of batches: equal losses, weights,
    master copies and running statistics after every step (the graph is replayed four times, with eager work of
    the program and synchronisations in between), and recording leaves the training state untouched."""
    from geo_amd import network
    crit = torch.nn.CrossEntropyLoss()
    batches = [_batch(64, seed=s) for s in (1, 2, 3, 4)]

    def make():
        m = _model(2, seed=5).train()
        m.fused_blocks = True
        copies = network.make_param_copies(m)
        return m, copies, torch.optim.Adam(copies, lr=2e-3, capturable=True, fused=fused_adam)

    eager, e_copies, e_opt = make()
    graphed, g_copies, g_opt = make()
    before = {k: v.clone() for k, v in graphed.state_dict().items()}
    step = network.GraphedTrainStep(graphed, crit, g_opt, g_copies, *batches[0])
    for k, v in graphed.state_dict().items():
        if k in before:
            assert torch.equal(v, before[k]), k
    for a, b in zip(e_copies, g_copies):
        assert torch.equal(a, b)
    for i, (x, t) in enumerate(batches):
        loss_e = network.train_step(eager, x.clone(), t, crit, e_opt, e_copies)
        torch.cuda.synchronize()
        loss_g = step(x, t).clone()
        torch.cuda.synchronize()
        assert torch.equal(loss_e, loss_g), (i, loss_e.item(), loss_g.item())
        for (name, a), (_, b) in zip(eager.state_dict().items(), graphed.state_dict().items()):
            assert torch.equal(a, b), (i, name)
        for a, b in zip(e_copies, g_copies):
            assert torch.equal(a, b), i
    assert torch.isfinite(loss_g)
