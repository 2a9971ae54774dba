"""The SC networks of the reference's training script restated on this build's layer modules:
the 4-layer CNN (network.py:126-190, ``CONV_tiny_add_partial``) and VGG-16 (network.py:12-124,
``VGG16_add_partial``), and the bookkeeping of one training step (utils_own.py:81-114).  The
reference's LeNet (``CONV_minimal_add_partial``) is not restated: it builds on a layer class that
does not exist in the reference (``utils_class.Linear_Or``, network.py:204-206).
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import utils_class

# loss scale of the reference's training loop (utils_own.py:18, :81)
SCALE_FACTOR = 128


class CONV_tiny_add_partial(nn.Module):
    """conv 3->32 k5 p2 @32x32, BN, AvgPool2, Hardtanh(0,1); 32->32 k5 p2 @16x16; 32->64 k5 p2
    @8x8; conv 64->classes k4 p0 @4x4 as the classifier; BN1d.  Per-layer stream length is
    2**err[i]; load_unit / load_wait are the progressive-loading settings per layer."""

    def __init__(self, num_classes=10, c_ins=3, uniform=False, generator="lfsr", sc_compute="1d_bin", legacy=False,
                 relu=False):
        super().__init__()
        self.bn1 = utils_class.BatchNorm2d_fixed(32)
        self.bn2 = utils_class.BatchNorm2d_fixed(32)
        self.bn3 = utils_class.BatchNorm2d_fixed(64)
        self.bn4 = utils_class.BatchNorm1d_fixed(num_classes)
        self.conv1 = utils_class.Conv2d_Add_Partial(c_ins, 32, kernel_size=5, padding=2, bias=False)
        self.conv2 = utils_class.Conv2d_Add_Partial(32, 32, kernel_size=5, padding=2, bias=False)
        self.conv3 = utils_class.Conv2d_Add_Partial(32, 64, kernel_size=5, padding=2, bias=False)
        self.fc1 = utils_class.Conv2d_Add_Partial(64, num_classes, kernel_size=4, padding=0, bias=False)
        self.tanh = nn.Hardtanh(0, 1)
        self.pool = nn.AvgPool2d(2)
        self.err = [7, 7, 7, 7]
        self.z_unit = [3, 3, 4, 4]
        self.load_unit = [2, 2, 2, 2]
        self.load_wait_w = [2, 2, 2, 2]
        # the reference's forward reads `load_wait`, which its training script sets from the
        # command line (main_conv.py:182); the default there is 2 per layer
        self.load_wait = [2, 2, 2, 2]
        self.num_classes = num_classes
        self.generator = generator
        self.compute = sc_compute
        self.legacy = legacy
        self.relu = relu
        # training mode on the GPU with the LFSR kernels: run every conv + batch norm + pool +
        # hardtanh block as one fused autograd node (same values; gradients to fp32 rounding)
        self.fused_blocks = False
        # batch statistics of the fused blocks: False = from exact integer sums of the counts (one HIP kernel,
        # independent of any reduction order), True = PyTorch's two float reductions, as BatchNorm*_fixed runs
        # them (utils_class.py:52-56): bit-identical to the module chain
        self.fused_torch_stats = False
        if uniform:
            self.conv1.weight_org *= 2
            self.conv2.weight_org *= 2
            self.conv1.weight.data *= 2
            self.conv2.weight.data *= 2

    def _sc(self, conv, x, i, wait_w_index=None):
        j = i if wait_w_index is None else wait_w_index
        return conv(x, err=self.err[i], forward=self.compute, generator=self.generator, z_unit=2 ** self.z_unit[i],
                    legacy=self.legacy, load_unit=self.load_unit[i], load_wait_w=self.load_wait[j],
                    load_wait_a=self.load_wait[i])

    def _fusable(self, x):
        return (self.fused_blocks and self.training and x.is_cuda and not self.legacy and self.generator == "lfsr"
                and self.compute in ("1d_bin", "z_bin", "yz_bin"))

    def _fused(self, conv, bn, x, i, j, **tail):
        return utils_class.sc_conv_block(conv, bn, x, err=self.err[i], forward=self.compute,
                                         z_unit=2 ** self.z_unit[i], load_unit=self.load_unit[i],
                                         load_wait_w=self.load_wait[j], load_wait_a=self.load_wait[i],
                                         torch_stats=self.fused_torch_stats, weight_ready=True, **tail)

    def _block(self, conv, bn, x, i):
        if self._fusable(x):
            return self._fused(conv, bn, x, i, i, relu=self.relu)
        x = bn(self._sc(conv, x, i))
        if self.relu:
            x = F.relu(x)
        return self.tanh(self.pool(x))

    def forward(self, x_in, target=None):
        if self._fusable(x_in):
            # the four layers' weight quantisation (utils_class.py:33) in one launch
            utils_class.quantize_weights([self.conv1, self.conv2, self.conv3, self.fc1])
        x = self._block(self.conv1, self.bn1, x_in, 0)
        x = self._block(self.conv2, self.bn2, x, 1)
        x = self._block(self.conv3, self.bn3, x, 2)
        # the classifier layer takes the third layer's weight wait (network.py:186)
        if self._fusable(x):
            y = self._fused(self.fc1, self.bn4, x, 3, 2, relu=False, pool=False, hardtanh=False, quant7=False)
            return y.view(-1, self.num_classes)
        x = self._sc(self.fc1, x, 3, wait_w_index=2)
        return self.bn4(x.view(-1, self.num_classes))


    # ---------------------------------------------------------------- fused inference path
    def train(self, mode=True):
        self._fused_state = None  # parameters may change: drop the cached inference state
        return super().train(mode)

    @torch.no_grad()
    def prepare_fused(self):
        """Cache what an inference forward does not need to recompute: per layer the weight streams
        of the 7-bit-quantised weights and the quantised per-channel affine of its fixed batch
        norm on the running statistics.  Call again after changing parameters or settings."""
        if self.legacy or self.generator != "lfsr" or self.compute not in ("1d_bin", "z_bin", "yz_bin"):
            raise NotImplementedError("forward_fused runs the LFSR kernels only")
        from . import capi, utils_functional as uf
        layers = [(self.conv1, self.bn1, 0, 0), (self.conv2, self.bn2, 1, 1), (self.conv3, self.bn3, 2, 2),
                  (self.fc1, self.bn4, 3, 2)]  # (conv, bn, layer index, index of its weight wait: network.py:186)
        mode = {"1d_bin": "y", "z_bin": "z", "yz_bin": "yz"}[self.compute]
        state = []
        for conv, bn, i, j in layers:
            conv.weight.data = uf.quantize(conv.weight_org, prec=7)
            w = conv.weight.data.float().contiguous()
            wait_w = self.load_wait[j]
            kw = dict(bit_length=2 ** self.err[i], padding=(int(conv.padding[0]), int(conv.padding[1])),
                      total_width=uf.prec_default, load_width=int(self.load_unit[i]), load_wait_w=int(wait_w),
                      load_wait_a=int(self.load_wait[i] if mode == "yz" else wait_w), accumulate=mode,
                      z_unit=max(1, min(2 ** self.z_unit[i], w.shape[1])))
            w_n, b_n = utils_class._fixed_affine(bn, None, bn.running_mean, bn.running_var)
            # the weight stream buffer is generated at the first forward: its stream words do not
            # depend on the input, but what else the buffer carries depends on the layer's geometry
            state.append(dict(w=w, w_shape=tuple(w.shape), kw=kw, wgt=None, wgt_for=None,
                              w_n=w_n.float().contiguous(), b_n=b_n.float().contiguous()))
        self._fused_state = state
        self._fused_graph = None

    def _fused_eager(self, x):
        from . import capi
        last = len(self._fused_state) - 1
        for i, st in enumerate(self._fused_state):
            d = capi.make_desc(x.shape, st["w_shape"], **st["kw"])
            if st["wgt_for"] != tuple(x.shape):
                st["wgt"], st["wgt_for"] = capi.weight_streams(st["w"], d), tuple(x.shape)
            counts = capi.conv2d_add_partial_from_streams(capi.act_streams(x, d), st["wgt"], d)
            L = st["kw"]["bit_length"]
            if i == last:
                logits, _ = capi.layer_epilogue(counts, L, st["w_n"], st["b_n"], relu=False, pool=False,
                                                hardtanh=False, quant7=False)
                return logits.view(-1, self.num_classes)
            _, x = capi.layer_epilogue(counts, L, st["w_n"], st["b_n"], relu=self.relu, want_act=False, want_q7=True)

    @torch.no_grad()
    def forward_fused(self, x_in, graph=False):
        """Inference forward with one fused epilogue kernel per layer in place of the element-wise
        op chain (fixed batch norm on the running statistics, relu, AvgPool2, Hardtanh, the next
        layer's 7-bit quantisation): layers hand each other uint8 7-bit integers, which the
        activation stream generator reads directly, and weight streams come from the cache of
        ``prepare_fused``.  Same logits, bit for bit, as ``forward`` in eval mode.  ``graph=True``
        records the launches of one forward into a HIP graph per input shape and replays it."""
        if self.training:
            raise RuntimeError("forward_fused is the inference path: call model.eval() first")
        from . import utils_functional as uf
        if getattr(self, "_fused_state", None) is None:
            self.prepare_fused()
        x = uf.quantize(x_in.detach().float(), prec=7).contiguous()
        if not graph:
            return self._fused_eager(x)
        g = self._fused_graph
        if g is None or g["x"].shape != x.shape:
            static_x = x.clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):  # warm the allocator and the kernels outside the capture
                self._fused_eager(static_x)
            torch.cuda.current_stream().wait_stream(side)
            cg = torch.cuda.CUDAGraph()
            with torch.cuda.graph(cg):
                out = self._fused_eager(static_x)
            g = self._fused_graph = dict(x=static_x, out=out, graph=cg)
        g["x"].copy_(x)
        g["graph"].replay()
        return g["out"].clone()


class VGG16_add_partial(nn.Module):
    """VGG-16 for SC (network.py:12-124): thirteen 3x3 SC convolutions in five groups
    (2, 2, 3, 3, 3 layers; AvgPool2 and Dropout2d after each group), a 1x1 SC convolution as the
    classifier, fixed batch norm + Hardtanh(0,1) after every layer.  err / z_unit / load_unit /
    load_wait hold one value per group plus one for the classifier; with ``half_pool`` the layer
    in front of a pooling uses half the group's stream length (not below 2**5).  Same attribute
    names as the reference, hence the same ``state_dict`` keys."""

    GROUPS = ((1, 2), (3, 4), (5, 6, 7), (8, 9, 10), (11, 12, 13))
    WIDTHS = (64, 128, 256, 512, 512)

    def __init__(self, uniform=False, sc_compute="1d_bin", generator="lfsr", legacy=False, half_pool=True):
        super().__init__()
        c_in = 3
        for group, width in zip(self.GROUPS, self.WIDTHS):
            for i in group:
                setattr(self, f"conv{i}", utils_class.Conv2d_Add_Partial(c_in, width, kernel_size=3, padding=1,
                                                                         bias=False))
                c_in = width
        for g in range(1, 6):
            setattr(self, f"drop{g}", nn.Dropout2d())
        self.fc1 = utils_class.Conv2d_Add_Partial(512, 10, kernel_size=1, padding=0, bias=False)
        self.pool = nn.AvgPool2d(2)
        for group, width in zip(self.GROUPS, self.WIDTHS):
            for i in group:
                setattr(self, f"bn{i}", utils_class.BatchNorm2d_fixed(width))
        self.bnfc1 = utils_class.BatchNorm1d_fixed(10)
        self.tanh = nn.Hardtanh(0, 1)
        self.err = [7, 7, 7, 7, 7, 7]
        self.z_unit = [5, 5, 5, 5, 5, 5]
        self.load_unit = [2, 2, 2, 2, 2, 2]
        self.load_wait = [2, 2, 2, 2, 2, 2]
        self.generator = generator
        self.compute = sc_compute
        self.legacy = legacy
        self.half_pool = half_pool
        # training mode on the GPU with the LFSR kernels: every conv + batch norm + [pool] + hardtanh
        # block as one fused autograd node (same values; gradients to fp32 rounding)
        self.fused_blocks = False
        if min(self.err) < 4:
            uniform = True
        if uniform:
            for mod in self.modules():
                if isinstance(mod, nn.Conv2d):
                    mod.weight.data.uniform_()
                    mod.weight_org.uniform_()

    def _sc(self, conv, x, g, err):
        return conv(x, err=err, forward=self.compute, generator=self.generator, z_unit=2 ** self.z_unit[g],
                    legacy=self.legacy, load_unit=self.load_unit[g], load_wait_w=self.load_wait[g],
                    load_wait_a=self.load_wait[g])

    def _fused(self, conv, bn, x, g, err, **tail):
        return utils_class.sc_conv_block(conv, bn, x, err=err, forward=self.compute, z_unit=2 ** self.z_unit[g],
                                         load_unit=self.load_unit[g], load_wait_w=self.load_wait[g],
                                         load_wait_a=self.load_wait[g], **tail)

    def forward(self, x):
        pool_offset = 1 if self.half_pool else 0
        fuse = (self.fused_blocks and self.training and x.is_cuda and not self.legacy and self.generator == "lfsr"
                and self.compute in ("1d_bin", "z_bin", "yz_bin"))
        for g, group in enumerate(self.GROUPS):
            for i in group:
                last = i == group[-1]
                err = max(self.err[g] - pool_offset, 5) if last else self.err[g]
                conv, bn = getattr(self, f"conv{i}"), getattr(self, f"bn{i}")
                if fuse:
                    # a dropout follows the group's last layer: its input must stay unquantised
                    x = self._fused(conv, bn, x, g, err, pool=last, quant7=not last)
                    continue
                x = bn(self._sc(conv, x, g, err))
                if last:
                    x = self.pool(x)
                x = self.tanh(x)
            x = getattr(self, f"drop{g + 1}")(x)
        if fuse:
            return self._fused(self.fc1, self.bnfc1, x, 5, self.err[5], pool=False, hardtanh=False,
                               quant7=False).view(-1, 10)
        x = self._sc(self.fc1, x, 5, self.err[5]).view(-1, 10)
        return self.bnfc1(x)


def make_param_copies(model):
    """Full-precision master copies the optimiser updates (main_conv.py:203-213)."""
    return [p.detach().clone().float().requires_grad_(True) for p in model.parameters()]


def apply_update(model, optimizer, param_copy):
    """The part of the reference's step that follows ``loss.backward()`` (utils_own.py:98-114): restore
    the full-precision weights, hand the gradients to the master copies and un-scale them, optimiser
    step on the copies, copy back, refresh ``weight_org`` clamped to [-1, 0.999]."""
    # (the reference first copies weight_org back into weight.data; the copy-back from the master copies below
    # overwrites every parameter before anything reads it, so that copy changes nothing and is not launched)
    params = list(model.parameters())
    # the per-parameter loops of the reference as multi-tensor calls: one kernel for all gradients,
    # one for all copies
    with_grad = [(master, p) for master, p in zip(param_copy, params) if p.grad is not None]
    for master, p in zip(param_copy, params):
        master.grad = None
    if with_grad:
        scaled = torch._foreach_div([p.grad.data.float() for _, p in with_grad], SCALE_FACTOR)
        for (master, _), g in zip(with_grad, scaled):
            master.grad = g
    optimizer.step()
    orgs = {id(m.weight): m.weight_org for m in model.modules() if hasattr(m, "weight_org")}
    if all(p.is_cuda and p.dtype == torch.float32 and p.data.is_contiguous() for p in params):
        # copy back and refresh weight_org, all parameters in one launch
        from . import capi
        capi.copy_back_clamp([master.data for master in param_copy], [p.data for p in params],
                             [orgs.get(id(p)) for p in params], -1, 0.999)
    else:
        torch._foreach_copy_([p.data for p in params], [master.data for master in param_copy])
        for p in params:
            if id(p) in orgs:
                torch.clamp(p.data, -1, 0.999, out=orgs[id(p)])
    optimizer.zero_grad()


def train_step(model, inputs, target, criterion, optimizer, param_copy):
    """One step of the reference's loop (utils_own.py:79-114): scaled loss, backward, then
    ``apply_update``.  Returns the unscaled loss."""
    output = model(inputs)
    loss = criterion(output, target) * SCALE_FACTOR
    for p in model.parameters():
        p.grad = None
    loss.backward()
    apply_update(model, optimizer, param_copy)
    return loss.detach() / SCALE_FACTOR


class GraphedTrainStep:
    """``train_step`` for a fixed batch shape, recorded once into a HIP graph and replayed: the step's ~130
    short launches then cost the host one submission instead of one each (at batch 256 the eager step of the
    4-layer CNN is bound by the host's launch rate, not by the GPU).  Same kernels, same arithmetic, same state:
    weights, master copies, optimiser moments and running statistics live where they did and are updated in
    place by the replayed kernels.

    The optimiser must keep its step count on the device (``torch.optim.Adam(..., capturable=True)``).  Recording
    needs the allocator and the kernels warmed up by real steps; the state they change is put back afterwards
    (model buffers and parameters, master copies, optimiser state), so constructing this object leaves the
    training state as it found it.  The model must be in training mode and stay as it is (same settings, same
    ``fused_blocks``) for as long as the graph is replayed."""

    def __init__(self, model, criterion, optimizer, param_copy, inputs, target, warmup=3):
        import copy
        self.model, self.optimizer, self.param_copy = model, optimizer, param_copy
        self.inputs, self.target = inputs.detach().clone(), target.detach().clone()
        model_state = {k: v.detach().clone() for k, v in model.state_dict().items()}
        masters = [m.detach().clone() for m in param_copy]
        had_state = {id(p) for p in optimizer.state}
        opt_state = copy.deepcopy({id(p): {k: v for k, v in st.items()} for p, st in optimizer.state.items()})
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, int(warmup))):
                train_step(model, self.inputs.clone(), self.target, criterion, optimizer, param_copy)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            # a second handle on the static batch: the layer re-points its input's .data at the quantised values,
            # which must not re-point self.inputs away from the memory the recorded kernels read
            self.loss = train_step(model, self.inputs.detach(), self.target, criterion, optimizer, param_copy)
        # put the training state back, in place: the graph holds the addresses
        with torch.no_grad():
            now = model.state_dict()
            for k, v in model_state.items():
                now[k].copy_(v)
            for m, saved in zip(param_copy, masters):
                m.copy_(saved)
            for p, st in optimizer.state.items():
                for k, v in st.items():
                    if not torch.is_tensor(v):
                        continue
                    if id(p) in had_state:
                        v.copy_(opt_state[id(p)][k])
                    else:
                        v.zero_()   # a fresh state is all zeros (step count, moments)
        torch.cuda.synchronize()

    def __call__(self, inputs, target):
        """One step on a batch of the recorded shape; returns the (unscaled) loss tensor of that step, which the
        next call overwrites."""
        self.inputs.copy_(inputs)
        self.target.copy_(target)
        self.graph.replay()
        return self.loss
