#!/usr/bin/env python3
"""Benchmark of the SC convolution hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--length 128]
                    [--no-cpu-baseline] [--no-configs]

One step = one pass of the hot path over one batch of synthetic input that is already
resident in HBM: float->code conversion, LFSR stream generation for weights and
activations, the AND/OR/popcount convolution, then the surrogate backward (both gradients)
for an upstream gradient of the output's shape.  ``--pass fwd`` times the forward alone.
Prints ONE JSON line; ``value`` is SC bit-MACs of the step divided by the step's whole
duration (the backward does no bit-MACs, so the forward-only rate is reported next to it).

The default workload is the configuration the headline metric is quoted on: SC conv2d
128->128 3x3 at 16x16, batch 256, pad 1, stream length 128, activations U[0,1), weights
U[-1,1) (with these distributions every OR rail saturates, so this input is for timing
only; the kernels have no data-dependent early exit).  After the headline the default run also times
the other benchmark configurations (C3 at stream lengths 32 and 256, C5, C4, the C2 training step) and
reports them under the key ``configs``.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X nominal peaks used for the roofline fractions
PEAK_VALU_WORD_OPS = 256 * 64 * 2.4e9   # CUs x lanes x clock: 32-bit VALU ops per second
PEAK_HBM_BYTES = 8.0e12


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C3", choices=["C1", "C2", "C3", "C4", "C5"],
                    help="C3 (default): the headline layer; C2: the 4-layer SC CNN training step")
    ap.add_argument("--length", type=int, default=0, help="stream length (default: the workload's)")
    ap.add_argument("--accumulate", default="y", choices=["y", "z", "yz", "full"],
                    help="accumulation mode of the single-layer workloads (default y: the headline)")
    ap.add_argument("--z-unit", type=int, default=32, help="channels per OR group for --accumulate yz")
    ap.add_argument("--generator", default="lfsr", choices=["lfsr", "acc", "rand"])
    ap.add_argument("--pass", dest="passes", default="fwdbwd", choices=["fwd", "fwdbwd"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--fused-only", action="store_true",
                    help="workload C2: time the fused, graph-replayed training step only (no module-chain and eager "
                         "legs): the run that kernel traces of the step are taken from")
    ap.add_argument("--probe-mfma-forward", action="store_true",
                    help="instead of a workload: the matrix-core probe (one stream cycle and kernel row of the headline "
                         "layer's forward as an fp4 GEMM tile per CU) and what it projects for the whole layer")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the other benchmark configurations that the default run times after the headline")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="also launch one plain device copy of this many MiB (reads MIB, writes MIB): the known-size "
                         "kernel that hardware traffic counters are scaled by")
    return ap.parse_args()


def time_events(fn, steps, warmup, torch):
    """Per-call durations (ms) measured with events on the stream fn launches on."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in evs]


def profiled_traffic(workload, L):
    """(HBM bytes per launch, kernel name) of the dominant kernel from the rocprofv3 counter runs
    summarised in profiles/traffic.json; (None, None) for a workload that has not been profiled.
    Not measured in this run: hardware counters need the profiler around the process."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f).get(f"{workload}_L{L}")
    except OSError:
        return None, None
    return (None, None) if t is None else (t["fetch_bytes"] + t["write_bytes"], t["kernel"])


def cpu_baseline(x, w, L, pad):
    """The reference's own CPU kernel (compiled from its source into oracle/_ref) when it is
    loadable here, else this repository's C restatement of it; timed on the host cores."""
    import torch
    from oracle import sc_oracle as so

    threads = torch.get_num_threads()
    ref = so.load_ref()
    if ref is not None:
        kind = "reference"

        def run():
            return ref.conv2d_add_partial_new(x, w, L, (pad, pad), (1, 1))
        variant = so.ref_variants_usable()[0]
        try:
            threads = len(os.sched_getaffinity(0))
        except AttributeError:
            pass
        threads = min(threads, so.max_threads())
        note = f"sc.cpp compiled -O3 -fopenmp ({variant} path), OpenMP over batch"
    else:
        kind = "port"
        threads = so.max_threads()
        xn, wn = x.numpy(), w.numpy()

        def run():
            return so.conv2d_add_partial(xn, wn, L, (pad, pad), fast=True)
        note = "C restatement (oracle/sc_oracle.c, fast loop order), OpenMP over batch"
    run()  # warm-up
    times = []
    budget_start = time.time()
    for _ in range(5):
        t = time.time()
        run()
        times.append(time.time() - t)
        if time.time() - budget_start > 25:
            break
    return kind, threads, statistics.median(times), note


C2_LAYERS = [  # (name, x shape, w shape, pad) of CONV_tiny_add_partial at batch 256
    ("conv1", (256, 3, 32, 32), (32, 3, 5, 5), 2),
    ("conv2", (256, 32, 16, 16), (32, 32, 5, 5), 2),
    ("conv3", (256, 32, 8, 8), (64, 32, 5, 5), 2),
    ("fc1", (256, 64, 4, 4), (10, 64, 4, 4), 0),
]


def network_step_result(args, torch):
    """4-layer SC CNN training step (network.py:126-190 topology, utils_own.py:81-114 step):
    batch 256 synthetic 3x32x32 images U[0,1), 10 uniform random classes, stream length 64,
    LFSR generators, progressive loading load_unit=2 / load_wait=2 (the training script's
    defaults), Adam lr 2e-3 on full-precision master copies."""
    from geo_amd import capi, network
    from geo_amd import workloads as wl

    L = args.length or 64
    torch.manual_seed(0)
    g = torch.Generator().manual_seed(0)
    x = torch.rand((256, 3, 32, 32), generator=g).cuda()
    t = torch.randint(10, (256,), generator=g).cuda()
    crit = torch.nn.CrossEntropyLoss()

    def timed_steps(fused_blocks, graph=False, torch_stats=False):
        """ms per training step.  fused_blocks: every conv + batch norm + pool + hardtanh block as one autograd
        node on the fused HIP tail kernels (same values as the module chain); graph: the step recorded once into
        a HIP graph and replayed (network.GraphedTrainStep); torch_stats: batch statistics from PyTorch's float
        reductions instead of the exact integer sums."""
        torch.manual_seed(0)
        model = network.CONV_tiny_add_partial().cuda().train()
        model.err = [L.bit_length() - 1] * 4
        model.load_unit = [2] * 4
        model.load_wait = [2] * 4
        model.fused_blocks = fused_blocks
        model.fused_torch_stats = torch_stats
        copies = network.make_param_copies(model)
        # the optimiser of the training script (main_conv.py:213); its multi-tensor form in one kernel, step
        # count on the device so that the step can be recorded
        opt = torch.optim.Adam(copies, lr=2e-3, capturable=True, fused=True) if graph \
            else torch.optim.Adam(copies, lr=2e-3)
        if graph:
            replay = network.GraphedTrainStep(model, crit, opt, copies, x, t)
            step = lambda: replay(x, t)
        else:
            step = lambda: network.train_step(model, x.clone(), t, crit, opt, copies)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    ms_per_step = timed_steps(True, graph=True)
    if args.fused_only:
        ms_module_chain = ms_eager = ms_torch_stats = None
    else:
        ms_module_chain = timed_steps(False)
        ms_eager = timed_steps(True)
        ms_torch_stats = timed_steps(True, graph=True, torch_stats=True)

    layers = {}
    B_total = 0
    word_ops_total = 0.0
    k_total = 0.0
    for name, sx, sw, pad in C2_LAYERS:
        xa, wa = wl.make_inputs(sx, sw, "q7", 0)
        xa, wa = xa.cuda(), wa.cuda()
        d = capi.make_desc(sx, sw, L, (pad, pad), 7, 2, 2, 2)
        ws = torch.empty(capi.workspace_size(d), dtype=torch.uint8, device="cuda")
        wsb = torch.empty(capi.backward_workspace_size(d), dtype=torch.uint8, device="cuda")
        out = torch.empty(capi.output_shape(d), dtype=torch.int32, device="cuda")
        gy = torch.randn(out.shape, device="cuda")
        f = time_events(lambda: capi.conv2d_add_partial_forward(xa, wa, L, (pad, pad), out=out, workspace=ws, desc=d),
                        args.steps, 2, torch)
        b = time_events(lambda: capi.conv2d_add_partial_backward(xa, wa, gy, L, (pad, pad), workspace=wsb, desc=d,
                                                                 need_grad_x=(name != "conv1")), args.steps, 2, torch)
        act = capi.act_streams(xa, d)
        wgt = capi.weight_streams(wa, d)
        k = time_events(lambda: capi.conv2d_add_partial_from_streams(act, wgt, d, out=out), args.steps, 2, torch)
        B = wl.bit_macs(sx, sw, pad, L)
        B_total += B
        ops = min_word_ops(sx, sw, pad, L)
        word_ops_total += ops
        k_total += sum(k) / len(k)
        layers[name] = {"fwd_ms": sum(f) / len(f), "bwd_ms": sum(b) / len(b), "conv_kernel_ms": sum(k) / len(k),
                        "bit_macs": B, "valu_frac": ops / (sum(k) / len(k) * 1e-3) / PEAK_VALU_WORD_OPS}
    achieved = word_ops_total / (k_total * 1e-3)
    result = {
        "metric": f"SC bit-MACs/sec over one training step of the 4-layer SC CNN at stream len {L}",
        "value": B_total / (ms_per_step * 1e-3), "unit": "bit-MAC/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": DTYPE_FWD_BWD,
        "data": "synthetic (torch.manual_seed(0); images U[0,1), uniform random labels)",
        "config": {"workload": "C2: 4-layer SC CNN (3->32 k5 @32, 32->32 k5 @16, 32->64 k5 @8, 64->10 k4 @4), batch "
                               f"256, stream length {L}, load_unit 2 / load_wait 2, fwd+bwd+Adam step, fused "
                               "conv + batch-norm + pool + hardtanh blocks, batch statistics from exact integer sums "
                               "of the counts, step replayed from a HIP graph",
                   "pass": "train step", "bit_macs_per_step": B_total},
        # the same step launched kernel by kernel from Python; with PyTorch's float reductions for the batch
        # statistics (bit-identical to the module chain); module by module with PyTorch ops between the SC kernels
        "eager_ms_per_step": ms_eager,
        "torch_statistics_ms_per_step": ms_torch_stats,
        "module_chain_ms_per_step": ms_module_chain,
        "layers": layers,
        "roofline": {"bound": "valu", "kernel": "the four layers' convolution launches together",
                     "achieved": achieved / 1e12, "peak": PEAK_VALU_WORD_OPS / 1e12, "unit": "T word-op/s",
                     "frac": achieved / PEAK_VALU_WORD_OPS, "kernel_ms_sum": k_total, "traffic": None},
    }
    return result


def bench_network_inference(args, torch):
    """4-layer SC CNN inference forward at batch 256 (eval mode, running statistics): the fused
    path (one epilogue kernel per layer, 7-bit integer activations between layers) with the
    module-by-module forward (PyTorch element-wise ops between the SC kernels) timed beside it."""
    from geo_amd import network
    from geo_amd import workloads as wl

    L = args.length or 64
    torch.manual_seed(0)
    model = network.CONV_tiny_add_partial().cuda().eval()
    model.err = [L.bit_length() - 1] * 4
    model.load_unit = [2] * 4
    model.load_wait = [2] * 4
    x = torch.rand((256, 3, 32, 32), generator=torch.Generator().manual_seed(0)).cuda()

    def fused():
        return model.forward_fused(x)

    def fused_eager():  # second timing loop: the same forward replayed from a HIP graph
        return model.forward_fused(x, graph=True)

    def modules():
        with torch.no_grad():
            return model(x.clone())

    same = bool(torch.equal(fused(), modules()))
    for _ in range(args.warmup):
        fused()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fused()
    torch.cuda.synchronize()
    ms_fused = (time.perf_counter() - t0) * 1e3 / args.steps
    t0 = time.perf_counter()
    for _ in range(args.steps):
        modules()
    torch.cuda.synchronize()
    ms_modules = (time.perf_counter() - t0) * 1e3 / args.steps
    fused_eager()  # records the graph
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fused_eager()
    torch.cuda.synchronize()
    ms_eager = (time.perf_counter() - t0) * 1e3 / args.steps
    B_total = sum(wl.bit_macs(sx, sw, pad, L) for _, sx, sw, pad in C2_LAYERS)
    # the epilogue kernel of the first layer alone, against the bytes it has to move
    from geo_amd import capi
    counts = torch.randint(-5 * L, 5 * L, (256, 32, 32, 32), dtype=torch.int32, device="cuda")
    wn = torch.rand(32, device="cuda")
    bn = torch.rand(32, device="cuda")
    e = time_events(lambda: capi.layer_epilogue(counts, L, wn, bn, want_act=False, want_q7=True), args.steps, 2, torch)
    e_ms = sum(e) / len(e)
    e_bytes = counts.numel() * 4 + counts.numel() // 4
    print(json.dumps({
        "metric": f"SC bit-MACs/sec over one inference forward of the 4-layer SC CNN at stream len {L}",
        "value": B_total / (ms_fused * 1e-3), "unit": "bit-MAC/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_fused, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32 bit-packed streams, int32 accumulate; u8 activations between layers",
        "data": "synthetic (torch.manual_seed(0); images U[0,1))",
        "config": {"workload": "C2: 4-layer SC CNN inference forward, batch 256, fused layer epilogues, cached weight "
                               "streams, stream "
                               f"length {L}, load_unit 2 / load_wait 2", "pass": "fwd", "bit_macs_per_step": B_total},
        "module_forward_ms": ms_modules, "fused_as_hip_graph_replay_ms": ms_eager, "fused_equals_module_forward": same,
        "roofline": {"bound": "hbm", "kernel": "k_layer_epilogue on (256, 32, 32, 32) counts", "achieved":
                     e_bytes / (e_ms * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
                     "frac": e_bytes / (e_ms * 1e-3) / 8e12, "kernel_ms_avg": e_ms, "algorithmic_bytes": e_bytes,
                     "traffic": None},
    }))


DTYPE_FWD = "u32 bit-packed streams, int32 popcount accumulate"
DTYPE_FWD_BWD = (DTYPE_FWD + " (forward); fp32 gradients: each fp32 product from bf16 MFMA products of a three-way "
                 "operand split, fp32 accumulate (backward)")


def min_word_ops(x_shape, w_shape, pad, L):
    """32-bit VALU lane operations no kernel for this problem can do without: one and-or per (activation
    word, weight) - a weight has a single non-zero rail (sc.cpp:301-304), so B/32 of them, not the 2*B/32
    of a kernel that processes both rails - plus one popcount-add per (output, rail, add group, pack)."""
    N, Cin, Wx, Hx = x_shape
    Cout, _, W, H = w_shape
    Wo, Ho = Wx + 2 * pad - W + 1, Hx + 2 * pad - H + 1
    B = N * Cout * Wo * Ho * Cin * W * H * L
    return B / 32 + 2 * N * Cout * Wo * Ho * H * ((L + 31) // 32)


def measure_layer(torch, workload, L, steps, warmup, with_bwd=True, accumulate="y", z_unit=32, generator="lfsr"):
    """Times one single-layer workload: whole step (wall clock around synchronised loops), forward and
    backward with events, the convolution kernel alone on pre-generated streams, stream generation."""
    from geo_amd import capi
    from geo_amd import workloads as wl

    sx, sw, pad, _, vx, vw = wl.SHAPES[workload]
    x, w = wl.make_inputs(sx, sw, "prescribed", 0, vx, vw)
    xd, wd = x.cuda(), w.cuda()
    desc = capi.make_desc(xd.shape, wd.shape, L, (pad, pad), accumulate=accumulate, z_unit=z_unit,
                          generator=generator, seed=1)
    ws = torch.empty(capi.workspace_size(desc), dtype=torch.uint8, device="cuda")
    out = torch.empty(capi.output_shape(desc), dtype=torch.int32, device="cuda")
    gy = torch.randn(out.shape, generator=torch.Generator().manual_seed(1)).cuda()
    ws_b = torch.empty(capi.backward_workspace_size(desc), dtype=torch.uint8, device="cuda") if with_bwd else None

    def fwd():
        capi.conv2d_add_partial_forward(xd, wd, L, (pad, pad), out=out, workspace=ws, desc=desc)

    def bwd():
        capi.conv2d_add_partial_backward(xd, wd, gy, L, (pad, pad), workspace=ws_b, desc=desc)

    def step():
        fwd()
        if with_bwd:
            bwd()

    # whole step: barrier-free on one GPU, synchronise both sides of the timed region
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    m = {"x": x, "w": w, "pad": pad, "desc": desc, "out_shape": tuple(out.shape)}
    m["ms_per_step"] = (time.perf_counter() - t0) * 1e3 / steps
    m["fwd_ms"] = time_events(fwd, steps, 2, torch)
    m["bwd_ms"] = time_events(bwd, steps, 2, torch) if with_bwd else None
    # dominant kernel alone (AND/OR/popcount on pre-generated streams), events on its stream
    act = capi.act_streams(xd, desc)
    wgt = capi.weight_streams(wd, desc)
    m["kernel_ms"] = time_events(lambda: capi.conv2d_add_partial_from_streams(act, wgt, desc, out=out), steps,
                                 warmup, torch)
    m["gen_ms"] = time_events(lambda: (capi.act_streams(xd, desc), capi.weight_streams(wd, desc)), min(steps, 10),
                              2, torch)
    m["rail"] = capi.skips_zero_rail(desc)
    m["B"] = wl.bit_macs(xd.shape, wd.shape, pad, L)
    m["min_word_ops"] = min_word_ops(xd.shape, wd.shape, pad, L)
    N, Cin, _, _ = xd.shape
    Cout, _, W, H = wd.shape
    m["bwd_flops"] = 12 * N * Cout * out.shape[2] * out.shape[3] * Cin * W * H
    m["alg_bytes"] = 4 * (xd.numel() + wd.numel() + out.numel())
    m["stream_bytes"] = 4 * (act.numel() + wgt.numel())
    m["out_bytes"] = 4 * out.numel()
    return m


def avg(v):
    return sum(v) / len(v)


def config_summary(m):
    """The per-configuration entry of the ``configs`` key."""
    k = avg(m["kernel_ms"])
    e = {"ms_per_step": m["ms_per_step"], "fwd_ms": avg(m["fwd_ms"]),
         "bwd_ms": avg(m["bwd_ms"]) if m["bwd_ms"] else None, "kernel_ms": k,
         "bit_macs_per_s": m["B"] / (m["ms_per_step"] * 1e-3),
         "fwd_bit_macs_per_s": m["B"] / (avg(m["fwd_ms"]) * 1e-3),
         "executed_frac": m["min_word_ops"] / (k * 1e-3) / PEAK_VALU_WORD_OPS,
         "bwd_tflops": m["bwd_flops"] / (avg(m["bwd_ms"]) * 1e-3) / 1e12 if m["bwd_ms"] else None}
    return e


def other_configs(args, torch):
    """The benchmark configurations besides the headline, timed the same way with fewer steps."""
    steps, warmup = min(args.steps, 10), min(args.warmup, 3)
    out = {}
    # the training step first and with the headline's step counts: its steps are three orders of magnitude
    # shorter than the layers' runs that follow
    net_args = argparse.Namespace(**vars(args))
    net_args.length = 64
    r = network_step_result(net_args, torch)
    out["C2_L64_train_step"] = {
        "ms_per_step": r["ms_per_step"], "eager_ms_per_step": r["eager_ms_per_step"],
        "torch_statistics_ms_per_step": r["torch_statistics_ms_per_step"],
        "module_chain_ms_per_step": r["module_chain_ms_per_step"], "workload": r["config"]["workload"],
        "bit_macs_per_s": r["value"], "kernel_ms": r["roofline"]["kernel_ms_sum"],
        "executed_frac": r["roofline"]["frac"],
        "fwd_ms": sum(l["fwd_ms"] for l in r["layers"].values()),
        "bwd_ms": sum(l["bwd_ms"] for l in r["layers"].values()), "bwd_tflops": None}
    torch.cuda.empty_cache()
    for name, workload, L in (("C3_L32", "C3", 32), ("C3_L256", "C3", 256), ("C5_L256", "C5", 256),
                              ("C4_L128", "C4", 128)):
        m = measure_layer(torch, workload, L, steps, warmup)
        out[name] = config_summary(m)
        del m
        torch.cuda.empty_cache()
    return out


def probe_mfma_forward(torch):
    """The headline layer's forward priced on the matrix cores by measurement: 512 position tiles x 384 (stream
    cycle, kernel row) slices = 768 slices per CU of a 128 x 256 x 384 fp4 GEMM tile with threshold and count,
    operands already expanded to one fp4 value per bit.  Times are for that slice count on 256 workgroups."""
    from geo_amd import capi
    wgs, slices = 256, 768
    a, b, _, _ = capi.probe_mfma_operands(2048, 384)   # 54 MB of A tiles (beyond L2), 20 MB of B tiles (inside)
    out = torch.empty((wgs, capi.PROBE_MFMA_ROWS, capi.PROBE_MFMA_COLS), dtype=torch.int32, device="cuda")

    def ms(mode, sixteenths=16):
        capi.probe_mfma_slices(mode, a, b, wgs, 8, sixteenths, out)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        capi.probe_mfma_slices(mode, a, b, wgs, slices, sixteenths, out)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1)

    macs = wgs * slices * capi.PROBE_MFMA_ROWS * capi.PROBE_MFMA_COLS * capi.PROBE_MFMA_K
    t = {"mfma_only_ms": ms(0), "with_lds_fragment_reads_ms": ms(1), "with_threshold_and_count_ms": ms(2)}
    for f in (16, 12, 8, 4):
        t[f"with_{78 * f // 16}_kb_of_operands_loaded_per_slice_ms"] = ms(3, f)
    for f in (16, 12, 8, 4):
        t[f"with_{78 * f // 16}_kb_per_slice_loaded_straight_into_lds_ms"] = ms(4, f)
    return {"probe": "SC forward of C3 (128->128 3x3 at 16x16, batch 256, L 128) as fp4 GEMM slices on the matrix cores",
            "slices_per_cu": slices, "tile": "128 positions x 256 rail-columns x 384 members", "times": t,
            "fp4_tflops_mfma_only": 2 * macs / (t["mfma_only_ms"] * 1e-3) / 1e12,
            "fp4_tflops_with_threshold": 2 * macs / (t["with_threshold_and_count_ms"] * 1e-3) / 1e12,
            "note": "operands arrive expanded to one fp4 value per stream bit; the vector-ALU kernel takes 1.30 ms for "
                    "the same layer from bit-packed streams"}


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
              "(the path shards over the batch with no communication in forward; nothing here uses a second GPU)",
              file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    if args.probe_mfma_forward:
        print(json.dumps(probe_mfma_forward(torch)))
        return
    if args.workload == "C2":
        if args.passes == "fwd":
            bench_network_inference(args, torch)
        else:
            print(json.dumps(network_step_result(args, torch)))
        return
    from geo_amd import capi
    from geo_amd import workloads as wl

    L = args.length or wl.SHAPES[args.workload][3]
    variant = args.accumulate != "y" or args.generator != "lfsr"
    with_bwd = args.passes == "fwdbwd"

    if args.copy_calibration:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    m = measure_layer(torch, args.workload, L, args.steps, args.warmup, with_bwd, args.accumulate, args.z_unit,
                      args.generator)
    x, w, pad = m["x"], m["w"], m["pad"]
    B = m["B"]
    ms_per_step = m["ms_per_step"]
    value = B / (ms_per_step * 1e-3)
    fwd_ms, bwd_ms, k_ms = m["fwd_ms"], m["bwd_ms"], m["kernel_ms"]
    fwd_avg, k_avg = avg(fwd_ms), avg(k_ms)
    bwd_avg = avg(bwd_ms) if with_bwd else None
    rail = m["rail"]
    ops = m["min_word_ops"]
    achieved = ops / (k_avg * 1e-3)
    issued = (B / 32 if rail else 2 * B / 32)
    probe_rate = capi.probe_and_or_rate()
    traffic, traffic_kernel = (None, None) if variant else profiled_traffic(args.workload, L)

    result = {
        "metric": "SC bit-MACs/sec over one layer step ("
                  + ("forward + surrogate backward" if with_bwd else "forward") + f") at stream len {L}",
        "value": value,
        "unit": "bit-MAC/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": DTYPE_FWD_BWD if with_bwd else DTYPE_FWD,
        "data": "synthetic (torch.manual_seed(0); activations U[0,1), weights U[-1,1))",
        "config": {"workload": f"{args.workload}: SC conv2d {tuple(x.shape)} * {tuple(w.shape)} pad {pad}, "
                               f"stream length {L}, " + {
                                   "y": "y-dimension partial binary accumulation", "z": "z-dimension accumulation",
                                   "yz": f"yz accumulation with z_unit {args.z_unit}",
                                   "full": "full OR accumulation"}[args.accumulate]
                               + f", {args.generator} generators",
                   "pass": args.passes, "bit_macs_per_step": B},
        "layer_ms": {"fwd": fwd_avg, "bwd": bwd_avg, "fwd_bit_macs_per_s": B / (fwd_avg * 1e-3),
                     "fwd_median": statistics.median(fwd_ms), "fwd_min": min(fwd_ms),
                     "bwd_median": statistics.median(bwd_ms) if with_bwd else None,
                     "bwd_min": min(bwd_ms) if with_bwd else None},
        "roofline": {
            "bound": "valu",
            "kernel": ("the rail-skipping convolution kernel (v_and_or_b32 on register-indexed accumulators: one "
                       "and-or per activation word and weight; k_conv_fwd_rail_lds where activation words are "
                       "shared through LDS)" if rail else "k_conv_fwd (v_and_or_b32 / v_bcnt_u32_b32, both rails)"),
            # work no kernel can avoid (one and-or per activation word and weight, plus the popcount-adds) per
            # second of the kernel's average launch duration, against lanes x clock
            "achieved": achieved / 1e12,
            "peak": PEAK_VALU_WORD_OPS / 1e12,
            "unit": "T word-op/s",
            "frac": achieved / PEAK_VALU_WORD_OPS,
            "min_word_ops": ops,
            "kernel_ms_avg": k_avg,
            "kernel_ms_min": min(k_ms),
            "measured_issue_rate": probe_rate / 1e12,
            "frac_of_measured_issue_rate": achieved / probe_rate,
            # and-or instructions this kernel issues (lane operations): B/32 when it skips the zero rail, else 2B/32
            "issued_and_or_word_ops": issued,
            # the same time priced with the two-rail count 2*B/32 that a kernel processing both rails would
            # execute (can pass the peak; not a roofline fraction)
            "two_rail_word_ops": 2 * B / 32,
            "two_rail_equivalent_rate": 2 * B / 32 / (k_avg * 1e-3) / 1e12,
            "hbm_algorithmic_bytes": m["alg_bytes"],
            "hbm_stream_bytes_read_by_kernel": m["stream_bytes"],
            "traffic": traffic,
            "traffic_source": (f"static: profiles/traffic.json, rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of "
                               f"{traffic_kernel}, scaled by a device copy of known size; not measured in this run")
                              if traffic else None,
            "hbm_frac_of_peak": (traffic if traffic else m["stream_bytes"] + m["out_bytes"]) / (k_avg * 1e-3)
                                / PEAK_HBM_BYTES,
        },
        "stages_ms": {"stream_generation": avg(m["gen_ms"]), "conv_kernel": k_avg, "backward": bwd_avg},
        "backward_flops": {"algorithmic": m["bwd_flops"],
                           "achieved_tflops": (m["bwd_flops"] / (bwd_avg * 1e-3) / 1e12) if bwd_avg else None,
                           "peak_tflops_fp32_mfma": 157.3,
                           "frac_of_bf16_mfma_peak_as_executed": (6 * m["bwd_flops"] / (bwd_avg * 1e-3) / 2.5e15)
                                                                 if bwd_avg else None,
                           "note": "fp32 in and out; aligned operands form each fp32 product from six bf16 MFMA "
                                   "products of a three-way split (fp32 accumulation, error as an fp32 GEMM), so "
                                   "the fp32 MFMA peak is a yardstick, not a bound; the bf16 fraction counts the six "
                                   "products against 2.5 PFLOP/s"},
    }
    if not args.no_cpu_baseline and not variant:  # the compiled reference has the y / LFSR op only
        kind, cores, sec, note = cpu_baseline(x, w, L, pad)
        result["cpu_baseline"] = {
            "value": B / sec, "unit": "bit-MAC/s", "cores": cores, "kind": kind,
            "sample": f"same workload, forward only (the reference has no native backward), full batch, median of "
                      f"up to 5 runs after 1 warm-up ({sec:.3f} s/run); {note}",
            "gpu_forward_over_cpu_forward": (B / (fwd_avg * 1e-3)) / (B / sec),
        }
    if not args.no_configs and not variant and args.workload == "C3" and L == 128 and with_bwd:
        del m
        torch.cuda.empty_cache()
        result["configs"] = other_configs(args, torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
