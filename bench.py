#!/usr/bin/env python3
"""Benchmark of the shift-kernel inference path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--layers]

One step = one forward pass of ResNet-18 (every conv and the FC replaced by shift layers,
weight_bits 5, activations 16.16) over one synthetic batch of 64 x 3 x 224 x 224 that is already
resident in HBM.  Prints ONE JSON line: images/s for the whole forward pass, the shift kernel's
rate against the VALU roofline (timed live with HIP events on the launch stream), the 4096^3
shift GEMM and the 3x3 conv of benchmark configuration 2, ResNet-50 (configuration 5) and ResNet-18
with 8-bit activations, and the CPU restatement of the reference's shift kernel timed on this host's cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X nominal figures the roofline is priced against
CU_COUNT = 256
LANES_PER_CU = 64
CLOCK_HZ = 2.4e9
LANE_OPS = CU_COUNT * LANES_PER_CU * CLOCK_HZ  # 39.3e12 int32 lane-operations per second
# The bound: a shift-add pair needs at least ONE vector instruction per lane (the accumulate; the shifted
# operand can be shared between output channels, which is what the shift-plane kernels do), so no int32
# kernel can exceed 39.3 Tpair/s; the int8 kernels hold two pixels per lane register: 0.5 per pair.
PEAK_PAIRS = LANE_OPS / 1.0
PEAK_PAIRS_INT8 = LANE_OPS / 0.5
# secondary figure: a kernel that shifts and accumulates every pair separately (v_ashrrev_i32 + v_xad_u32)
PEAK_PAIRS_TWO_INSTR = LANE_OPS / 2.0
HBM_PEAK = 8.0e12

BATCH = 64
CHW = (3, 224, 224)

# the kernel behind the 3x3 convolutions of the headline network, as rocprofv3 names it
DOMINANT_KERNEL = "ds::shift_planes_wide_coop_kernel<4, 2, true, false>"
# HBM bytes of one launch of that kernel on the layer1 shape: 77.0 MB read + 69.5 MB written (FETCH_SIZE /
# WRITE_SIZE counters scaled by a 64 MiB copy kernel's readings); 106.6 MB are algorithmic, the rest are
# the partial tiles that workgroups exchange through the workspace and what is left of the re-read halo rows
TRAFFIC_LAYER1_BYTES = 146.5e6


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_model(device):
    from deepshift_amd import convert, workloads
    g = torch.Generator().manual_seed(0)
    model = workloads.ResNet18()
    for m in model.modules():
        if isinstance(m, (torch.nn.Conv2d, torch.nn.Linear)):
            torch.nn.init.kaiming_normal_(m.weight, generator=g)
    workloads.randomize_batchnorm(model, g)
    model.eval()
    model, n = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True,
                                        weight_bits=5, act_integer_bits=16, act_fraction_bits=16)
    model = model.to(device)
    convert.round_shift_weights(model)
    x = torch.randn(BATCH, *CHW, generator=g).to(device)
    return model, x, n


def host_threads():
    """Threads for the CPU legs: every core this process may use (os.cpu_count(), capped by the
    OMP_NUM_THREADS the box exports for its CPU share)."""
    n = os.cpu_count() or 1
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", n)))
    except ValueError:
        pass
    return max(1, n)


def _oracle_chain(oracle, so, fused_mod, xq_img, residual_img):
    """What one fused shift convolution must produce for one image, by the oracle: the reference's chain
    conv kernel -> y.float()/2^F (modules.py:161-162) -> eval BatchNorm -> + residual -> ReLU
    [-> max pooling] -> the consumer's round_to_fixed + cast + padding (modules.py:317,153,
    kernels.py:32-36).  Returns (float result, consumer's fixed-point input or None)."""
    from deepshift_amd import modules
    conv = fused_mod.conv
    shift, sign = modules.module_codes(conv)
    bias = None
    if conv.bias is not None:
        bias = oracle.quantize(conv.bias.detach().float().cpu().numpy(), conv.act_integer_bits,
                               conv.act_fraction_bits)
    y = oracle.conv2d(xq_img, shift.cpu().numpy().astype(np.int32), sign.cpu().numpy().astype(np.int32), bias,
                      conv.stride, nthreads=host_threads())
    scale = None if fused_mod.scale is None else fused_mod.scale.cpu().numpy()
    offs = None if fused_mod.shift is None else fused_mod.shift.cpu().numpy()
    v = so.np_dequantize_affine(y, conv.act_fraction_bits, scale, offs, residual_img, fused_mod.relu)
    if fused_mod.pool is not None:
        v = so.np_max_pool2d(v, *fused_mod.pool)
    q = None
    if fused_mod.emit is not None:
        padding, I, Fq = fused_mod.emit[:3]
        q = so.np_requantize(v, I, Fq, tuple(padding))
    return v, q


def _split_result(fused_mod, result):
    """(float result or None, fixed-point result or None) of a fused convolution's return value."""
    if fused_mod.emit is None:
        return result, None
    if fused_mod.emit[3]:
        return result[0], result[1]
    return None, result


def parity_gate(fused, x, images=None):
    """Before any timing: one forward pass of the FUSED model that is about to be timed, with a hook on every
    fused shift-convolution launch it issues (ds_conv2d_tiled_fused_i32, ds_conv2d_tiled_fused_pair_i32, the
    stem's ds_conv2d_tiled_i32 + pooling pass); each launch's own inputs and outputs -- the tensors the
    timed launches read and write -- are then compared, for the first and the last image, bit for bit with
    the oracle's restatement of the reference chain on the same inputs.  Returns the number of launches
    checked."""
    from deepshift_amd import fuse
    from oracle import shift_oracle as so
    oracle = so.get()
    images = list(images) if images is not None else [0, x.shape[0] - 1]
    records = []

    def hook(mod, inp, out):
        records.append((mod, inp, out))   # (a hook's return value would replace the module's output)

    watched = [m for m in fused.modules() if isinstance(m, (fuse.FusedConv2dShift, fuse.FusedShortcutPair))]
    hooks = [m.register_forward_hook(hook) for m in watched]
    with torch.no_grad():
        fused(x)
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()

    def img_of(t, i):
        return None if t is None else t[i:i + 1].cpu().numpy()

    def fixed_input(mod, t, i):
        conv = mod.conv
        if mod.prequantized:
            return t[i:i + 1].cpu().numpy().astype(np.int32)
        return so.np_requantize(t[i:i + 1].float().cpu().numpy(), conv.act_integer_bits, conv.act_fraction_bits,
                                tuple(conv.padding))

    def compare(mod, result, xq_img, res_img, i, what):
        got_f, got_q = _split_result(mod, result)
        want_f, want_q = _oracle_chain(oracle, so, mod, xq_img, res_img)
        if got_f is not None and not np.array_equal(got_f[i:i + 1].cpu().numpy(), want_f):
            raise SystemExit("parity gate failed: %s, image %d: float result differs from the oracle chain" % (what, i))
        if got_q is not None and not np.array_equal(got_q[i:i + 1].cpu().numpy().astype(np.int32), want_q):
            raise SystemExit("parity gate failed: %s, image %d: fixed-point result differs from the oracle chain"
                             % (what, i))

    checked = 0
    for n, (mod, inp, out) in enumerate(records):
        for i in images:
            if isinstance(mod, fuse.FusedShortcutPair):
                xq = inp[0]
                res = [inp[k] if len(inp) > k else None for k in (1, 2)]
                pad = tuple(mod.first.conv.padding)
                xa = xq[i:i + 1].cpu().numpy()
                # the shortcut reads the centre taps: the padded tensor without the first convolution's padding
                xb = xa[:, :, pad[0]:xa.shape[2] - pad[0], pad[1]:xa.shape[3] - pad[1]]
                compare(mod.first, out[0], xa, img_of(res[0], i), i, "launch %d (pair, k x k)" % n)
                compare(mod.shortcut, out[1], np.ascontiguousarray(xb), img_of(res[1], i), i,
                        "launch %d (pair, shortcut)" % n)
            else:
                res = inp[1] if len(inp) > 1 else None
                compare(mod, out, fixed_input(mod, inp[0], i), img_of(res, i), i, "launch %d" % n)
        checked += 1
    return checked


def time_steps(model, x, steps, warmup):
    with torch.no_grad():
        for _ in range(warmup):
            model(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            model(x)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps


def kernel_timings(model, x, steps):
    """Re-runs `steps` forward passes with every shift-kernel launch bracketed by HIP events on
    its launch stream; returns per-layer (kind, M, K, N, mean seconds)."""
    from deepshift_amd import kernels
    sink = []
    kernels.set_timing_sink(sink)
    with torch.no_grad():
        for _ in range(steps):
            model(x)
    torch.cuda.synchronize()
    kernels.set_timing_sink(None)
    per_step = len(sink) // steps
    layers = []
    for i in range(per_step):
        kind, M, K, N = sink[i][:4]
        secs = [sink[s * per_step + i][4].elapsed_time(sink[s * per_step + i][5]) * 1e-3
                for s in range(steps)]
        layers.append(dict(kind=kind, M=M, K=K, N=N, seconds=float(np.mean(secs))))
    return layers


def replay_timing(model, x, select, rounds=20):
    """Average duration of the launches `select` picks out of one forward pass, timed as a run: the pass is
    recorded once (kernels.set_replay_sink: every fused shift convolution hands back a closure that issues
    the same launch again on the same tensors), then `rounds` rounds of the selected launches go to the
    stream back to back between two HIP events.  Unlike an event pair around a single launch, which also
    times the launch's own dispatch (about 10 us), this is the kernel's duration plus the gap to the next
    launch -- what the rocprofv3 kernel trace of the step shows for the same kernel."""
    from deepshift_amd import kernels
    recorded = []
    kernels.set_replay_sink(recorded)
    with torch.no_grad():
        model(x)
    torch.cuda.synchronize()
    kernels.set_replay_sink(None)
    launches = [r[4] for r in recorded if select(dict(kind=r[0], M=r[1], K=r[2], N=r[3]))]
    if not launches:
        return None, 0
    for fn in launches:
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(rounds):
        for fn in launches:
            fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / (rounds * len(launches)), len(launches)


def algorithmic_bytes(layer, unique_input_elems=None):
    """int32 input once + packed words (bits 4: 6 codes per word) + int32 bias + int32 output."""
    comm = (layer["K"] + 5) // 6
    xin = unique_input_elems if unique_input_elems is not None else layer["M"] * layer["K"]
    return 4 * xin + 4 * layer["N"] * comm + 4 * layer["N"] + 4 * layer["M"] * layer["N"]


def calibrate_valu(device):
    from deepshift_amd import _lib
    blocks, iters = 256 * 16, 4000
    sink = torch.empty(blocks * 256, dtype=torch.int32, device=device)
    st = _lib.current_stream(device)
    _lib.call("ds_valu_calibrate", _lib.ptr(sink), blocks, 10, st)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    _lib.call("ds_valu_calibrate", _lib.ptr(sink), blocks, iters, st)
    e1.record()
    torch.cuda.synchronize()
    return blocks * 256 * iters * 64 / (e0.elapsed_time(e1) * 1e-3)


def config2(device, reps=10):
    """Benchmark configuration 2: the 3x3 conv (32x64x56x56, 64 -> 64) and the 4096^3 shift GEMM."""
    from deepshift_amd import kernels, utils
    g = torch.Generator().manual_seed(0)
    out = {}

    def codes(shape):
        return (torch.randint(-15, 1, shape, generator=g).float(),
                (torch.randint(0, 2, shape, generator=g) * 2 - 1).float())

    def timeit(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    x = torch.randn(32, 64, 56, 56, generator=g).clamp_min(0).to(device)
    shift, sign = codes((64, 64, 3, 3))
    cw = utils.compress_bits(shift, sign)
    xq = kernels.quantize_pad(x, (1, 1))
    tiled = kernels._tiled_of(cw, 64, 64, 3, 3)
    t = timeit(lambda: kernels.conv2d_tiled(xq, tiled, None, 64, (3, 3), (1, 1), cw.bits, cw.base))
    pairs = 32 * 56 * 56 * 576 * 64
    out["conv3x3_64x64_32x56x56"] = dict(ms=t * 1e3, gops=2 * pairs / t / 1e9, valu_frac=pairs / t / PEAK_PAIRS)
    # the float multiply-accumulate comparator on the same shape (kernel only, padded input resident)
    from deepshift_amd.unoptimized import kernels as float_kernels
    import torch.nn.functional as F
    wf = torch.randn(64, 64, 3, 3, generator=g).to(device)
    xp = F.pad(x, (1, 1, 1, 1))
    tf = timeit(lambda: float_kernels.conv2d(xp, wf, None, (1, 1), (1, 1)))
    out["conv3x3_64x64_32x56x56"].update(float_multiply_ms=tf * 1e3, shift_over_float_multiply=t / tf)

    x = torch.randn(4096, 4096, generator=g).clamp_min(0).to(device)
    shift, sign = codes((4096, 4096))
    cw = utils.compress_bits(shift, sign)
    xT = kernels.quantize_transpose(x)
    tiled = kernels._tiled_of(cw, 4096, 4096)
    t = timeit(lambda: kernels.linear_tiled(xT, 4096, tiled, None, 4096, cw.bits, cw.base))
    pairs = 4096 ** 3
    out["gemm_4096"] = dict(ms=t * 1e3, gops=2 * pairs / t / 1e9, valu_frac=pairs / t / PEAK_PAIRS)
    wf = torch.randn(4096, 4096, generator=g).to(device)
    tf = timeit(lambda: float_kernels.linear(x, wf, None))  # includes its input transpose
    out["gemm_4096"].update(float_multiply_ms=tf * 1e3, shift_over_float_multiply=t / tf)
    return out


def fused_model_timing(device, cls, batch, weight_bits, integer_bits, fraction_bits, workload, steps=5,
                       chw=CHW, peak=PEAK_PAIRS, graph_replay=False):
    """Steps/s and shift-kernel rate of a converted, fused network on synthetic input."""
    from deepshift_amd import convert, fuse
    g = torch.Generator().manual_seed(0)
    model = cls()
    for m in model.modules():
        if isinstance(m, (torch.nn.Conv2d, torch.nn.Linear)):
            torch.nn.init.kaiming_normal_(m.weight, generator=g)
    from deepshift_amd import workloads
    workloads.randomize_batchnorm(model, g)
    model.eval()
    model, _ = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True,
                                        weight_bits=weight_bits, act_integer_bits=integer_bits,
                                        act_fraction_bits=fraction_bits)
    model = model.to(device)
    convert.round_shift_weights(model)
    x = torch.randn(batch, *chw, generator=g).to(device)
    with torch.no_grad():
        fused = fuse.fuse_conv_epilogues(model)
    sec = time_steps(fused, x, steps, 2)
    layers = kernel_timings(fused, x, 3)
    pairs = sum(L["M"] * L["K"] * L["N"] for L in layers)
    kernel_s = sum(L["seconds"] for L in layers)
    out = dict(workload=workload, ms_per_step=sec * 1e3, images_per_s=batch / sec, shift_layers=len(layers),
               pairs_per_step=pairs, shift_kernel_ms_per_step=kernel_s * 1e3,
               shift_tpairs_per_s=pairs / kernel_s / 1e12,
               valu_bound_tpairs_per_s=peak / 1e12, valu_frac=pairs / kernel_s / peak,
               frac_of_two_instruction_peak=pairs / kernel_s / PEAK_PAIRS_TWO_INSTR)
    if graph_replay:
        out.update(graph_replay_timing(fused, x, steps))
    return out


def graph_replay_timing(fused, x, steps):
    """The step replayed from a captured HIP graph (what the GPU needs for it, with no launch left on the host),
    beside the eager figure.  Every replay is checked against the eager result, with eager steps and
    synchronisations between the replays."""
    try:
        with torch.no_grad():
            want = fused(x).clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(2):
                    fused(x)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                y_graph = fused(x)
            same = True
            for _ in range(3):
                graph.replay()
                torch.cuda.synchronize()
                same = same and bool(torch.equal(y_graph, want))
                same = same and bool(torch.equal(fused(x), want))
                torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                graph.replay()
            torch.cuda.synchronize()
            sec = (time.perf_counter() - t0) / steps
        return dict(ms_per_step_graph_replay=sec * 1e3, graph_replay_equals_eager=same)
    except Exception as exc:  # capture is an extra: the eager figure stands without it
        return dict(ms_per_step_graph_replay=None, graph_replay_error=str(exc)[:200])


def config5(device, steps=5):
    """Benchmark configuration 5: ResNet-50, batch 128, weight_bits 3 (2-bit shift fields), activations
    3.5 (8 bits).  Every convolution has a multiple of 64 channels, so the fused pipeline runs them on
    the int8 kernel (two pixels per register); the FC stays on the int32 kernel."""
    from deepshift_amd import workloads
    return fused_model_timing(device, workloads.ResNet50, 128, 3, 3, 5,
                              "ResNet-50, batch 128 x 3x224x224, weight_bits 3, activations 3.5", steps,
                              peak=PEAK_PAIRS_INT8)


def config4_act8(device, steps=5):
    """The headline network with the reference's 8-bit activation format (`-ab 3 5`, weight_bits 5):
    the 3x3 layers and the stem run on the int8 kernel, the three 1x1 shortcuts and the FC on the
    int32 kernels."""
    from deepshift_amd import workloads
    return fused_model_timing(device, workloads.ResNet18, BATCH, 5, 3, 5,
                              "ResNet-18, batch 64 x 3x224x224, weight_bits 5, activations 3.5", steps,
                              peak=PEAK_PAIRS_INT8)


def config3(device, steps=10):
    """Benchmark configuration 3: ResNet-20 (CIFAR topology, 19 convolutions + FC), batch 256 x 3x32x32,
    weight_bits 5, activations 16.16."""
    from deepshift_amd import workloads
    return fused_model_timing(device, workloads.ResNet20, 256, 5, 16, 16,
                              "ResNet-20, batch 256 x 3x32x32, weight_bits 5, activations 16.16", steps,
                              chw=(3, 32, 32), graph_replay=True)


def config1(device, with_cpu=True, reps=50):
    """Benchmark configuration 1: the 784-512-512-10 LinearShift MLP at batch 64, ternary signs, shifts in
    [-15, 0], 16.16 -- microseconds per forward on the GPU, and the same network on this host through the
    oracle's restatement of the reference's CPU kernel (the path the reference runs this model on,
    mnist.py:213 with --no-cuda) and through the library's own host kernel (use_cuda=False)."""
    from deepshift_amd import convert, modules, workloads
    g = torch.Generator().manual_seed(0)
    x = torch.rand(64, 784, generator=g)

    def build(use_cuda):
        gg = torch.Generator().manual_seed(1)
        model, _ = convert.convert_to_shift(workloads.MLP(), 0, 'PS', convert_weights=False, use_kernel=True,
                                            use_cuda=use_cuda, weight_bits=6)
        for layer in model.layers:
            layer.sign.data = torch.randint(-1, 2, layer.sign.shape, generator=gg).float()
            layer.shift.data = torch.randint(-15, 1, layer.shift.shape, generator=gg).float()
            layer.bias.data = torch.randn(layer.bias.shape, generator=gg) * 0.01
        return model.eval()

    from deepshift_amd import fuse
    plain_model = build(True).to(device)
    xd = x.to(device)
    with torch.no_grad():
        gpu_model = fuse.fuse_conv_epilogues(plain_model)  # each layer and its ReLU: one launch
        for _ in range(5):
            plain_model(xd)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            plain_model(xd)
        torch.cuda.synchronize()
        plain_s = (time.perf_counter() - t0) / reps
        for _ in range(5):
            y_gpu = gpu_model(xd)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            gpu_model(xd)
        torch.cuda.synchronize()
        gpu_s = (time.perf_counter() - t0) / reps
    layers = kernel_timings(gpu_model, xd, 5)
    # the three layers as ONE launch (ds_linear_chain_f32: a persistent grid with barriers between the layers),
    # which the fused model does not choose for layers this wide: timed for the record, checked against it
    one_launch_s, one_launch_same = None, None
    chains = [m for m in gpu_model.modules() if isinstance(m, fuse.FusedLinearChain)]
    if chains:
        chains[0].force = True
        with torch.no_grad():
            for _ in range(5):
                y_one = gpu_model(xd)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                gpu_model(xd)
            torch.cuda.synchronize()
            one_launch_s = (time.perf_counter() - t0) / reps
        one_launch_same = bool(torch.equal(y_one, y_gpu)) and chains[0].status() == 0
        chains[0].force = False
    out = {"workload": "MLP 784-512-512-10, batch 64, ternary signs, shifts [-15, 0] (converted with weight_bits 6 so "
                       "that -15 survives the clamp; 6-bit reference words because of the zero code), activations "
                       "16.16; each layer and its ReLU one launch (ds_linear_small_f32)",
           "us_per_forward": gpu_s * 1e6, "us_per_forward_unfused": plain_s * 1e6,
           "shift_launches_per_forward": len(layers),
           "us_per_forward_one_launch": None if one_launch_s is None else one_launch_s * 1e6,
           "one_launch_equals_three": one_launch_same,
           "shift_kernel_us_per_forward": sum(L["seconds"] for L in layers) * 1e6,
           "pairs_per_forward": sum(64 * l.in_features * l.out_features for l in plain_model.layers)}
    # The eager forward is bound by the host's five launches; the same forward replayed from a captured HIP
    # graph shows what the GPU needs for it (replays are checked against the eager result).
    try:
        side = torch.cuda.Stream(device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.no_grad(), torch.cuda.stream(side):
            for _ in range(3):
                gpu_model(xd)
        torch.cuda.current_stream(device).wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(graph):
            y_graph = gpu_model(xd)
        same = True
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            same = same and bool(torch.equal(y_graph, y_gpu))
        t0 = time.perf_counter()
        for _ in range(reps):
            graph.replay()
        torch.cuda.synchronize()
        out["us_per_forward_graph_replay"] = (time.perf_counter() - t0) / reps * 1e6
        out["graph_replay_equals_eager"] = same
    except Exception as exc:  # capture is an extra: the eager figure stands without it
        out["us_per_forward_graph_replay"] = None
        out["graph_replay_error"] = str(exc)[:200]
    if with_cpu:
        from oracle import shift_oracle
        oracle = shift_oracle.get()
        threads = host_threads()
        cpu_model = build(False)
        codes = [(modules.module_codes(l), l.bias.detach().numpy()) for l in cpu_model.layers]

        def oracle_forward(nthreads):
            h = x.numpy()
            for i, ((shift, sign), bias) in enumerate(codes):
                y = oracle.linear(oracle.cast(h, 16), shift.numpy().astype(np.int8), sign.numpy().astype(np.int32),
                                  oracle.cast(bias, 16), nthreads)
                h = y.astype(np.float32) / np.float32(65536.0)
                if i < 2:
                    h = np.maximum(h, 0)
            return h

        want = oracle_forward(threads)
        identical = bool(np.array_equal(y_gpu.cpu().numpy(), want))
        t0 = time.perf_counter()
        for _ in range(5):
            oracle_forward(threads)
        t_multi = (time.perf_counter() - t0) / 5
        t0 = time.perf_counter()
        oracle_forward(1)
        t_single = time.perf_counter() - t0
        with torch.no_grad():
            host = cpu_model(x)
            t0 = time.perf_counter()
            for _ in range(5):
                cpu_model(x)
            t_twin = (time.perf_counter() - t0) / 5
        out["cpu"] = {"kind": "port", "cores": threads, "us_per_forward": t_multi * 1e6,
                      "single_thread_us_per_forward": t_single * 1e6, "gpu_equals_cpu_bit_for_bit": identical,
                      "host_twin_us_per_forward": t_twin * 1e6,
                      "host_twin_equals_gpu": bool(torch.equal(host, y_gpu.cpu()))}
        if not identical:
            raise SystemExit("configuration 1: the GPU forward differs from the oracle chain")
    return out


def pmc_target(device):
    """Counter targets for `rocprofv3 --pmc`: a plain copy of 64 MiB (reads 64 MiB, writes 64 MiB: the scale
    of the byte counters), then one launch each of the kernels of the headline step, three times over:
      * the dominant kernel on the layer1 shape (3x3, 64 -> 64, batch 64, 56x56), with the fused epilogue
        (shift_planes_wide_coop_kernel<4, 2, true, false>) and with the plain int32 output (<.., false, false>);
      * the stem (7x7 stride 2, 3 -> 64, 224x224): shift_planes_wide_coop_kernel<4, 1, false, false>, whole
        tiles one per wave (K = 147 leaves a partial last group: the zero-top form runs its padding codes);
      * a down-sampling block's first 3x3 stride-2 convolution with its 1x1 shortcut as one launch
        (<4, 2, true, true>), 64 -> 128 channels at 56x56;
      * the int8 kernel's fused launch (shift_pairs_fused_kernel<2, true, false>: eight-wave workgroups,
        BatchNorm affine, ReLU and the next 1x1 layer's int8 input from the epilogue) on a ResNet-50 3x3 layer,
        128 -> 128 at 28x28, batch 128, weight_bits 3;
      * the cooperative two-instruction kernel (shift_coop_kernel) on ResNet-20's 3x3 layers at batch 256:
        16 -> 16 channels at 32x32 (<4, 4, 16, 4, true>) and 32 -> 32 at 16x16 (<4, 2, 32, 8, true>), both with
        residual, ReLU, float and fixed-point outputs."""
    from deepshift_amd import _lib, kernels, utils
    g = torch.Generator().manual_seed(0)
    n = 16 * 1024 * 1024
    src = torch.randint(0, 2 ** 20, (n,), generator=g, dtype=torch.int32).to(device)
    dst = torch.empty_like(src)

    def layer(O, C, F, lo=-14):
        shift = torch.randint(lo, 1, (O, C, F, F), generator=g).float()  # the range the weight_bits clamp leaves
        sign = (torch.randint(0, 2, (O, C, F, F), generator=g) * 2 - 1).float()
        cw = utils.compress_bits(shift, sign)
        return cw, kernels._tiled_of(cw, O, C, F, F), kernels.kernel_bits(cw)

    x1 = torch.randint(0, 2 ** 20, (BATCH, 64, 58, 58), generator=g, dtype=torch.int32).to(device)
    cw1, tiled1, kb1 = layer(64, 64, 3)
    scale = torch.rand(64, generator=g).to(device) * 2.0 ** -6
    offs = torch.randn(64, generator=g).to(device)
    xs = torch.randint(-2 ** 17, 2 ** 17, (BATCH, 3, 230, 230), generator=g, dtype=torch.int32).to(device)
    cws, tileds, kbs = layer(64, 3, 7)
    cwa, tileda, kba = layer(128, 64, 3)
    cwb, tiledb, kbb = layer(128, 64, 1)
    scale2 = torch.rand(128, generator=g).to(device) * 2.0 ** -6
    offs2 = torch.randn(128, generator=g).to(device)
    x8 = torch.randint(0, 97, (128, 128, 30, 30), generator=g, dtype=torch.int32).to(torch.int8).to(device)
    cw8, _, _ = layer(128, 128, 3, lo=-2)
    fields = kernels.paired_fields(cw8, 128, 3, 5)
    blob8 = kernels._paired_of(cw8, fields, 128, 128, 3, 3)
    narrow = []
    for ch, size in ((16, 32), (32, 16)):
        xn = torch.randint(0, 2 ** 20, (256, ch, size + 2, size + 2), generator=g, dtype=torch.int32).to(device)
        cwn, tiledn, kbn = layer(ch, ch, 3)
        narrow.append((xn, tiledn, kbn, ch, torch.rand(ch, generator=g).to(device) * 2.0 ** -6,
                       torch.randn(ch, generator=g).to(device),
                       torch.randn(256, ch, size, size, generator=g).to(device), {}))
    cache, cache2, cache8 = {}, {}, {}
    torch.cuda.synchronize()
    for _ in range(3):
        _lib.call("ds_copy_i32", _lib.ptr(src), _lib.ptr(dst), n, _lib.current_stream(device))
        # as the fused pipeline issues it between two convolutions of a block: BatchNorm affine, ReLU and
        # the next layer's padded fixed-point input from the kernel's epilogue ...
        kernels.conv2d_tiled_fused(x1, tiled1, None, 64, (3, 3), (1, 1), kb1, 16, scale, offs, None, True,
                                   ((1, 1), 16, 16, torch.int32), False, cache)
        # ... and with the plain int32 output of ds_conv2d_tiled_i32
        kernels.conv2d_tiled(x1, tiled1, None, 64, (3, 3), (1, 1), kb1, cw1.base)
        kernels.conv2d_tiled(xs, tileds, None, 64, (7, 7), (2, 2), kbs, cws.base)
        kernels.conv2d_tiled_fused_pair(
            x1, (2, 2), 16,
            dict(tiled=tileda, O=128, kernel_size=(3, 3), crop=(0, 0), bits=kba, scale=scale2, shift=offs2, relu=True,
                 emit=((1, 1), 16, 16, torch.int32), want_float=False, q_cache=cache2),
            dict(tiled=tiledb, O=128, kernel_size=(1, 1), crop=(1, 1), bits=kbb, scale=scale2, shift=offs2,
                 want_float=True))
        kernels.conv2d_paired_fused(x8, blob8, None, 128, (3, 3), (1, 1), fields[1], 96, 5, scale2, offs2, None, True,
                                    ((0, 0), 3, 5, torch.int8), False, cache8)
        for xn, tiledn, kbn, ch, sc, of, res, qc in narrow:
            kernels.conv2d_tiled_fused(xn, tiledn, None, ch, (3, 3), (1, 1), kbn, 16, sc, of, res, True,
                                       ((1, 1), 16, 16, torch.int32), True, qc)
    torch.cuda.synchronize()


def pmc_target_other(device):
    """Counter targets for `rocprofv3 --pmc`, the launches below the 3x3 layers of the headline step: the
    64 MiB copy (scale of the byte counters), then, three times over,
      * benchmark configuration 2's convolution (3x3, 64 -> 64, 56x56, batch 32: 784 tiles on 512
        workgroups) through ds_conv2d_tiled_i32;
      * its 4096^3 shift GEMM through ds_linear_tiled_i32 (one tile per wave + transpose of the
        channel-major scratch);
      * the int8 kernel's fused launch (ds_conv2d_paired_fused_i8: BatchNorm affine, ReLU and the next layer's
        padded int8 input from the epilogue) on ResNet-50's 1x1 convolutions with K = 256 (256 -> 64 at 56x56
        and 256 -> 128 at 28x28, both at batch 128, weight_bits 3, activations in [0, 96]) and on a block end
        of its first stage (64 -> 256 at 56x56: residual in, float result and unpadded int8 input out);
      * the one-launch LinearShift kernel (ds_linear_small_f32) on the three layers of the MNIST MLP at
        batch 64 and on ResNet-18's classifier (64 x 512 x 1000)."""
    from deepshift_amd import _lib, kernels, utils
    g = torch.Generator().manual_seed(0)
    n = 16 * 1024 * 1024
    src = torch.randint(0, 2 ** 20, (n,), generator=g, dtype=torch.int32).to(device)
    dst = torch.empty_like(src)

    def codes(shape, lo=-14):
        shift = torch.randint(lo, 1, shape, generator=g).float()
        sign = (torch.randint(0, 2, shape, generator=g) * 2 - 1).float()
        return utils.compress_bits(shift, sign)

    x2 = torch.randint(0, 2 ** 20, (32, 64, 58, 58), generator=g, dtype=torch.int32).to(device)
    cw2 = codes((64, 64, 3, 3), lo=-15)
    tiled2 = kernels._tiled_of(cw2, 64, 64, 3, 3)
    xg = torch.randn(4096, 4096, generator=g).clamp_min(0).to(device)
    cwg = codes((4096, 4096), lo=-15)
    xT = kernels.quantize_transpose(xg)
    tiledg = kernels._tiled_of(cwg, 4096, 4096)
    int8 = []
    for (C, H, O, block_end) in ((256, 56, 64, False), (256, 28, 128, False), (64, 56, 256, True)):
        x8 = torch.randint(0, 97, (128, C, H, H), generator=g, dtype=torch.int32).to(torch.int8).to(device)
        cw8 = codes((O, C, 1, 1), lo=-2)
        fields = kernels.paired_fields(cw8, O, 3, 5)
        res8 = torch.randn(128, O, H, H, generator=g).to(device) if block_end else None
        int8.append((x8, kernels._paired_of(cw8, fields, O, C, 1, 1), O, fields[1],
                     (torch.rand(O, generator=g) * 2.0 ** -5).to(device), torch.randn(O, generator=g).to(device), {},
                     res8))
    small = []
    for (M, K, N) in ((64, 784, 512), (64, 512, 512), (64, 512, 10), (64, 512, 1000)):
        cws = codes((N, K))
        small.append((torch.rand(M, K, generator=g).to(device), kernels._tiled_of(cws, N, K), N,
                      kernels.kernel_bits(cws)))
    torch.cuda.synchronize()
    for _ in range(3):
        _lib.call("ds_copy_i32", _lib.ptr(src), _lib.ptr(dst), n, _lib.current_stream(device))
        kernels.conv2d_tiled(x2, tiled2, None, 64, (3, 3), (1, 1), cw2.bits, cw2.base)
        kernels.linear_tiled(xT, 4096, tiledg, None, 4096, cwg.bits, cwg.base)
        for x8, blob8, O, fb, sc8, of8, cache8, res8 in int8:
            kernels.conv2d_paired_fused(x8, blob8, None, O, (1, 1), (1, 1), fb, 96, 5, sc8, of8, res8, True,
                                        ((1, 1) if res8 is None else (0, 0), 3, 5, torch.int8), res8 is not None,
                                        cache8)
        for xs, tileds, N, kb in small:
            kernels.linear_small(xs, tileds, None, N, kb, 0, 16, 16, False, True)
    torch.cuda.synchronize()


def cpu_baseline(shapes):
    """The oracle's restatement of the reference CPU kernel (shift_cpu.cpp loop nests, batch rows /
    images split over threads) on every shift layer of ResNet-18 at a reduced batch."""
    from oracle import shift_oracle
    oracle = shift_oracle.get()
    threads = host_threads()
    batch = threads
    rng = np.random.default_rng(0)

    def run(nthreads, nb):
        total = 0.0
        for L in shapes:
            if L["kind"] == "conv":
                ph, pw = L["padding"]
                xp = rng.integers(0, 2 ** 20, size=(nb, L["C"], L["H"] + 2 * ph, L["W"] + 2 * pw)).astype(np.int32)
                s = rng.integers(-15, 1, size=(L["O"], L["C"], L["FH"], L["FW"])).astype(np.int8)
                sg = rng.choice(np.array([-1, 1], np.int32), size=s.shape)
                t0 = time.perf_counter()
                oracle.conv2d(xp, s, sg, None, L["stride"], nthreads=nthreads)
                total += time.perf_counter() - t0
            else:
                xr = rng.integers(0, 2 ** 20, size=(nb, L["K"])).astype(np.int32)
                s = rng.integers(-15, 1, size=(L["N"], L["K"])).astype(np.int8)
                sg = rng.choice(np.array([-1, 1], np.int32), size=s.shape)
                t0 = time.perf_counter()
                oracle.linear(xr, s, sg, None, nthreads)
                total += time.perf_counter() - t0
        return total

    t_multi = run(threads, batch)
    t_single = run(1, 1)

    # The reference's own CPU kernel (oracle/_ref, compiled from its shift_cpu.cpp) on one layer, beside
    # the port on the same data: it confirms that the port is a fair stand-in.  Its time includes the
    # pybind conversion of nested Python lists, which is how the reference calls it.
    check = None
    ref = shift_oracle.load_reference_cpu_kernel()
    if ref is not None:
        x = rng.integers(0, 2 ** 20, size=(1, 64, 58, 58)).astype(np.int32)
        s = rng.integers(-15, 1, size=(64, 64, 3, 3)).astype(np.int32)
        sg = rng.choice(np.array([-1, 1], np.int32), size=s.shape)
        lists = (x.tolist(), s.tolist(), sg.tolist(), [0] * 64)
        t0 = time.perf_counter()
        y_ref = ref.convolution_kernel(*lists, (1, 1), (0, 0))
        t_ref = time.perf_counter() - t0
        t0 = time.perf_counter()
        y_port = oracle.conv2d(x, s.astype(np.int8), sg, None, (1, 1), nthreads=1)
        t_port = time.perf_counter() - t0
        check = {"layer": "3x3 conv 64->64, 56x56, batch 1 (one thread)", "reference_s": t_ref, "port_s": t_port,
                 "identical": bool(np.array_equal(np.array(y_ref, np.int64).astype(np.int32), y_port))}
    return {
        "reference_kernel_check": check,
        "value": batch / t_multi, "unit": "images/s", "cores": threads, "host_cpu_count": os.cpu_count(),
        "kind": "port",
        "sample": "all 21 shift layers of ResNet-18 at batch %d (one image per thread), kernel time "
                  "only, int32 inputs resident in host memory; single thread on 1 image: %.3f images/s"
                  % (batch, 1.0 / t_single),
        "single_thread_value": 1.0 / t_single,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--layers", action="store_true", help="per-layer table on stderr")
    ap.add_argument("--resnet-only", action="store_true",
                    help="skip config 2 and the VALU calibration (clean kernel-trace profiles)")
    ap.add_argument("--config5-only", action="store_true",
                    help="only benchmark configuration 5 (ResNet-50, 8-bit activations); prints its JSON object")
    ap.add_argument("--config1-only", action="store_true",
                    help="only benchmark configuration 1 (the MNIST MLP, batch 64); prints its JSON object")
    ap.add_argument("--config3-only", action="store_true",
                    help="only benchmark configuration 3 (ResNet-20, batch 256); prints its JSON object")
    ap.add_argument("--pmc-target", action="store_true",
                    help="only launch the counter targets: a 64 MiB copy kernel and the dominant shift "
                         "kernel (ResNet-18 layer1 3x3 conv, batch 64), 3 times each")
    ap.add_argument("--pmc-target-other", action="store_true",
                    help="only launch the second set of counter targets: configuration 2's convolution and "
                         "GEMM, int8 1x1 launches with K = 256, the one-launch linear kernel")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path "
                         "(the workload shards over batch rows with no communication); use --gpus 1")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a ROCm GPU")
    device = torch.device("cuda:0")

    if args.pmc_target:
        pmc_target(device)
        return
    if args.pmc_target_other:
        pmc_target_other(device)
        return
    if args.config5_only:
        print(json.dumps(config5(device, args.steps)), flush=True)
        return
    if args.config3_only:
        print(json.dumps(config3(device, args.steps)), flush=True)
        return
    if args.config1_only:
        print(json.dumps(config1(device, with_cpu=not args.no_cpu)), flush=True)
        return

    from deepshift_amd import workloads
    model, x, n_conv = build_model(device)
    # The measured pipeline: the converted model with the fp32 glue after every shift conv
    # (BatchNorm, residual add, ReLU) folded into that conv's dequantisation pass.  The shift
    # kernels and their int32 results are the same as in the plain converted model, which is timed
    # as well for reference.
    from deepshift_amd import fuse
    with torch.no_grad():
        fused = fuse.fuse_conv_epilogues(model)
        want, got = model(x[:4]), fused(x[:4])
    if not torch.allclose(got, want, rtol=0, atol=2e-3 * float(want.abs().max()) + 1e-4):
        raise SystemExit("fused pipeline diverges from the plain converted model")
    checked = parity_gate(fused, x)
    log("parity gate passed on the %d convolution launches of the timed model; %d conv + 1 fc shift layers"
        % (checked, n_conv))
    sec_unfused = time_steps(model, x, max(2, args.steps // 2), args.warmup)
    sec_per_step = time_steps(fused, x, args.steps, args.warmup)
    layers = kernel_timings(fused, x, max(3, min(args.steps, 10)))
    shapes = workloads.shift_layer_shapes(workloads.ResNet18(), CHW, BATCH)
    assert len(shapes) == 21

    pairs = sum(L["M"] * L["K"] * L["N"] for L in layers)
    assert pairs == sum(S["M"] * S["K"] * S["N"] for S in shapes)
    kernel_s = sum(L["seconds"] for L in layers)
    alg_bytes = 0

    def shape_bytes(S):
        uniq = S["Nb"] * S["C"] * S["H"] * S["W"] if S["kind"] == "conv" else None
        return algorithmic_bytes(S, uniq)

    # The fused graph may run the two branches of a block in another order than the module tree, and it
    # runs a down-sampling block's first convolution and its 1x1 shortcut as ONE launch (timed with the
    # pairs of both): match the timed launches to the traced shapes by their (M, K, N).
    pool = list(shapes)
    for L in layers:
        S = next((c for c in pool if (c["M"], c["K"], c["N"]) == (L["M"], L["K"], L["N"])), None)
        if S is not None:
            pool.remove(S)
            L["bytes"], L["name"] = shape_bytes(S), S["name"]
        else:
            A = next(c for c in pool if (c["M"], c["N"]) == (L["M"], L["N"]) and c["K"] < L["K"] and c["kind"] == "conv"
                     and c["FH"] > 1)
            B = next(c for c in pool if c["M"] == L["M"] and c["kind"] == "conv" and c["FH"] == 1
                     and A["K"] + c["K"] * c["N"] // A["N"] == L["K"])
            pool.remove(A)
            pool.remove(B)
            # the shortcut reads the same input tensor: its bytes are the weights and the second output
            L["bytes"] = shape_bytes(A) + shape_bytes(B) - 4 * B["Nb"] * B["C"] * B["H"] * B["W"]
            L["name"] = A["name"] + " + " + B["name"].split(".")[-2]
        alg_bytes += L["bytes"]
    assert not pool
    if args.layers:
        for L in layers:
            p = L["M"] * L["K"] * L["N"]
            log("%-32s M=%-7d K=%-5d N=%-5d %8.1f us  %6.2f Tpair/s  %5.1f%% valu  %5.1f%% hbm" % (
                L["name"], L["M"], L["K"], L["N"], L["seconds"] * 1e6, p / L["seconds"] / 1e12,
                100 * p / L["seconds"] / PEAK_PAIRS, 100 * L["bytes"] / L["seconds"] / HBM_PEAK))

    # The dominant kernel: the launches of the 3x3 convolutions (16 of the 21, 92 % of the pairs) all run
    # the same kernel; its roofline figures come from their HIP-event durations.
    is_dominant = lambda L: L["kind"] == "conv" and L["K"] % 9 == 0 and L["K"] >= 576
    dominant = [L for L in layers if is_dominant(L)]
    dom_pairs = sum(L["M"] * L["K"] * L["N"] for L in dominant)
    # their average duration: as a run of back-to-back launches (the figure the kernel trace agrees with) ...
    run_avg_s, run_n = replay_timing(fused, x, is_dominant)
    assert run_n == len(dominant), "the replayed launches are not the step's dominant launches"
    dom_s = run_avg_s * len(dominant)
    # ... and from an event pair around each launch inside the step, which also times the dispatch
    dom_s_bracketed = sum(L["seconds"] for L in dominant)
    dom_bytes = sum(L["bytes"] for L in dominant)

    peak_cal = None if args.resnet_only else calibrate_valu(device)
    cfg1 = None if args.resnet_only else config1(device, with_cpu=not args.no_cpu)
    cfg2 = None if args.resnet_only else config2(device)
    cfg3 = None if args.resnet_only else config3(device)
    cfg5 = None if args.resnet_only else config5(device)
    cfg4_act8 = None if args.resnet_only else config4_act8(device)
    result = {
        "metric": "resnet18_bs64_images_per_s",
        "value": BATCH / sec_per_step,
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec_per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int32",
        "data": "synthetic",
        "config": {"workload": "ResNet-18, batch 64 x 3x224x224, all 20 conv + FC as shift layers "
                               "(benchmark configuration 4); weight_bits 5 (4-bit shift + sign, 6 codes per "
                               "word), activations 16.16; BatchNorm, residual, ReLU and the next layer's "
                               "fixed-point conversion in each convolution's epilogue, the stem's max "
                               "pooling in one conversion pass, global average pooling fp32 PyTorch",
                   "batch": BATCH, "shift_layers": 21, "shift_launches": len(layers), "pairs_per_step": pairs},
        "unfused_images_per_s": BATCH / sec_unfused,
        # the same step replayed from a captured HIP graph: an extra beside `value`, which is the eager step
        **graph_replay_timing(fused, x, args.steps),
        "shift_kernel_ms_per_step": kernel_s * 1e3,
        "shift_gops": 2 * pairs / kernel_s / 1e9,
        "shift_layers_images_per_s": BATCH / kernel_s,
        "roofline": {
            # Bound: vector ALU.  peak = 256 CUs x 64 lanes x 2.4 GHz / 1 vector instruction per pair (the
            # accumulate; no int32 kernel can need fewer) = 39.3 Tpair/s.  achieved = the pairs of the
            # dominant kernel's launches / their duration in this run, timed with HIP events around runs of
            # those launches (replay_timing); avg_launch_us_in_step: an event pair around each one.
            "bound": "valu",
            "kernel": DOMINANT_KERNEL,
            "launches_per_step": len(dominant),
            "achieved": dom_pairs / dom_s / 1e12,
            "peak": PEAK_PAIRS / 1e12,
            "unit": "Tpair/s",
            "frac": dom_pairs / dom_s / PEAK_PAIRS,
            "avg_launch_us": dom_s / len(dominant) * 1e6,
            "avg_launch_us_in_step": dom_s_bracketed / len(dominant) * 1e6,
            "frac_in_step": dom_pairs / dom_s_bracketed / PEAK_PAIRS,
            "pairs_per_launch": dom_pairs / len(dominant),
            # HBM bytes of one launch of the dominant kernel on the layer1 shape (M = 200704, K = 576,
            # N = 64; 106.6 MB algorithmic), a constant copied from the FETCH_SIZE / WRITE_SIZE runs in
            # profiles/shift_kernel_layer1_conv_counters.md -- not measured in this run
            "traffic": TRAFFIC_LAYER1_BYTES,
            "traffic_source": "profiles/shift_kernel_layer1_conv_counters.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)",
            # the whole step (all 21 launches, pre-fill passes included) against the same bound
            "step_achieved": pairs / kernel_s / 1e12,
            "step_frac": pairs / kernel_s / PEAK_PAIRS,
            # secondary: against a kernel that spends two vector instructions on every pair
            "peak_two_instruction": PEAK_PAIRS_TWO_INSTR / 1e12,
            "frac_of_two_instruction_peak": dom_pairs / dom_s / PEAK_PAIRS_TWO_INSTR,
            "peak_two_instruction_calibrated": peak_cal / 1e12 if peak_cal else None,
            "hbm_achieved_GBps": dom_bytes / dom_s / 1e9,
            "hbm_frac": dom_bytes / dom_s / HBM_PEAK,
            "algorithmic_bytes_per_step": alg_bytes,
        },
        "config1": cfg1,
        "config2": cfg2,
        "config3": cfg3,
        "config5": cfg5,
        "config4_act8": cfg4_act8,
        "shift_gemm_gops": cfg2["gemm_4096"]["gops"] if cfg2 else None,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(workloads.shift_layer_shapes(workloads.ResNet18(), CHW, 1))
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
