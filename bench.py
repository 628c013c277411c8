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
VALU_INSTR_PER_PAIR = 2  # v_ashrrev_i32 + v_xad_u32
PEAK_PAIRS = CU_COUNT * LANES_PER_CU * CLOCK_HZ / VALU_INSTR_PER_PAIR  # 19.66e12 pairs/s
HBM_PEAK = 8.0e12

BATCH = 64
CHW = (3, 224, 224)


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


def parity_gate(model, x):
    """Before any timing: the first 3x3 shift conv of the network on a one-image slice of its real
    input, GPU int32 output against the oracle, bit for bit."""
    from deepshift_amd import kernels, modules
    from oracle import shift_oracle
    oracle = shift_oracle.get()
    layer = [m for m in model.modules() if isinstance(m, modules.Conv2dShift)][1]
    captured = {}
    h = layer.register_forward_hook(lambda mod, inp, out: captured.setdefault("x", inp[0]))
    with torch.no_grad():
        model(x[:2])
    h.remove()
    xin = captured["x"][:1].contiguous()
    xq = kernels.quantize_pad(xin, layer.padding, 16, 16)
    tiled = kernels._tiled_of(layer.conc_weight, layer.out_channels, layer.in_channels, *layer.kernel_size)
    y = kernels.conv2d_tiled(xq, tiled, None, layer.out_channels, layer.kernel_size, layer.stride,
                             layer.conc_weight.bits, layer.conc_weight.base)
    shift = layer.shift.detach().clamp(*layer.shift_range).round().cpu().numpy().astype(np.int32)
    sign = layer.sign.detach().round().sign().cpu().numpy().astype(np.int32)
    want = oracle.conv2d(xq.cpu().numpy(), shift, sign, None, layer.stride,
                         nthreads=min(16, os.cpu_count() or 1))
    if not np.array_equal(y.cpu().numpy(), want):
        raise SystemExit("parity gate failed: GPU shift conv differs from the oracle")


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


def fused_model_timing(device, cls, batch, weight_bits, integer_bits, fraction_bits, workload, steps=5):
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
    x = torch.randn(batch, *CHW, generator=g).to(device)
    with torch.no_grad():
        fused = fuse.fuse_conv_epilogues(model)
    sec = time_steps(fused, x, steps, 2)
    layers = kernel_timings(fused, x, 3)
    pairs = sum(L["M"] * L["K"] * L["N"] for L in layers)
    kernel_s = sum(L["seconds"] for L in layers)
    return dict(workload=workload, ms_per_step=sec * 1e3, images_per_s=batch / sec, shift_layers=len(layers),
                pairs_per_step=pairs, shift_kernel_ms_per_step=kernel_s * 1e3,
                shift_tpairs_per_s=pairs / kernel_s / 1e12,
                frac_of_two_instruction_peak=pairs / kernel_s / PEAK_PAIRS)


def config5(device, steps=5):
    """Benchmark configuration 5: ResNet-50, batch 128, weight_bits 3 (2-bit shift fields), activations
    3.5 (8 bits).  Every convolution has a multiple of 64 channels, so the fused pipeline runs them on
    the int8 kernel (two pixels per register); the FC stays on the int32 kernel."""
    from deepshift_amd import workloads
    return fused_model_timing(device, workloads.ResNet50, 128, 3, 3, 5,
                              "ResNet-50, batch 128 x 3x224x224, weight_bits 3, activations 3.5", steps)


def config4_act8(device, steps=5):
    """The headline network with the reference's 8-bit activation format (`-ab 3 5`, weight_bits 5):
    the 3x3 layers and the stem run on the int8 kernel, the three 1x1 shortcuts and the FC on the
    int32 kernels."""
    from deepshift_amd import workloads
    return fused_model_timing(device, workloads.ResNet18, BATCH, 5, 3, 5,
                              "ResNet-18, batch 64 x 3x224x224, weight_bits 5, activations 3.5", steps)


def pmc_target(device):
    """Counter targets for `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`: a plain copy of 64 MiB (reads
    64 MiB, writes 64 MiB: the scale of the counters) and the dominant shift-kernel launch."""
    from deepshift_amd import _lib, kernels, utils
    g = torch.Generator().manual_seed(0)
    n = 16 * 1024 * 1024
    src = torch.randint(0, 2 ** 20, (n,), generator=g, dtype=torch.int32).to(device)
    dst = torch.empty_like(src)
    x = torch.randint(0, 2 ** 20, (BATCH, 64, 58, 58), generator=g, dtype=torch.int32).to(device)
    shift = torch.randint(-14, 1, (64, 64, 3, 3), generator=g).float()  # the range of weight_bits 5
    sign = (torch.randint(0, 2, (64, 64, 3, 3), generator=g) * 2 - 1).float()
    cw = utils.compress_bits(shift, sign)
    tiled = kernels._tiled_of(cw, 64, 64, 3, 3)
    torch.cuda.synchronize()
    for _ in range(3):
        _lib.call("ds_copy_i32", _lib.ptr(src), _lib.ptr(dst), n, _lib.current_stream(device))
        kernels.conv2d_tiled(x, tiled, None, 64, (3, 3), (1, 1), kernels.kernel_bits(cw), cw.base)
    torch.cuda.synchronize()


def cpu_baseline(shapes):
    """The oracle's restatement of the reference CPU kernel (shift_cpu.cpp loop nests, batch rows /
    images split over threads) on every shift layer of ResNet-18 at a reduced batch."""
    from oracle import shift_oracle
    oracle = shift_oracle.get()
    threads = min(16, os.cpu_count() or 1)
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
        "value": batch / t_multi, "unit": "images/s", "cores": threads, "kind": "port",
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
    ap.add_argument("--pmc-target", action="store_true",
                    help="only launch the counter targets: a 64 MiB copy kernel and the dominant shift "
                         "kernel (ResNet-18 layer1 3x3 conv, batch 64), 3 times each")
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
    if args.config5_only:
        print(json.dumps(config5(device, args.steps)), flush=True)
        return

    from deepshift_amd import workloads
    model, x, n_conv = build_model(device)
    parity_gate(model, x)
    log("parity gate passed; %d conv + 1 fc shift layers" % n_conv)

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
    sec_unfused = time_steps(model, x, max(2, args.steps // 2), args.warmup)
    sec_per_step = time_steps(fused, x, args.steps, args.warmup)
    layers = kernel_timings(fused, x, max(3, min(args.steps, 10)))
    shapes = workloads.shift_layer_shapes(workloads.ResNet18(), CHW, BATCH)
    assert len(layers) == len(shapes) == 21

    pairs = sum(L["M"] * L["K"] * L["N"] for L in layers)
    kernel_s = sum(L["seconds"] for L in layers)
    alg_bytes = 0
    # the fused graph may run the two branches of a block in another order than the module tree:
    # match the timed launches to the traced shapes by their (M, K, N)
    pool = list(shapes)
    for L in layers:
        S = next(c for c in pool if (c["M"], c["K"], c["N"]) == (L["M"], L["K"], L["N"]))
        pool.remove(S)
        uniq = S["Nb"] * S["C"] * S["H"] * S["W"] if S["kind"] == "conv" else None
        L["bytes"] = algorithmic_bytes(L, uniq)
        alg_bytes += L["bytes"]
        L["name"] = S["name"]
    if args.layers:
        for L in layers:
            p = L["M"] * L["K"] * L["N"]
            log("%-22s M=%-7d K=%-5d N=%-5d %8.1f us  %6.2f Tpair/s  %5.1f%% valu  %5.1f%% hbm" % (
                L["name"], L["M"], L["K"], L["N"], L["seconds"] * 1e6, p / L["seconds"] / 1e12,
                100 * p / L["seconds"] / PEAK_PAIRS, 100 * L["bytes"] / L["seconds"] / HBM_PEAK))

    peak_cal = None if args.resnet_only else calibrate_valu(device)
    cfg2 = None if args.resnet_only else config2(device)
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
                               "word), activations 16.16; BatchNorm/residual/ReLU folded into each "
                               "conv's dequantisation pass, pooling fp32 PyTorch",
                   "batch": BATCH, "shift_layers": 21, "pairs_per_step": pairs},
        "unfused_images_per_s": BATCH / sec_unfused,
        "shift_kernel_ms_per_step": kernel_s * 1e3,
        "shift_gops": 2 * pairs / kernel_s / 1e9,
        "shift_layers_images_per_s": BATCH / kernel_s,
        "roofline": {
            "bound": "valu",
            "kernel": "ds::shift_planes_wide_cu_kernel<4> (16 launches) + ds::shift_planes_wide_balanced_kernel<4> "
                      "(1 launch) + ds::shift_kernel (4 launches) per step",
            "achieved": pairs / kernel_s / 1e12,
            "peak": PEAK_PAIRS / 1e12,
            "unit": "Tpair/s",
            "frac": pairs / kernel_s / PEAK_PAIRS,
            # HBM bytes of one launch of the dominant shape (layer1 3x3 conv, 8 of the 21 launches are
            # this size): 109.4 MB read + 67.1 MB written (tiles shared by two workgroups are combined
            # with atomic adds), from the FETCH_SIZE / WRITE_SIZE runs summarised in
            # profiles/shift_kernel_layer1_conv_counters.md (106.6 MB algorithmic)
            "traffic": 176.5e6,
            # vector instructions the dominant kernel issues per pair (SQ_INSTS_VALU, same profile):
            # `peak` prices a pair at 2 instructions, so its fraction can exceed 1
            "valu_instr_per_pair": 1.28,
            # the same lanes x nominal clock priced at the kernel's own instruction count: the ceiling of
            # this kernel design, below 1 by the vector-issue gaps (two scalar instructions per code)
            "peak_at_kernel_mix": PEAK_PAIRS * VALU_INSTR_PER_PAIR / 1.28 / 1e12,
            "frac_at_kernel_mix": pairs / kernel_s / (PEAK_PAIRS * VALU_INSTR_PER_PAIR / 1.28),
            "avg_launch_us": kernel_s / len(layers) * 1e6,
            "peak_calibrated": peak_cal / 1e12 if peak_cal else None,
            "frac_of_calibrated": pairs / kernel_s / peak_cal if peak_cal else None,
            "hbm_achieved_GBps": alg_bytes / kernel_s / 1e9,
            "hbm_frac": alg_bytes / kernel_s / HBM_PEAK,
            "algorithmic_bytes_per_step": alg_bytes,
        },
        "config2": cfg2,
        "config5": cfg5,
        "config4_act8": cfg4_act8,
        "shift_gemm_gops": cfg2["gemm_4096"]["gops"] if cfg2 else None,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(workloads.shift_layer_shapes(workloads.ResNet18(), CHW, 1))
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
