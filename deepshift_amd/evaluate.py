"""Evaluation harness in the style of the reference's ``mnist.py -e`` / ``imagenet.py -e``
(mnist.py:94-150,213; imagenet.py:240-250) for machines without the datasets:

    python -m deepshift_amd.evaluate -e --arch resnet18 --shift-depth 1000 --use-kernel True
    python -m deepshift_amd.evaluate -e --arch mlp --batch-size 64 -wb 5 -ab 16 16 --use-kernel True
    python -m deepshift_amd.evaluate -e --arch resnet20 --use-kernel True --shift-depth 0   # float comparator

The model is built with random initial weights (or ``--weights state_dict.pt``), converted with
``convert_to_shift`` exactly as the reference scripts do, and run on synthetic inputs (or
``--data file.pt`` holding ``{"input": float [N,C,H,W] or [N,784], "target": int64 [N]}``).  It
reports the time per batch on the kernel path, the agreement of the kernel path with the float
shift path of the same converted model and, when targets are given, top-1 accuracy.  Training is not
part of this build.
"""
import argparse
import json
import sys
import time

import torch

from . import convert, export, fuse, workloads
from .unoptimized import convert_to_unoptimized

ARCHS = {
    "mlp": (workloads.MLP, (784,)),
    "resnet18": (workloads.ResNet18, (3, 224, 224)),
    "resnet20": (workloads.ResNet20, (3, 32, 32)),
    "resnet50": (workloads.ResNet50, (3, 224, 224)),
}


def _bool(text):
    if text.lower() in ("1", "true", "yes", "y", "on"):
        return True
    if text.lower() in ("0", "false", "no", "n", "off"):
        return False
    raise argparse.ArgumentTypeError("expected a boolean, got %r" % text)


def build_parser():
    p = argparse.ArgumentParser(prog="python -m deepshift_amd.evaluate", description=__doc__.split("\n\n")[0])
    p.add_argument("-a", "--arch", default="mlp", choices=sorted(ARCHS))
    p.add_argument("--weights", default="", metavar="WEIGHTS_PATH", help="state_dict of the unconverted model")
    p.add_argument("--packed", default="", metavar="PACKED_PATH", help="packed sign+shift export to load")
    p.add_argument("--export-packed", default="", metavar="PACKED_PATH", help="write the packed export and go on")
    p.add_argument("--data", default="", metavar="DATA_PATH", help="torch file with 'input' and optional 'target'")
    p.add_argument("--shift-depth", type=int, default=1000, help="how many layers to convert, counted from the end")
    p.add_argument("-st", "--shift-type", default="PS", choices=["Q", "PS"])
    p.add_argument("-wb", "--weight-bits", type=int, default=5)
    p.add_argument("-ab", "--activation-bits", nargs=2, type=int, default=[16, 16], metavar=("I", "F"))
    p.add_argument("--batch-size", type=int, default=64)
    p.add_argument("--iterations", type=int, default=10, help="timed forward passes")
    p.add_argument("--seed", type=int, default=1)
    p.add_argument("-e", "--evaluate", action="store_true", help="evaluate (the only mode of this build)")
    p.add_argument("--use-kernel", type=_bool, default=False)
    p.add_argument("--fuse", type=_bool, default=True, help="fold BatchNorm/residual/ReLU into the kernel path")
    p.add_argument("--json", action="store_true", help="print one JSON object instead of text")
    return p


def _timed(model, x, iterations):
    with torch.no_grad():
        out = model(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iterations):
            out = model(x)
        torch.cuda.synchronize()
    return out, (time.perf_counter() - t0) / max(iterations, 1)


def main(argv=None):
    args = build_parser().parse_args(argv)
    if not args.evaluate:
        sys.exit("this build has no training loop: pass -e / --evaluate")
    if not torch.cuda.is_available():
        sys.exit("no GPU: the shift kernels of this build run on the GPU only")
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(args.seed)
    torch.manual_seed(args.seed)
    cls, chw = ARCHS[args.arch]
    model = cls()
    if args.weights:
        model.load_state_dict(torch.load(args.weights, map_location="cpu", weights_only=True))
    else:
        workloads.randomize_batchnorm(model, g)
    model.eval()

    target = None
    if args.data:
        blob = torch.load(args.data, map_location="cpu", weights_only=True)
        x, target = blob["input"].float(), blob.get("target")
    else:
        x = torch.rand(args.batch_size, *chw, generator=g) if args.arch == "mlp" else \
            torch.randn(args.batch_size, *chw, generator=g)
    x = x.to(dev)
    I, F = args.activation_bits
    report = {"arch": args.arch, "batch": int(x.shape[0]), "shift_type": args.shift_type,
              "weight_bits": args.weight_bits, "activation_bits": [I, F], "use_kernel": args.use_kernel}

    if args.shift_depth == 0 and args.use_kernel:
        # the reference's shift-against-multiply mode: float multiply kernels of the same structure
        # (imagenet.py:245-246)
        with torch.no_grad():
            want = model.to(dev)(x)
        model = convert_to_unoptimized(model).to(dev)
        out, sec = _timed(model, x, args.iterations)
        report.update(mode="float multiply comparator", converted_layers=0,
                      max_abs_diff_vs_pytorch=float((out - want).abs().max()))
    else:
        kw = dict(convert_weights=True, weight_bits=args.weight_bits, act_integer_bits=I, act_fraction_bits=F)
        model, n = convert.convert_to_shift(model, args.shift_depth, args.shift_type, use_kernel=False, **kw)
        model = model.to(dev)
        # convert_to_shift's own count follows the reference and leaves Linear layers out
        n = len(export._shift_layers(model))
        with torch.no_grad():
            reference_out = model(x)  # float shift path of the converted model
        for m in model.modules():
            if hasattr(m, "use_kernel"):
                m.use_kernel = args.use_kernel
        if args.packed:
            report["packed_layers_loaded"] = export.load_packed(model, args.packed)
        if args.export_packed:
            export.save_packed(model, args.export_packed)
            report["packed_export"] = args.export_packed
        run = fuse.fuse_conv_epilogues(model) if (args.use_kernel and args.fuse and args.arch != "mlp") else model
        out, sec = _timed(run, x, args.iterations)
        scale = float(reference_out.abs().max()) or 1.0
        report.update(mode="shift kernels" if args.use_kernel else "float shift path", converted_layers=n,
                      max_abs_diff_vs_float_shift_path=float((out - reference_out).abs().max()),
                      output_scale=scale,
                      argmax_agreement=float((out.argmax(1) == reference_out.argmax(1)).float().mean()))
    report.update(ms_per_batch=sec * 1e3, images_per_s=x.shape[0] / sec)
    if target is not None:
        report["top1"] = float((out.argmax(1).cpu() == target).float().mean())
    if args.json:
        print(json.dumps(report))
    else:
        for k, v in report.items():
            print("%-34s %s" % (k, v))
    return report


if __name__ == "__main__":
    main()
