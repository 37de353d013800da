"""Timing CLI that writes the reference's benchmark CSV.

Same flags, timing protocol and CSV schema as the reference's
``src/ksmm_py/benchmark/ksmm_time.py`` (:20-48 flags, :61-67 columns
``pattern,batch-size,algo,bs_position,precision,vsize,device_name,mean,median,iqr,times``,
:148-164 ``--correctness``, :168-190 ``blocked_autorange`` with the 11x re-run), so its result
files and plotting scripts take rows produced here:

    python -m ksmm_amd.bench_csv --saving-csv out.csv --patterns 6,64,64,1 1,768,192,2 \\
        --algo kernel --bs-last 1 --device cuda --precision fp32 --batch-size 25088 --correctness

Additions: ``--precision fp8`` (e4m3 weights and input, fp16 output) and the feed-forward
granularities of the reference's ViT benchmark (scripts/2_benchmark_ksvit_time.sh:23,49-51;
src/ksmm_py/model/vit.py:416-431) built from KSLinear chains: ``linear_up`` / ``linear_down``
(one projection, ``--patterns_up`` / ``--patterns_down``), their ``_bias`` forms, and ``ffn``
(up + bias + GELU, then down + bias).  With ``--algo kernel`` bias and GELU run inside the last
factor's kernel.  ``--granularity linear`` (default) is the reference's ksmm_time.py case.
"""
import argparse
import csv
import os
import sys

import torch
import torch.utils.benchmark as benchmark

from . import KSLinear

COLUMNS = ["pattern", "batch-size", "algo", "bs_position", "precision", "vsize", "device_name", "mean", "median",
           "iqr", "times"]
KEY = COLUMNS[:7]
GRANULARITIES = ["linear", "linear_bias", "linear_up", "linear_up_bias", "linear_down", "linear_down_bias", "ffn"]
DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "fp8": torch.float8_e4m3fn}


def parse_patterns(patterns):
    """["a,b,c,d", ...] -> [[a, b, c, d], ...] (benchmark/utils.py:135-148)."""
    out = []
    for r in patterns or []:
        vals = [int(s) for s in r.split(",")]
        assert len(vals) == 4, "a pattern is four integers a,b,c,d"
        out.append(vals)
    return out


def get_args(argv=None):
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--saving-csv", type=str)
    p.add_argument("--device-id", type=int, default=0)
    p.add_argument("--patterns", type=str, nargs="+", default=[])
    p.add_argument("--patterns_up", type=str, nargs="+", default=[])
    p.add_argument("--patterns_down", type=str, nargs="+", default=[])
    p.add_argument("--granularity", choices=GRANULARITIES, default="linear")
    p.add_argument("--algo", choices=["dense", "bmm", "kernel", "einsum"], default="kernel")
    p.add_argument("--bs-last", type=int, choices=[0, 1], default=0, help="0 batch-size-first, 1 batch-size-last")
    p.add_argument("--device", choices=["cuda", "cpu"], default="cpu")
    p.add_argument("--precision", choices=sorted(DTYPES), default="fp32")
    p.add_argument("--batch-size", type=int, default=1)
    p.add_argument("--vsize", type=int, default=4)
    p.add_argument("--min-run-time", type=float, default=0.25)
    p.add_argument("--correctness", action="store_true")
    p.add_argument("--seed", type=int, default=0)
    args = p.parse_args(argv)
    args.bs_last = args.bs_last == 1
    return args


class FeedForward(torch.nn.Module):
    """up -> GELU -> down with biases (vit.py:416-431), both projections Kronecker-sparse."""

    def __init__(self, up, down):
        super().__init__()
        self.up, self.down = up, down

    def forward(self, x, x_scale=None):
        return self.down(self.up(x, x_scale))


def build_model(args):
    """The module to time and the pattern list that names it in the CSV."""
    dtype = DTYPES[args.precision]
    dev = args.device

    def layer(patterns, bias, act=None):
        return KSLinear(parse_patterns(patterns), bias=bias, algo=args.algo, dtype=dtype, bs_last=args.bs_last,
                        vsize=args.vsize, device=dev, act=act)

    g = args.granularity
    if g in ("linear", "linear_bias"):
        pats = args.patterns
        model = layer(pats, g.endswith("_bias"))
    elif g in ("linear_up", "linear_up_bias"):
        pats = args.patterns_up or args.patterns
        model = layer(pats, g.endswith("_bias"))
    elif g in ("linear_down", "linear_down_bias"):
        pats = args.patterns_down or args.patterns
        model = layer(pats, g.endswith("_bias"))
    else:
        assert args.patterns_up and args.patterns_down, "ffn needs --patterns_up and --patterns_down"
        pats = args.patterns_up + args.patterns_down
        model = FeedForward(layer(args.patterns_up, True, act="gelu"), layer(args.patterns_down, True))
    assert pats, "no patterns given"
    return model.eval(), pats


def in_size_of(model):
    return (model.up if isinstance(model, FeedForward) else model).in_size


def reference_output(model, x, bs_last):
    """The layer's dense product applied on the CPU in fp32 (ksmm_time.py:148-157), with the
    bias and GELU of the granularity."""
    def one(ksl, y):
        dense = ksl.get_dense_product(torch.float32).to("cpu")
        y = torch.mm(dense, y) if bs_last else torch.mm(dense, y.t()).t()
        if ksl.bias is not None:
            y = y + ksl.bias.detach().to("cpu", torch.float32)
        return torch.nn.functional.gelu(y) if ksl.act == "gelu" else y

    y = x.detach().to("cpu", torch.float32)
    for ksl in ((model.up, model.down) if isinstance(model, FeedForward) else (model,)):
        y = one(ksl, y)
    return y


def save_results(args, pats, m, device_name):
    """Insert or replace the row with this configuration (ksmm_time.py:51-118; the reference
    compares vsize with the precision there, so it never replaces: here the key is the seven
    configuration columns)."""
    row = {"pattern": str([list(p) for p in parse_patterns(pats)]) if args.granularity == "linear"
           else "%s:%s" % (args.granularity, [list(p) for p in parse_patterns(pats)]),
           "batch-size": args.batch_size, "algo": args.algo, "bs_position": "bs_last" if args.bs_last else "bs_first",
           "precision": args.precision, "vsize": args.vsize, "device_name": device_name, "mean": m.mean,
           "median": m.median, "iqr": m.iqr, "times": str(m.times)}
    rows = []
    if os.path.exists(args.saving_csv):
        with open(args.saving_csv, newline="") as f:
            reader = csv.DictReader(f)
            missing = [c for c in COLUMNS if c not in (reader.fieldnames or [])]
            if missing:
                raise ValueError("Column %s not found in the CSV file. Please provide a valid CSV file." % missing[0])
            rows = list(reader)
    same = [i for i, r in enumerate(rows) if all(str(r[k]) == str(row[k]) for k in KEY)]
    assert len(same) <= 1, "The CSV file should not contain multiple rows with the same configuration."
    if same:
        rows[same[0]] = row
    else:
        rows.append(row)
    os.makedirs(os.path.dirname(os.path.abspath(args.saving_csv)), exist_ok=True)
    with open(args.saving_csv, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=COLUMNS, extrasaction="ignore")
        w.writeheader()
        w.writerows(rows)
    return row


def forward_pass(model, x, x_scale=None):
    """utils.py:6-8 of the reference; ``x_scale`` is the per-tensor scale of an e4m3 input."""
    with torch.no_grad():
        return model(x) if x_scale is None else model(x, x_scale)


def main(argv=None):
    args = get_args(argv)
    print("\n", args)
    if args.device == "cuda":
        torch.cuda.set_device(args.device_id)
        device_name = torch.cuda.get_device_name(args.device_id)
    else:
        import platform

        device_name = platform.processor() or "cpu"
    torch.manual_seed(args.seed)
    model, pats = build_model(args)
    n_in = in_size_of(model)
    x = torch.randn((n_in, args.batch_size) if args.bs_last else (args.batch_size, n_in))
    x_scale = None
    if args.precision == "fp8" and args.algo == "kernel":
        # e4m3 input: quantised once, outside the timed region; its scale travels with it (the
        # layer's own weight scales stay as they are, so get_dense_product() is the dequantised
        # weight matrix and the reference below is that matrix times the dequantised input)
        from . import quantize_fp8

        xq, xs = quantize_fp8(x)
        x_scale = float(xs)
        x_dev, x_ref = xq.to(args.device), xq.to(torch.float32) * xs
    else:
        dt = torch.float32 if args.precision == "fp8" else DTYPES[args.precision]
        x_dev = x.to(dt).to(args.device)
        x_ref = x_dev
    if args.correctness:
        want = reference_output(model, x_ref, args.bs_last)
        got = forward_pass(model, x_dev, x_scale).to("cpu", torch.float32)
        rel_err = torch.norm(want - got) / torch.norm(want)
        print("Relative error = {0:e}".format(rel_err))
        main.last_relative_error = float(rel_err)
    t = benchmark.Timer(stmt="forward_pass(model, x, x_scale)",
                        globals={"model": model, "x": x_dev, "x_scale": x_scale, "forward_pass": forward_pass},
                        num_threads=torch.get_num_threads())
    m = t.blocked_autorange(min_run_time=args.min_run_time)
    if m.number_per_run <= 10:  # not enough measurements (ksmm_time.py:181-190)
        m = t.blocked_autorange(min_run_time=11.0 * max(m.mean, m.median))
    print(m)
    if args.saving_csv:
        save_results(args, pats, m, device_name)
    return m


main.last_relative_error = None  # what the last --correctness run printed (for callers and tests)


if __name__ == "__main__":
    main(sys.argv[1:])
