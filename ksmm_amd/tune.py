"""Tuner: measures the kernel families/instances of libksmm_hip.so on a list of (a,b,c,d)
patterns and writes the table the library's automatic dispatch consults.

The reference tunes its CUDA kernels by brute force over hyper-parameters and stores the
winners in ``*.best`` files that are turned into ``best_kernel_*`` if-chains
(src/ksmm_py/layer/kronecker_sparse/kernel.py:151-257,
kernel_bs_first_float.cuh:8-21).  Here the candidates are the instances of the kernel families
(wave, stream, weight-stationary, GEMM, k-loop tiles), each forced through
``ksmm_factor_forward_algo`` and checked against the CPU oracle on sampled batch columns; the
fastest one per (pattern, element types, layout) goes into ``ksmm_amd/csrc/ksmm_tuned.inc``,
which is compiled into the library, named by its stable instance id.

    python -m ksmm_amd.tune --patterns FILE [--dtypes fp32,fp16,fp8] [--layouts last,first]
                            [--batch 25088] [--json OUT.json] [--merge A.json B.json ...]
                            [--emit ksmm_amd/csrc/ksmm_tuned.inc] [--emit-best ksmm_amd/tuned]
                            [--update ksmm_amd/csrc/ksmm_tuned.inc] [--update-best ksmm_amd/tuned]

``FILE`` holds one ``a,b,c,d`` per line (the reference's patterns.in has that format).  Several
runs (e.g. one per element type) can be merged with ``--merge`` before ``--emit``.
``--emit-best DIR`` writes ``kernel_bs_{first,last}_{float,half,fp8e4m3}.best``: one line per
pattern, ``batch a b c d <kernel> ms std mse`` as in the reference's files of that name
(kernel_bs_last_float.best:9), with the kernel named by family, instance id, parameter and
tile shape instead of the CUDA hyper-parameters.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

DT = {"fp32": torch.float32, "fp16": torch.float16, "fp8": torch.float8_e4m3fn}
COMBO = {"fp32": 0, "fp16": 1, "fp8": 2}


def _time_graph(fn, n_sets, steps):
    """Average seconds per call of fn(i): `steps` launches captured into a HIP graph on a side
    stream and replayed between two events on that stream."""
    fn(0)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for i in range(steps):
                fn(i % n_sets)
        graph.replay()
        stream.synchronize()
        t0 = torch.cuda.Event(enable_timing=True)
        t1 = torch.cuda.Event(enable_timing=True)
        t0.record(stream)
        graph.replay()
        t1.record(stream)
        stream.synchronize()
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) / 1e3 / steps


def _count(algo, make_variant, combo, bs_last, limit=1024):
    """Number of instances of a (sub-)family: indices are dense, the first one without an id ends it."""
    from . import _lib
    from .kernel import variant_id

    n = 0
    while n < limit:
        try:
            variant_id(algo, make_variant(n), combo, bs_last)
        except _lib.KsmmError:
            break
        n += 1
    return n


def candidates(bs_last=True, combo=1):
    """(algo, variant) pairs worth trying; the library refuses those that do not fit."""
    out = []
    if bs_last:
        for inst in range(_count(2, lambda i: i, combo, True, 255)):   # wave family: instance x tiles per wave
            for it in (0, 1, 2, 4, 8):
                out.append((2, inst | (it << 8)))
            for it in (0, 2, 4):                 # the same with tiles dealt round-robin
                out.append((2, inst | (it << 8) | (1 << 16)))
            out.append((2, inst | (2 << 16)))    # one round of workgroups, balanced dealing
    else:
        for inst in range(_count(2, lambda i: 1000 + i, combo, False)):   # batch-size-first row kernel
            out.append((2, 1000 + inst))
    for sub in (2, 4, 1, 3):                     # stream, direct-to-LDS GEMM, weight-stationary, d > 1 tiles
        for inst in range(_count(3, lambda i, sub=sub: (sub << 24) | i, combo, bs_last, 255)):
            out.append((3, (sub << 24) | inst))
    return out


def kloop_candidates(combo, bs_last):
    """k-loop tiles: only when nothing else fits."""
    return [(3, inst) for inst in range(_count(3, lambda i: i, combo, bs_last, 255))]


def _sample_cols(batch, n=48):
    idx = set(range(min(4, batch))) | set(range(max(0, batch - 4), batch))
    idx |= set(range(0, batch, max(1, batch // n)))
    return np.array(sorted(idx))


def tune_pattern(pattern, prec, bs_last, batch, lib_mod, rotation_bytes=1.3e9, tile_subs=None):
    from . import Kernel, generate_factor, quantize_fp8
    from .kernel import query_tile, variant_id
    from .layer import from_kernel_format_to_abcd

    a, b, c, d = pattern
    dt = DT[prec]
    out_dt = torch.float16 if prec == "fp8" else dt
    if query_tile(batch, pattern, dt, dt, bs_last)["algo"] == 1:
        # only the generic kernel (or the transposed route, which uses the batch-size-last
        # table) takes it in this layout: nothing to tune
        return {"pattern": list(pattern), "prec": prec, "bs_last": bool(bs_last), "batch": batch, "auto_us": None,
                "best_us": None, "algo": 0, "variant": -1, "n_candidates": 0}
    es_in = 1 if prec == "fp8" else (2 if prec == "fp16" else 4)
    es_out = 2 if prec != "fp32" else 4
    in_size, out_size = a * c * d, a * b * d
    per_set = batch * (in_size * es_in + out_size * es_out)
    # Consecutive launches rotate over distinct input/output sets of at least 1.2 GB in total (at
    # most 24 sets), as bench.py does: the 256 MB last-level cache cannot hand a set back to the
    # launch that uses it next, so candidates are ranked cold, the way they are used.
    n_sets = max(2, min(24, int(math.ceil(rotation_bytes / max(per_set, 1)))))
    g = torch.Generator(device="cuda").manual_seed(1)
    w4 = (torch.rand(a, b, c, d, generator=g, device="cuda") * 2 - 1) / math.sqrt(c)
    if prec == "fp8":
        wq, _ = quantize_fp8(w4.cpu())
        fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), dt, "cuda")
    else:
        fac = generate_factor(a, b, c, d, "kernel", w4.cpu(), dt, "cuda")
    xs, ys = [], []
    for _ in range(n_sets):
        x = torch.randn((in_size, batch) if bs_last else (batch, in_size), generator=g, device="cuda")
        xs.append(x.clamp_(-3, 3).to(dt) if prec == "fp8" else x.to(dt))
        ys.append(torch.empty((out_size, batch) if bs_last else (batch, out_size), dtype=out_dt, device="cuda"))

    def run(algo, variant, j=0):
        return Kernel.forward(xs[j], fac, bs_last, a, b, c, d, out=ys[j], algo=algo, variant=variant)

    # the checker: float64 oracle on sampled batch columns of the first input set (columns are
    # independent), on the values the device holds (rounded / dequantised operands)
    from oracle import ks_oracle as O

    cols = _sample_cols(batch)
    cols_t = torch.from_numpy(cols).cuda()
    xsub = (xs[0][:, cols_t] if bs_last else xs[0][cols_t, :]).to(torch.float32).double().cpu().numpy()
    wr = from_kernel_format_to_abcd(fac.to(torch.float32).cpu(), pattern).double().numpy()
    z = O.ks_apply_einsum(wr, xsub, bs_last)
    tol = {"fp32": 1e-5, "fp16": 2e-3, "fp8": 5e-3}[prec]

    def check(y):
        ysub = (y[:, cols_t] if bs_last else y[cols_t, :]).to(torch.float32).double().cpu().numpy()
        return O.rel_fro_error(ysub, z), float(np.mean((ysub - z) ** 2))

    combo = COMBO[prec]
    # what the heuristics pick, without the tuned table (variant -3)
    auto_err, auto_mse = check(run(0, -3))
    t_auto = _time_graph(lambda j: run(0, -3, j), n_sets, 6)
    steps = int(min(40, max(6, 1.5e-3 / max(t_auto, 1e-6))))
    results = []
    tried_any = False
    pools = (candidates(bs_last, combo), kloop_candidates(combo, bs_last))
    if tile_subs is not None:
        # a retune after instances were added to some tile sub-families: only those, against what
        # the present table (or, without a row, the heuristic) picks
        now = query_tile(batch, pattern, dt, dt, bs_last)
        pool = [(al, v) for al, v in pools[0] + pools[1] if al == 3 and (v >> 24) in tile_subs]
        if now["algo"] in (2, 3) and (now["algo"], now["variant"]) not in pool:
            pool.append((now["algo"], now["variant"]))
        pools = (pool,)
    for pool in pools:
        for algo, variant in pool:
            try:
                y = run(algo, variant)
            except lib_mod.KsmmError as e:
                if e.status == -6:
                    continue
                raise
            tried_any = True
            err, mse = check(y)
            if not err <= tol:
                print("  MISMATCH", pattern, prec, bs_last, algo, hex(variant), err, flush=True)
                continue
            t = _time_graph(lambda j: run(algo, variant, j), n_sets, steps)
            results.append((t, algo, variant, err, mse))
        if tried_any:
            break  # k-loop tiles only when no other family took the problem
    results.sort()
    best = results[0] if results else None
    t_a, t_b = [t_auto], [best[0]] if best else []
    if best:
        # confirm: heuristic choice and winner timed alternately, three runs each
        for _ in range(2):
            t_a.append(_time_graph(lambda j: run(0, -3, j), n_sets, steps))
            t_b.append(_time_graph(lambda j: run(best[1], best[2], j), n_sets, steps))
    # roofline bound of the factor: HBM at 8 TB/s against the dense MFMA peak of the type the
    # kernels multiply in (fp32 157.3, fp16 2516.6, e4m3 GEMM tiles 5033.2 TFLOP/s)
    peak = {"fp32": 157.3e12, "fp16": 2516.6e12, "fp8": 5033.2e12}[prec]
    bound = max(per_set / 8e12, 2.0 * batch * a * b * c * d / peak)
    entry = {"pattern": list(pattern), "prec": prec, "bs_last": bool(bs_last), "batch": batch,
             "auto_us": min(t_a) * 1e6, "auto_mean_us": float(np.mean(t_a)) * 1e6, "auto_std_us": float(np.std(t_a)) * 1e6,
             "auto_rel_err": auto_err, "auto_mse": auto_mse, "auto_tile": query_tile(batch, pattern, dt, dt, bs_last, 0, -3),
             "bound_us": bound * 1e6, "best_us": None, "algo": 0, "variant": -1, "n_candidates": len(results)}
    if best:
        iid, par = variant_id(best[1], best[2], combo, bs_last)
        entry.update({"best_us": min(t_b) * 1e6, "best_mean_us": float(np.mean(t_b)) * 1e6,
                      "best_std_us": float(np.std(t_b)) * 1e6, "algo": best[1], "variant": best[2], "id": iid,
                      "param": par, "rel_err": best[3], "mse": best[4],
                      "tile": query_tile(batch, pattern, dt, dt, bs_last, best[1], best[2])})
    return entry


def _entry_id(e):
    """(instance id, parameter) of an entry for the library at hand, or None when the kernel it
    measured cannot be named any more.  The id recorded at measuring time is used when it still
    resolves to a kernel with the recorded tile; otherwise (an older run, or a build whose ids
    were formed differently) the recorded variant is tried, under the same check: a variant is a
    position in an instance table and only means the same kernel while that table is unchanged."""
    from . import _lib
    from .kernel import query_tile, variant_from_id, variant_id

    a, b, c, d = e["pattern"]
    dt = DT[e["prec"]]
    want = e.get("tile") or {}

    def same_kernel(variant):
        try:
            t = query_tile(e.get("batch", 25088), (a, b, c, d), dt, None, e["bs_last"], e["algo"], variant)
        except _lib.KsmmError:
            return False
        return all(t[k] == want[k] for k in ("tile_m", "tile_n", "tile_k", "tile_d", "threads") if k in want)

    if "id" in e and e["id"]:
        try:
            v = variant_from_id(e["algo"], e["id"], e.get("param", 0), COMBO[e["prec"]], e["bs_last"])
            if same_kernel(v):
                return e["id"], e.get("param", 0)
        except _lib.KsmmError:
            pass
    if same_kernel(e["variant"]):
        return variant_id(e["algo"], e["variant"], COMBO[e["prec"]], e["bs_last"])
    return None


def emit(entries, path, batch):
    """Write the C table: one row per entry where the tuned choice beats the heuristic by > 3 %."""
    rows = []
    for e in entries:
        if e.get("best_us") is None or e.get("auto_us") is None or e["algo"] == 0:
            continue
        if not e["best_us"] < 0.97 * e["auto_us"]:
            continue
        a, b, c, d = e["pattern"]
        named = _entry_id(e)
        if named is None:
            print("dropped (kernel not in this library): %s %s bs_last=%s variant %s" % (
                e["pattern"], e["prec"], e["bs_last"], hex(e["variant"])), file=sys.stderr)
            continue
        iid, par = named
        rows.append((a, b, c, d, COMBO[e["prec"]], 1 if e["bs_last"] else 0, e["algo"], iid, par,
                     e["best_us"], e["auto_us"]))
    rows.sort(key=lambda r: (r[:6], r[9]))  # by key, fastest first
    rows = [r for i, r in enumerate(rows) if i == 0 or r[:6] != rows[i - 1][:6]]  # one row per key
    with open(path, "w") as f:
        f.write("// Generated by `python -m ksmm_amd.tune` on MI355X (gfx950) at batch %d: fastest measured\n" % batch)
        f.write("// (family, instance id, parameter) per (a, b, c, d, element-type combination, layout), kept only\n")
        f.write("// where it beats the heuristic choice by more than 3 %.  Sorted by key for binary search.\n")
        f.write("// {a, b, c, d, combo, bs_last, algo, instance id, parameter},  // tuned us (heuristic us)\n")
        for r in rows:
            f.write("{%d, %d, %d, %d, %d, %d, %d, %du, %d},  // %.1f (%.1f)\n" % r)
    return len(rows)


def update_inc(entries, path, batch):
    """Re-measured patterns into an existing table: the rows of every (pattern, type, layout) in
    ``entries`` are replaced by what ``emit`` would write for them (or dropped when the heuristic
    is now within 3 %); all other rows stay as they are."""
    import re
    import tempfile

    keep = []
    redone = {(tuple(e["pattern"]), COMBO[e["prec"]], 1 if e["bs_last"] else 0) for e in entries}
    row_re = re.compile(r"^\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+)u, (-?\d+)\},\s*//\s*([\d.]+) \(([\d.]+)\)")
    for line in open(path):
        m = row_re.match(line)
        if not m:
            continue
        v = [int(g) for g in m.groups()[:9]]
        if (tuple(v[:4]), v[4], v[5]) in redone:
            continue
        keep.append(tuple(v) + (float(m.group(10)), float(m.group(11))))
    with tempfile.NamedTemporaryFile("r", suffix=".inc") as tmp:
        emit(entries, tmp.name, batch)
        for line in open(tmp.name):
            m = row_re.match(line)
            if m:
                keep.append(tuple(int(g) for g in m.groups()[:9]) + (float(m.group(10)), float(m.group(11))))
    keep.sort(key=lambda r: r[:6])
    head = [l for l in open(path) if l.startswith("//")]
    with open(path, "w") as f:
        f.writelines(head)
        for r in keep:
            f.write("{%d, %d, %d, %d, %d, %d, %d, %du, %d},  // %.1f (%.1f)\n" % r)
    return len(keep)


def update_best(entries, directory):
    """The same for the ``*.best`` text files: lines of re-measured patterns are replaced."""
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        written = emit_best(entries, tmp)
        for name in written:
            new_lines = [l for l in open(os.path.join(tmp, name)) if not l.startswith("#")]
            key = lambda l: tuple(l.split()[:5])
            fresh = {key(l): l for l in new_lines}
            old_path = os.path.join(directory, name)
            old_lines = [l for l in open(old_path)] if os.path.exists(old_path) else []
            head = [l for l in old_lines if l.startswith("#")] or [open(os.path.join(tmp, name)).readline()]
            body = {key(l): l for l in old_lines if not l.startswith("#")}
            body.update(fresh)
            with open(old_path, "w") as f:
                f.writelines(head[:1])
                for k in sorted(body, key=lambda k: tuple(int(v) for v in k)):
                    f.write(body[k])
    return written


BEST_NAME = {"fp32": "float", "fp16": "half", "fp8": "fp8e4m3"}
FAMILY = {0: "auto", 1: "generic", 2: "wave", 3: "tile"}


def emit_best(entries, directory):
    """Per element type and layout, one ``*.best`` text file in the reference's spirit
    (kernel_bs_last_float.best: ``batch a b c d TILEX TILEK TILEY TX TY VSIZE ms std mse``):
    ``batch a b c d family instance_id parameter tile_m tile_n tile_k tile_d threads ms std mse``
    for the fastest measured kernel, followed by the heuristic choice's ``ms std`` and the
    factor's roofline floor.  Times are milliseconds per launch (mean and standard deviation of
    the repeated HIP-graph timings), mse is the mean squared error against the float64 oracle on
    the sampled batch columns."""
    os.makedirs(directory, exist_ok=True)
    written = {}
    for prec in ("fp32", "fp16", "fp8"):
        for bs_last in (False, True):
            sel = [e for e in entries if e["prec"] == prec and e["bs_last"] == bs_last and e.get("auto_us")]
            if not sel:
                continue
            sel.sort(key=lambda e: e["pattern"])
            name = "kernel_bs_%s_%s.best" % ("last" if bs_last else "first", BEST_NAME[prec])
            with open(os.path.join(directory, name), "w") as f:
                f.write("# batch a b c d family instance_id parameter tile_m tile_n tile_k tile_d threads ms std mse "
                        "| heuristic_ms heuristic_std roofline_floor_ms\n")
                for e in sel:
                    a, b, c, d = e["pattern"]
                    use_best = e.get("best_us") is not None and e["algo"] != 0 and e["best_us"] <= e["auto_us"]
                    if use_best:
                        t = e.get("tile", {})
                        fam = FAMILY[e["algo"]]
                        iid, par = _entry_id(e) or (0, 0)
                        ms, std, mse = e.get("best_mean_us", e["best_us"]) / 1e3, e.get("best_std_us", 0.0) / 1e3, e.get("mse", float("nan"))
                    else:
                        t = e.get("auto_tile", {})
                        fam, iid, par = FAMILY.get(t.get("algo", 0), "auto"), 0, 0
                        ms, std, mse = e.get("auto_mean_us", e["auto_us"]) / 1e3, e.get("auto_std_us", 0.0) / 1e3, e.get("auto_mse", float("nan"))
                    f.write("%d %d %d %d %d %s %d %d %d %d %d %d %d %.6f %.6f %.3e | %.6f %.6f %.6f\n" % (
                        e.get("batch", 25088), a, b, c, d, fam, iid, par, t.get("tile_m", 0), t.get("tile_n", 0),
                        t.get("tile_k", 0), t.get("tile_d", 0), t.get("threads", 0), ms, std, mse,
                        e.get("auto_mean_us", e["auto_us"]) / 1e3, e.get("auto_std_us", 0.0) / 1e3,
                        e.get("bound_us", 0.0) / 1e3))
            written[name] = len(sel)
    return written


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--patterns")
    ap.add_argument("--dtypes", default="fp32,fp16")
    ap.add_argument("--layouts", default="last")
    ap.add_argument("--batch", type=int, default=25088)
    ap.add_argument("--json")
    ap.add_argument("--merge", nargs="*", default=[])
    ap.add_argument("--emit")
    ap.add_argument("--emit-best", help="directory for the kernel_bs_*_*.best text files")
    ap.add_argument("--update", help="an existing table (.inc): replace the rows of the measured patterns, keep the rest")
    ap.add_argument("--update-best", help="directory of existing *.best files: replace the lines of the measured patterns")
    ap.add_argument("--shard", default="0/1", help="i/n: take every n-th pattern starting at i")
    ap.add_argument("--time-limit", type=float, default=1e9, help="stop (and save) after this many seconds")
    ap.add_argument("--tile-subs", help="comma-separated tile sub-families (0 k-loop tiles, 2 stream, 4 GEMM, "
                    "1 weight-stationary, 3 d > 1 tiles): try only their instances and the present table's pick")
    args = ap.parse_args()
    entries = []
    for p in args.merge:
        entries += json.load(open(p))
    # the same (pattern, type, layout) measured twice: the file named first wins
    seen = set()
    entries = [e for e in entries
               if (k := (tuple(e["pattern"]), e["prec"], bool(e["bs_last"]))) not in seen and not seen.add(k)]
    if args.patterns:
        from . import _lib

        _lib.load()
        pats = [tuple(int(v) for v in l.strip().split(",")) for l in open(args.patterns) if l.strip()]
        pats = list(dict.fromkeys(pats))
        si, sn = (int(v) for v in args.shard.split("/"))
        pats = pats[si::sn]
        t_start = time.time()
        done = {(tuple(e["pattern"]), e["prec"], e["bs_last"]) for e in entries}
        for prec in args.dtypes.split(","):
            for layout in args.layouts.split(","):
                bs_last = layout == "last"
                for i, p in enumerate(pats):
                    if (p, prec, bs_last) in done:
                        continue
                    if time.time() - t_start > args.time_limit:
                        break
                    try:
                        e = tune_pattern(p, prec, bs_last, args.batch, _lib,
                                         tile_subs=[int(v) for v in args.tile_subs.split(",")] if args.tile_subs else None)
                    except torch.cuda.OutOfMemoryError:
                        print("  OOM", p, prec, layout, flush=True)
                        torch.cuda.empty_cache()
                        continue
                    entries.append(e)
                    print("%s %s %s: auto %s us, best %s us (algo %d variant %s, %d candidates) [%d/%d]" % (
                        prec, layout, p, "%.1f" % e["auto_us"] if e["auto_us"] else "-",
                        "%.1f" % e["best_us"] if e["best_us"] else "-", e["algo"],
                        hex(e["variant"]) if e["variant"] >= 0 else e["variant"], e["n_candidates"], i + 1, len(pats)),
                        flush=True)
                    if args.json and (i % 20 == 19):
                        json.dump(entries, open(args.json, "w"))
        if args.json:
            json.dump(entries, open(args.json, "w"))
    elif args.json and entries:
        json.dump(entries, open(args.json, "w"))
    if args.emit:
        n = emit(entries, args.emit, args.batch)
        print("wrote %d rows to %s" % (n, args.emit))
    if args.update:
        print("%s now holds %d rows" % (args.update, update_inc(entries, args.update, args.batch)))
    if args.update_best:
        for name, n in update_best(entries, args.update_best).items():
            print("updated %d patterns in %s" % (n, os.path.join(args.update_best, name)))
    if args.emit_best:
        for name, n in emit_best(entries, args.emit_best).items():
            print("wrote %d patterns to %s" % (n, os.path.join(args.emit_best, name)))


if __name__ == "__main__":
    main()
