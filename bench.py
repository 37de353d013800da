#!/usr/bin/env python3
"""Benchmark of the KS hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all 0|1]
    python bench.py --factor fp16:last:1,768,192,16     (one factor only: per-kernel profiling runs)

A step is one forward pass of one KS factor over a batch of 25 088 columns.  The headline
workload is BASELINE configuration 2: a single fp32 factor with pattern (1,48,48,16)
(768 -> 768), batch-size-last.  The JSON line also carries every other configuration
(µs per factor and per KSLinear, effective GB/s and TFLOP/s, fraction of the bounding
roofline, parity error against the CPU oracle on sampled columns), the roofline record of
the headline kernel and the CPU baseline (the reference's ``algo='bmm'`` algorithm restated
with torch.bmm, timed on this host's cores).

Inputs are synthetic (seeded), resident in HBM before the timed region.  To keep the 256 MB
last-level cache from serving repeated launches, consecutive steps rotate through distinct
input/output buffers whose total footprint exceeds 1 GB.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

BATCH = 25088
SEED = 0
FP8 = torch.float8_e4m3fn
CONFIGS = [
    # name, patterns, precision, bs_last, weight bound
    ("C2_bs_last", [(1, 48, 48, 16)], "fp32", True, None),
    ("C2_bs_first", [(1, 48, 48, 16)], "fp32", False, None),
    ("C1_readme", [(6, 64, 64, 1), (1, 768, 192, 2)], "fp32", True, None),
    ("C3_bs_last", [(4, 192, 192, 1)], "fp16", True, None),
    ("C3_bs_first", [(4, 192, 192, 1)], "fp16", False, None),
    ("C4_vit_b_up", [(12, 64, 64, 1), (1, 1536, 384, 2)], "fp16", False, None),
    ("C5_butterfly", [(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)], "fp8", True, 0.25),
]
DT = {"fp32": torch.float32, "fp16": torch.float16, "fp8": FP8}
TOL = {"fp32": 1e-5, "fp16": 2e-3, "fp8": 5e-2}


def make_weights(patterns, bound, gen):
    out = []
    for (a, b, c, d) in patterns:
        s = bound if bound is not None else 1.0 / math.sqrt(c)
        out.append((torch.rand(a, b, c, d, generator=gen) * 2 - 1) * s)
    return out


def time_launches(fn, n_sets, steps, warmup):
    """Average seconds per call of fn(i) (i rotates over buffer sets).

    The `steps` launches are captured once into a HIP graph on a side stream and replayed, so
    that the timed region holds back-to-back kernels rather than Python launch overhead; HIP
    events are recorded on the stream the graph (and hence every kernel) runs on, with a
    device-wide synchronisation on both sides."""
    for i in range(warmup):
        fn(i % n_sets)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for i in range(steps):
                fn(i % n_sets)
        graph.replay()  # untimed: first replay uploads the graph
        stream.synchronize()
        torch.cuda.synchronize()
        t0 = torch.cuda.Event(enable_timing=True)
        t1 = torch.cuda.Event(enable_timing=True)
        t0.record(stream)
        graph.replay()
        t1.record(stream)
        stream.synchronize()
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) / 1e3 / steps


def pattern_copy_us(p, bs_last, srcs, dsts, steps, warmup):
    """Time of a tile-at-a-time copy that touches memory the way a factor with square blocks does
    and computes nothing (ksbench_tilecopy_probe), best of the tile widths the probe takes; None where the
    pattern has no such copy (b != c, input and output element sizes differ, bs_first, whose
    rows are contiguous)."""
    import ctypes

    from ksmm_amd import _lib, bench_lib

    a, b, c, d = p
    es = srcs[0].element_size()
    if b != c or dsts[0].element_size() != es or srcs[0].shape != dsts[0].shape:
        return None
    if bs_last:
        cases = [(BATCH * es, a, c, d, tb) for tb in (256, 1024, 4096) if c <= 48 * (4096 // tb)]
    else:
        return None
    lib = bench_lib.load()
    best = None
    for row_bytes, pa, rows, pd, tb in cases:
        def run(j):
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check(lib.ksbench_tilecopy_probe(srcs[j].data_ptr(), dsts[j].data_ptr(), row_bytes, pa, rows, pd, tb, stream))

        run(0)
        torch.cuda.synchronize()
        if not torch.equal(srcs[0].view(torch.uint8), dsts[0].view(torch.uint8)):
            raise RuntimeError("tile copy probe: output differs from input")
        sec = time_launches(run, len(srcs), max(10, steps // 4), max(3, warmup // 4))
        best = sec if best is None else min(best, sec)
    return best * 1e6


def bench_config(name, patterns, prec, bs_last, bound, steps, warmup, check=True):
    """Per-factor and whole-chain timings of one configuration."""
    from ksmm_amd import Kernel, generate_factor, quantize_fp8, query_tile
    from ksmm_amd.roofline import factor_roofline, factor_work

    gen = torch.Generator().manual_seed(SEED)
    ws4 = make_weights(patterns, bound, gen)
    in_size = patterns[0][0] * patterns[0][2] * patterns[0][3]
    dt = DT[prec]
    out_dt = torch.float16 if prec == "fp8" else dt
    # enough rotating buffer sets to exceed the last-level cache several times over
    widest = max([in_size] + [p[0] * p[1] * p[3] for p in patterns])
    per_set = 2 * widest * BATCH * 4
    n_sets = max(2, min(8, int(math.ceil(1.2e9 / per_set))))
    xs, scales = [], []
    for i in range(n_sets):
        g = torch.Generator().manual_seed(SEED + 1 + i)
        x = torch.randn(BATCH, in_size, generator=g)
        x = x.t().contiguous() if bs_last else x
        if prec == "fp8":
            q, s = quantize_fp8(x)
            xs.append(q.cuda())
            scales.append(float(s))
        else:
            xs.append(x.to(dt).cuda())
            scales.append(1.0)
    facs, wscales = [], []
    for p, w4 in zip(patterns, ws4):
        if prec == "fp8":
            q4, s = quantize_fp8(w4)
            facs.append(generate_factor(*p, "kernel", q4.float(), FP8, "cuda"))
            wscales.append(float(s))
        else:
            facs.append(generate_factor(*p, "kernel", w4, dt, "cuda"))
            wscales.append(1.0)

    result = {"name": name, "precision": prec, "bs_last": bs_last, "patterns": patterns, "factors": []}
    # ---- per factor: input of factor i is the (precomputed) output of factor i-1 ----------
    cur = xs
    for i, p in enumerate(patterns):
        a, b, c, d = p
        out_size = a * b * d
        shape = (out_size, BATCH) if bs_last else (BATCH, out_size)
        outs = [torch.empty(shape, dtype=out_dt, device="cuda") for _ in range(n_sets)]
        sc = [wscales[i] * (scales[j] if i == 0 else 1.0) for j in range(n_sets)]

        def run(j, cur=cur, outs=outs, sc=sc, i=i, p=p):
            Kernel.forward(cur[j], facs[i], bs_last, *p, scale=sc[j], out=outs[j])

        copy_us = pattern_copy_us(p, bs_last, cur, outs, steps, warmup)
        sec = time_launches(run, n_sets, steps, warmup)
        stream_us = same_bytes_stream_copy_us(cur[0].numel() * cur[0].element_size()
                                              + outs[0].numel() * outs[0].element_size(), steps, warmup)
        x_dt = cur[0].dtype
        roof = factor_roofline(BATCH, p, x_dt, facs[i].dtype, out_dt, sec)
        tile = query_tile(BATCH, p, x_dt, facs[i].dtype, bs_last)
        result["factors"].append({
            "pattern": p, "us": sec * 1e6, "gbs": roof["gbs"], "tflops": roof["tflops"],
            "bound": roof["bound"], "roofline_frac": roof["frac"], "floor_us": roof["floor_us"],
            "x_dtype": str(x_dt).replace("torch.", ""), "algo": tile["algo"], "variant": tile["variant"],
            # a tile-at-a-time copy with this factor's addresses and no arithmetic (None: no such copy)
            "pattern_copy_us": copy_us,
            # the streaming copy (non-temporal, persistent grid) moving as many bytes as this factor
            # reads and writes, half of them each way: what the memory system gives a kernel that
            # does nothing else
            "stream_copy_us": stream_us, "frac_of_stream_copy": stream_us / (sec * 1e6)})
        cur = outs
    # ---- whole KSLinear (chain launcher) ----------------------------------------------------
    if len(patterns) > 1:
        ws_bytes = torch.empty(2 * (widest * BATCH * 4 + 256), dtype=torch.uint8, device="cuda")

        def run_chain(j, fuse=True):
            sc = list(wscales)
            sc[0] *= scales[j]
            return Kernel.chain_forward(xs[j], facs, patterns, bs_last, scales=sc, fuse=fuse,
                                        workspace=ws_bytes)

        sec = time_launches(run_chain, n_sets, max(3, steps // 2), max(1, warmup // 2))
        result["kslinear_us"] = sec * 1e6
        sec = time_launches(lambda j: run_chain(j, False), n_sets, max(3, steps // 2), max(1, warmup // 2))
        result["kslinear_unfused_us"] = sec * 1e6
        final = run_chain(0)
        # the layer as a network uses it: bias (and, for the ViT up-projection, GELU) applied by the
        # last factor's kernel, against the same chain followed by a separate elementwise pass
        out_size = patterns[-1][0] * patterns[-1][1] * patterns[-1][3]
        bias = (torch.rand(out_size, generator=torch.Generator().manual_seed(SEED + 99)) - 0.5).to(out_dt).cuda()
        act = "gelu" if name == "C4_vit_b_up" else None
        outs_ep = [torch.empty_like(final) for _ in range(n_sets)]

        def run_chain_ep(j):
            sc = list(wscales)
            sc[0] *= scales[j]
            return Kernel.chain_forward(xs[j], facs, patterns, bs_last, scales=sc, fuse=True, workspace=ws_bytes,
                                        bias=bias, act=act, out=outs_ep[j])

        def run_chain_then_torch(j):
            y = run_chain(j)
            y = y + (bias[:, None] if bs_last else bias)
            return torch.nn.functional.gelu(y) if act else y

        sec = time_launches(run_chain_ep, n_sets, max(3, steps // 2), max(1, warmup // 2))
        result["kslinear_bias%s_fused_us" % ("_gelu" if act else "")] = sec * 1e6
        sec = time_launches(run_chain_then_torch, n_sets, max(3, steps // 2), max(1, warmup // 2))
        result["kslinear_bias%s_separate_pass_us" % ("_gelu" if act else "")] = sec * 1e6
    else:
        result["kslinear_us"] = result["factors"][0]["us"]
        final = cur[0]
    # ---- parity on sampled batch columns ---------------------------------------------------
    if check:
        from oracle import ks_oracle as O
        import numpy as np

        cols = np.unique(np.concatenate([np.arange(0, BATCH, 197), np.arange(BATCH - 4, BATCH)]))
        g = torch.Generator().manual_seed(SEED + 1)
        x0 = torch.randn(BATCH, in_size, generator=g)
        x0 = x0.t().contiguous() if bs_last else x0
        if prec == "fp8":
            xr = xs[0].cpu().to(torch.float32).double().numpy() * scales[0]
            wr = [f.double().numpy() for f in
                  [quantize_fp8(w)[0].to(torch.float32) * quantize_fp8(w)[1] for w in ws4]]
        else:
            xr = x0.to(dt).double().numpy()
            wr = [w.to(dt).double().numpy() for w in ws4]
        xsub = xr[:, cols] if bs_last else xr[cols, :]
        z = O.chain_apply(wr, xsub, bs_last)
        yh = final.float().cpu().numpy()
        ysub = yh[:, cols] if bs_last else yh[cols, :]
        result["rel_fro_error"] = O.rel_fro_error(ysub, z)
        result["tolerance"] = TOL[prec]
        result["parity_ok"] = bool(result["rel_fro_error"] <= TOL[prec])
    return result


FFN_UP = [(6, 64, 64, 1), (1, 768, 192, 2)]      # 384 -> 1536
FFN_DOWN = [(6, 64, 256, 1), (1, 128, 128, 3)]   # 1536 -> 384


def bench_ffn(steps, warmup, prec="fp16", bs_last=False):
    """The feed-forward block of the reference's ViT-S benchmark (scripts/2_benchmark_ksvit_time.sh:5,
    48-50; src/ksmm_py/model/vit.py:416-431) at B = 25 088 rows (196 tokens x 128 images), in its
    default layout: up-projection + bias + GELU (both inside the last factor's kernel), then
    down-projection + bias, two chain launches; per factor of the down-projection as well.  Checked
    against the float64 oracle on sampled rows."""
    from ksmm_amd import Kernel, generate_factor
    from ksmm_amd.roofline import factor_roofline

    dt = DT[prec]
    gen = torch.Generator().manual_seed(SEED + 11)
    w_up, w_dn = make_weights(FFN_UP, None, gen), make_weights(FFN_DOWN, None, gen)
    f_up = [generate_factor(*p, "kernel", w, dt, "cuda") for p, w in zip(FFN_UP, w_up)]
    f_dn = [generate_factor(*p, "kernel", w, dt, "cuda") for p, w in zip(FFN_DOWN, w_dn)]
    n_in, n_hid = 384, 1536
    b_up = (torch.randn(n_hid, generator=gen) * 0.1).to(dt).cuda()
    b_dn = (torch.randn(n_in, generator=gen) * 0.1).to(dt).cuda()
    n_sets = 8
    shape = lambda n: (n, BATCH) if bs_last else (BATCH, n)
    xs = []
    for i in range(n_sets):
        x = torch.randn(BATCH, n_in, generator=gen)
        xs.append((x.t().contiguous() if bs_last else x).to(dt).cuda())
    hid = [torch.empty(shape(n_hid), dtype=dt, device="cuda") for _ in range(n_sets)]
    outs = [torch.empty(shape(n_in), dtype=dt, device="cuda") for _ in range(n_sets)]
    ws = torch.empty(2 * (n_hid * BATCH * 4 + 256), dtype=torch.uint8, device="cuda")

    def up(j):
        return Kernel.chain_forward(xs[j], f_up, FFN_UP, bs_last, fuse=True, workspace=ws, bias=b_up, act="gelu",
                                    out=hid[j])

    def down(j):
        return Kernel.chain_forward(hid[j], f_dn, FFN_DOWN, bs_last, fuse=True, workspace=ws, bias=b_dn, out=outs[j])

    def ffn(j):
        up(j)
        return down(j)

    res = {"name": "ffn_vit_s", "precision": prec, "bs_last": bs_last, "patterns_up": FFN_UP,
           "patterns_down": FFN_DOWN, "batch": BATCH}
    res["ffn_us"] = time_launches(ffn, n_sets, steps, warmup) * 1e6
    res["up_bias_gelu_us"] = time_launches(up, n_sets, steps, warmup) * 1e6
    res["down_bias_us"] = time_launches(down, n_sets, steps, warmup) * 1e6
    # the down-projection's factors on their own (input of the second = output of the first)
    mid = [torch.empty(shape(FFN_DOWN[0][0] * FFN_DOWN[0][1] * FFN_DOWN[0][3]), dtype=dt, device="cuda")
           for _ in range(n_sets)]
    res["down_factors"] = []
    for i, (p, src, dst) in enumerate(((FFN_DOWN[0], hid, mid), (FFN_DOWN[1], mid, outs))):
        def run(j, p=p, src=src, dst=dst, i=i):
            Kernel.forward(src[j], f_dn[i], bs_last, *p, out=dst[j])

        sec = time_launches(run, n_sets, steps, warmup)
        roof = factor_roofline(BATCH, p, dt, dt, dt, sec)
        res["down_factors"].append({"pattern": p, "us": sec * 1e6, "bound": roof["bound"],
                                    "roofline_frac": roof["frac"], "floor_us": roof["floor_us"]})
    # parity of the whole block on sampled rows
    from oracle import ks_oracle as O
    import numpy as np

    ffn(0)
    torch.cuda.synchronize()
    rows = np.unique(np.concatenate([np.arange(0, BATCH, 397), np.arange(BATCH - 2, BATCH)]))
    xr = xs[0].cpu().double().numpy()
    xsub = xr[:, rows] if bs_last else xr[rows, :]
    wr_up = [w.to(dt).double().numpy() for w in w_up]
    wr_dn = [w.to(dt).double().numpy() for w in w_dn]
    bu, bd = b_up.cpu().double().numpy(), b_dn.cpu().double().numpy()
    h = O.chain_apply(wr_up, xsub, bs_last) + (bu[:, None] if bs_last else bu)
    h = torch.nn.functional.gelu(torch.from_numpy(h)).to(dt).double().numpy()  # the hidden tensor is stored in `dt`
    z = O.chain_apply(wr_dn, h, bs_last) + (bd[:, None] if bs_last else bd)
    yh = outs[0].float().cpu().numpy()
    ysub = yh[:, rows] if bs_last else yh[rows, :]
    res["rel_fro_error"] = O.rel_fro_error(ysub, z)
    res["tolerance"] = TOL[prec]
    res["parity_ok"] = bool(res["rel_fro_error"] <= TOL[prec])
    return res


def bench_backward(name, pattern, prec, bs_last, steps, warmup):
    """µs of the input gradient (dX = K^T dY, on the forward kernels with transposed blocks) and of
    the weight gradient (dW = sum over the batch of dY x X^T per block, per-split partial sums added
    in a fixed order) of one factor at B = 25 088, each against its own roofline: both move the two
    batch-sized operands once and do the forward's 2*B*a*b*c*d flops."""
    from ksmm_amd import Kernel, generate_factor, _lib
    from ksmm_amd.kernel import dtype_code
    from ksmm_amd.roofline import HBM_PEAK_GBS, MFMA_PEAK_TFLOPS

    HBM_BW = HBM_PEAK_GBS * 1e9
    peak = MFMA_PEAK_TFLOPS[prec] * 1e12

    a, b, c, d = pattern
    dt = DT[prec]
    es = torch.empty(0, dtype=dt).element_size()
    gen = torch.Generator().manual_seed(SEED + 7)
    (w4,) = make_weights([pattern], None, gen)
    fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
    n_sets = max(2, min(8, int(math.ceil(1.2e9 / (2 * max(a * c * d, a * b * d) * BATCH * 4)))))
    shape_x = (a * c * d, BATCH) if bs_last else (BATCH, a * c * d)
    shape_y = (a * b * d, BATCH) if bs_last else (BATCH, a * b * d)
    xs = [torch.randn(shape_x, generator=gen).to(dt).cuda() for _ in range(n_sets)]
    dys = [torch.randn(shape_y, generator=gen).to(dt).cuda() for _ in range(n_sets)]
    lib = _lib.load()
    need = lib.ksmm_factor_backward_workspace(BATCH, a, b, c, d, dtype_code(dt), int(bs_last))
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    nnz = a * b * c * d
    flops = 2.0 * BATCH * nnz
    nbytes = BATCH * (a * c * d + a * b * d) * es + nnz * es
    floor = max(nbytes / HBM_BW, flops / peak)
    out = {"name": name, "pattern": pattern, "precision": prec, "bs_last": bs_last, "workspace_bytes": int(need),
           "bytes": nbytes, "flops": flops, "floor_us": floor * 1e6,
           "bound": "hbm" if nbytes / HBM_BW >= flops / peak else "mfma"}
    for key, kw in (("dx", {"need_weight": False}), ("dw", {"need_input": False})):
        def run(j):
            Kernel.backward(dys[j], xs[j], fac, bs_last, a, b, c, d, workspace=ws, **kw)

        sec = time_launches(run, n_sets, steps, warmup)
        out[key + "_us"] = sec * 1e6
        out[key + "_roofline_frac"] = floor / sec
        out[key + "_gbs"] = nbytes / sec / 1e9
        out[key + "_tflops"] = flops / sec / 1e12
    return out


_STREAM_COPY_US = {}


def same_bytes_stream_copy_us(total_bytes, steps, warmup):
    """µs the streaming copy of the benchmark library takes to move `total_bytes` (half read,
    half written) with the buffer rotation of the factor timings; one measurement per size."""
    import ctypes

    from ksmm_amd import _lib, bench_lib

    half = (total_bytes // 2 + 15) // 16 * 16
    if half not in _STREAM_COPY_US:
        lib = bench_lib.load()
        n_sets = max(2, min(8, int(math.ceil(1.2e9 / (2 * half)))))
        src = [torch.empty(half, dtype=torch.uint8, device="cuda").random_() for _ in range(n_sets)]
        dst = [torch.empty_like(t) for t in src]

        def run(j):
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check(lib.ksbench_stream_copy(src[j].data_ptr(), dst[j].data_ptr(), half, 2048, stream))

        _STREAM_COPY_US[half] = time_launches(run, n_sets, max(20, steps // 2), max(5, warmup // 2)) * 1e6
        del src, dst
    return _STREAM_COPY_US[half]


def copy_reference(steps, warmup):
    """Plain elementwise stream (y = x + 1) over the headline workload's bytes (77 MB in, 77 MB out) with
    the same buffer rotation and timing: what this particular GPU sustains for the simplest
    read+write stream, next to the 8 TB/s datasheet figure."""
    n_sets = 4
    src = [torch.randn(768, BATCH, device="cuda") for _ in range(n_sets)]
    dst = [torch.empty_like(t) for t in src]

    def run(j):
        torch.add(src[j], 1.0, out=dst[j])  # one elementwise kernel: 1 read + 1 write stream

    sec = time_launches(run, n_sets, steps, warmup)
    nbytes = 2 * src[0].numel() * 4
    return {"us": sec * 1e6, "gbs": nbytes / sec / 1e9, "frac_of_8tbs": nbytes / sec / 8e12,
            "bytes": nbytes, "kernel": "torch.add(x, 1, out=y) elementwise kernel"}


def stream_copy_reference(steps, warmup):
    """A hand-written streaming copy of the headline workload's bytes (ksbench_stream_copy: a
    persistent grid, four 16-byte vectors per thread and round, non-temporal loads and stores),
    best of a few grid sizes: the fastest way found to move these bytes on this GPU, i.e. the
    ceiling a bandwidth-bound factor is measured against next to the 8 TB/s datasheet figure."""
    import ctypes

    from ksmm_amd import _lib, bench_lib

    lib = bench_lib.load()
    n_sets = 4
    src = [torch.randn(768, BATCH, device="cuda") for _ in range(n_sets)]
    dst = [torch.zeros_like(t) for t in src]
    nbytes = 2 * src[0].numel() * 4
    res = {"bytes": nbytes, "kernel": "ksbench_stream_copy: persistent grid x 256 threads, 4 x 16 B per thread "
                                      "and round, non-temporal loads and stores"}
    best = None
    for wgs in (1024, 2048, 4096):
        def run(j):
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check(lib.ksbench_stream_copy(src[j].data_ptr(), dst[j].data_ptr(), src[j].numel() * 4, wgs, stream))

        dst[0].zero_()
        run(0)
        torch.cuda.synchronize()
        if not torch.equal(src[0], dst[0]):
            raise RuntimeError("stream copy: output differs from input")
        sec = time_launches(run, n_sets, steps, warmup)
        res["workgroups_%d_us" % wgs] = sec * 1e6
        best = sec if best is None else min(best, sec)
    res.update({"us": best * 1e6, "gbs": nbytes / best / 1e9, "frac_of_8tbs": nbytes / best / 8e12})
    return res


def tiled_copy_reference(steps, warmup):
    """A tile-at-a-time copy of the headline operand (ksbench_tilecopy_probe, no arithmetic): one
    workgroup per tile of 48 rows, every load of the tile issued before its first store, which is
    what a register-stationary block kernel has to do.  Timed with the tile addresses of the
    headline factor (1,48,48,16), fp32, bs_last (48 rows 16 apart, pieces of 256 B .. 4 KB per
    row) and, with the same tile size, on linear memory (48 consecutive 1 KB pieces): the two
    differ little, both are well above the streaming copy (`copy_reference`), so the gap is the
    price of moving whole tiles, not of the strided layout."""
    import ctypes

    from ksmm_amd import _lib, bench_lib

    lib = bench_lib.load()
    n_sets = 4
    src = [torch.randn(768, BATCH, device="cuda") for _ in range(n_sets)]
    dst = [torch.zeros_like(t) for t in src]
    nbytes = 2 * src[0].numel() * 4
    res = {"bytes": nbytes, "kernel": "ksbench_tilecopy_probe: tiles of 48 rows x tile_bytes, rows 16 apart; "
                                      "linear: the same tiles as 48 consecutive pieces of linear memory"}
    cases = [("tile_%dB" % tb, (BATCH * 4, 1, 48, 16, tb)) for tb in (256, 1024, 4096)]
    cases.append(("linear_tile_1024B", (1024, 768 * BATCH * 4 // 1024 // 48, 48, 1, 1024)))
    for key, (row_bytes, pa, rows, pd, tile_bytes) in cases:
        def run(j):
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check(lib.ksbench_tilecopy_probe(src[j].data_ptr(), dst[j].data_ptr(), row_bytes, pa, rows, pd,
                                               tile_bytes, stream))

        dst[0].zero_()
        run(0)
        torch.cuda.synchronize()
        if not torch.equal(src[0], dst[0]):
            raise RuntimeError("tile copy probe: output differs from input")
        sec = time_launches(run, n_sets, steps, warmup)
        res[key] = {"us": sec * 1e6, "gbs": nbytes / sec / 1e9, "frac_of_8tbs": nbytes / sec / 8e12}
    return res


def mfma_reference():
    """Rate at which the matrix cores multiply operands held in registers (no memory traffic at
    all), with all-ones and with random operands: what this GPU sustains next to the datasheet
    peaks the MFMA-bound rooflines are priced against (fp16 2516.6, fp32 157.3 TFLOP/s)."""
    import ctypes

    from ksmm_amd import _lib, bench_lib
    from ksmm_amd.kernel import dtype_code

    lib = bench_lib.load()
    out = torch.empty(lib.ksbench_mfma_probe_bytes(), dtype=torch.uint8, device="cuda")
    res = {}
    for name, dt, iters in (("f16_32x32x16", dtype_code(torch.float16), 20000),
                            ("f32_16x16x4", dtype_code(torch.float32), 20000)):
        for random in (0, 1):
            flops = ctypes.c_double(0.0)

            def run(_):
                stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                _lib.check(lib.ksbench_mfma_probe(dt, iters, random, out.data_ptr(), out.numel(), ctypes.byref(flops), stream))

            sec = time_launches(run, 1, 3, 1)
            res["%s_%s_tflops" % (name, "random" if random else "ones")] = flops.value / sec / 1e12
    return res


def cpu_baseline(patterns, bs_last, budget_s=12.0, min_run_time=0.25, dtype=torch.float32, batch=BATCH, bound=None):
    """The reference's algo='bmm' CPU algorithm (restated in oracle/) on all host cores;
    protocol of the reference's ksmm_time.py: blocked_autorange(min_run_time=0.25), re-run with
    11*max(mean, median) when fewer than 10 runs fit.  ``dtype``: the type torch.bmm runs in
    (fp16 is what the reference's CPU path does for dtype=float16); ``batch`` below the full
    25 088 columns bounds the slow fp16 leg (columns are independent: time scales with them)."""
    import torch.utils.benchmark as tb
    from oracle import ks_oracle as O

    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or os.cpu_count() or 1
    cores = min(cores, os.cpu_count() or cores)
    torch.set_num_threads(cores)
    gen = torch.Generator().manual_seed(SEED)
    ws4 = make_weights(patterns, bound, gen)
    wb = [torch.from_numpy(O.pack_bmm_format(w.numpy())).to(dtype) for w in ws4]
    in_size = patterns[0][0] * patterns[0][2] * patterns[0][3]
    x = torch.randn(batch, in_size, generator=gen).to(dtype)
    x = x.t().contiguous() if bs_last else x
    with torch.no_grad():
        timer = tb.Timer(stmt="f(wb, x, patterns, bs_last)",
                         globals={"f": O.torch_bmm_chain, "wb": wb, "x": x, "patterns": patterns,
                                  "bs_last": bs_last}, num_threads=torch.get_num_threads())
        m = timer.blocked_autorange(min_run_time=min_run_time)
        if m.number_per_run <= 10:
            m = timer.blocked_autorange(min_run_time=min(budget_s, 11 * max(m.mean, m.median)))
        calls = len(m.times) * m.number_per_run
        if len(m.times) < 5 and m.median * m.number_per_run * 5 <= budget_s:
            # blocked_autorange may return one block: time a few more of the same size so that the
            # spread over blocks (iqr) is a spread
            per_block = m.number_per_run
            blocks = [timer.timeit(per_block) for _ in range(5)]
            m = tb.Measurement.merge(blocks)[0]  # (times become per-call means of each block)
            calls = 5 * per_block
    name = str(dtype).replace("torch.", "")
    return {"value": m.median * 1e6, "unit": "us", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%s (B=%d of %d, %s, bs_last=%s, patterns=%s), %d timed calls of torch.bmm "
                      "+ permute copies in %d blocks; median of the blocks"
                      % ("full workload" if batch == BATCH else "a share of the batch columns", batch, BATCH, name,
                         bs_last, patterns, calls, len(m.times)),
            "mean_us": m.mean * 1e6, "iqr_us": m.iqr * 1e6, "host_cpu_count": os.cpu_count()}


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "bench_hbm_traffic.txt")


def measured_traffic(name, algo, variant):
    """HBM bytes per launch of a benchmark kernel from the tracked counter summary
    profiles/bench_hbm_traffic.txt (counters cannot be collected from inside a timed run).  Lines:
        CALIB fetch=<FETCH_SIZE KiB read per KiB a copy kernel of known size fetches> write=<same for WRITE_SIZE>
        TRAFFIC <config> factor=<i> algo=<a> variant=<hex> fetch_kib=<per dispatch> write_kib=<per dispatch>
    Returns None when there is no line for this configuration with the kernel (algo, variant) that
    ran: a figure measured on another kernel does not carry over."""
    try:
        lines = open(TRAFFIC_FILE).read().splitlines()
    except OSError:
        return None
    calib = None
    for l in lines:
        f = dict(t.split("=", 1) for t in l.split()[1:] if "=" in t)
        if l.startswith("CALIB"):
            calib = (float(f["fetch"]), float(f["write"]))
        elif l.startswith("TRAFFIC") and calib and l.split()[1] == name and int(f["factor"]) == 0 \
                and int(f["algo"]) == algo and int(f["variant"], 16) == variant:
            return int((float(f["fetch_kib"]) / calib[0] + float(f["write_kib"]) / calib[1]) * 1024)
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--all", type=int, default=1, help="also time the other configurations")
    ap.add_argument("--cpu", type=int, default=1, help="time the CPU baseline")
    ap.add_argument("--copy-calib", type=int, default=0,
                    help="also run N plain device copies of 77 MB (counter calibration for profiling runs)")
    ap.add_argument("--backward", type=int, default=1,
                    help="also time the backward pass (input and weight gradients) of the headline factor and of "
                         "the ViT-B up-projection factors")
    ap.add_argument("--ffn", type=int, default=1,
                    help="also time the feed-forward block of the reference's ViT-S benchmark (up + bias + GELU, "
                         "down + bias) in its default layout")
    ap.add_argument("--factor", default=None,
                    help="time one factor only, e.g. fp16:last:1,768,192,16 (per-kernel profiling runs); "
                         "prints that configuration's JSON instead of the headline line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build is single-GPU (the KS path shards on the batch axis without "
              "communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from ksmm_amd import _lib
    from ksmm_amd.roofline import factor_roofline

    _lib.load()  # fails loudly if the HIP library is missing
    t_start = time.time()
    if args.copy_calib:
        # a copy kernel of known size (read 77 070 336 B, write 77 070 336 B) so that HBM byte
        # counters of a profiling run can be scaled
        src = torch.randn(768, BATCH, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(args.copy_calib):
            torch.add(src, 1.0, out=dst)  # one elementwise kernel per call: 1 read + 1 write stream
        torch.cuda.synchronize()
    if args.factor:
        prec, layout, pat = args.factor.split(":")
        pattern = tuple(int(v) for v in pat.split(","))
        res = bench_config("factor", [pattern], prec, layout == "last", None, args.steps, args.warmup)
        print(json.dumps(res))
        return
    head = bench_config(*CONFIGS[0], steps=args.steps, warmup=args.warmup)
    sec = head["factors"][0]["us"] / 1e6
    roof = factor_roofline(BATCH, CONFIGS[0][1][0], torch.float32, torch.float32, torch.float32, sec)
    hf = head["factors"][0]
    traffic = measured_traffic(CONFIGS[0][0], hf["algo"], hf["variant"])
    others = []
    if args.all:
        for cfg in CONFIGS[1:]:
            others.append(bench_config(*cfg, steps=max(20, args.steps // 2), warmup=max(5, args.warmup // 2)))
    copy_ref = copy_reference(max(20, args.steps // 2), max(5, args.warmup // 2))
    stream_ref = stream_copy_reference(max(20, args.steps // 2), max(5, args.warmup // 2))
    tiled_ref = tiled_copy_reference(max(20, args.steps // 2), max(5, args.warmup // 2))
    mfma_ref = mfma_reference()
    backward = []
    if args.backward:
        bsteps, bwarm = max(10, args.steps // 4), max(3, args.warmup // 4)
        backward.append(bench_backward("C2_bs_last", (1, 48, 48, 16), "fp32", True, bsteps, bwarm))
        backward.append(bench_backward("C4_vit_b_up_f0", (12, 64, 64, 1), "fp16", False, bsteps, bwarm))
        backward.append(bench_backward("C4_vit_b_up_f1", (1, 1536, 384, 2), "fp16", False, bsteps, bwarm))
    ffn = bench_ffn(max(10, args.steps // 4), max(3, args.warmup // 4)) if args.ffn else None
    cpu = cpu_baseline(CONFIGS[0][1], True) if args.cpu else None
    if args.cpu:
        # the same CPU algorithm beside every other configuration (fp32 on the host, whatever the
        # device precision; a short sample each so that the whole run stays within minutes)
        head["cpu_bmm_us"], head["cpu_cores"] = cpu["value"], cpu["cores"]
        for cfg, res in zip(CONFIGS[1:], others):
            c = cpu_baseline(cfg[1], cfg[3], budget_s=4.0, min_run_time=0.1, bound=cfg[4])
            res["cpu_bmm_us"], res["cpu_cores"], res["cpu_sample"] = c["value"], c["cores"], c["sample"]
            if cfg[2] == "fp16":
                # the reference's CPU path in the configuration's own type: torch.bmm in fp16, on an
                # eighth of the batch columns (slow on the host; the time is per call of that share)
                share = BATCH // 8
                h = cpu_baseline(cfg[1], cfg[3], budget_s=3.0, min_run_time=0.1, dtype=torch.float16, batch=share)
                res["cpu_bmm_fp16_us_share"], res["cpu_bmm_fp16_share_columns"] = h["value"], share
                res["cpu_bmm_fp16_us_scaled_to_full_batch"] = h["value"] * (BATCH / share)
                res["cpu_fp16_sample"] = h["sample"]
    line = {
        "metric": "us_per_ks_factor", "value": head["factors"][0]["us"], "unit": "us",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seed %d): x~N(0,1), W~U(-1/sqrt(c),1/sqrt(c))" % SEED,
        "config": {"workload": "single KS factor (1,48,48,16) 768->768, fp32, bs_last, B=25088",
                   "batch": BATCH, "pattern": [1, 48, 48, 16], "layout": "bs_last"},
        "roofline": {"bound": roof["bound"], "achieved": roof["achieved"], "peak": roof["peak"],
                     "unit": roof["unit"], "frac": roof["frac"], "traffic": traffic},
        "cpu_baseline": cpu,
        "copy_reference": copy_ref,
        "stream_copy_reference": stream_ref,
        "tiled_copy_reference": tiled_ref,
        "mfma_reference": mfma_ref,
        "parity": {"rel_fro_error": head.get("rel_fro_error"), "tolerance": head.get("tolerance"),
                   "ok": head.get("parity_ok")},
        "configs": [head] + others,
        "backward": backward,
        "ffn": ffn,
        "wall_s": time.time() - t_start,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
