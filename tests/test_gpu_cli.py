"""GPU checks around the kernel path that go through its user-facing wrappers: the timing CLI
with ``--algo kernel --device cuda --correctness`` (the reference's ksmm_time.py:148-164 check),
``get_dense_product() @ x`` against the kernel output, rows of the measured table of every kernel
family at the batch size they were measured at, and KSLinear with gradients enabled."""
import csv

import numpy as np
import pytest
import torch

from tests.util import TOL, TORCH_DTYPE, oracle_chain, round_to, sample_columns, seeded_input, seeded_weights
from oracle import ks_oracle as O

pytestmark = pytest.mark.gpu

# what the contract allows against a reference that does not share the kernel's operand rounding
CLI_TOL = {"fp32": 1e-5, "fp16": 2e-3, "fp8": 5e-2}
VIT_S_UP = ["6,64,64,1", "1,768,192,2"]        # scripts/2_benchmark_ksvit_time.sh:48-50
VIT_S_DOWN = ["6,64,256,1", "1,128,128,3"]


def _cli(argv):
    from ksmm_amd import bench_csv

    bench_csv.main.last_relative_error = None
    bench_csv.main(argv)
    assert bench_csv.main.last_relative_error is not None
    return bench_csv.main.last_relative_error


def _rows(path):
    with open(path, newline="") as f:
        return list(csv.DictReader(f))


@pytest.mark.parametrize("bs_last", [0, 1])
@pytest.mark.parametrize("prec", ["fp32", "fp16", "fp8"])
def test_cli_correctness_on_the_kernel_path(prec, bs_last, tmp_path, capsys):
    """`--algo kernel --device cuda --correctness` on the README chain: the printed relative
    error (layer output against get_dense_product() @ x in fp32 on the CPU) is within the
    tolerance of the precision, and the CSV gets its row."""
    from ksmm_amd import bench_csv

    out = tmp_path / "times.csv"
    err = _cli(["--saving-csv", str(out), "--patterns"] + VIT_S_UP +
               ["--algo", "kernel", "--device", "cuda", "--precision", prec, "--bs-last", str(bs_last),
                "--batch-size", "2048", "--correctness", "--min-run-time", "0.02"])
    assert "Relative error = " in capsys.readouterr().out
    assert err <= CLI_TOL[prec], (prec, bs_last, err)
    rows = _rows(out)
    assert len(rows) == 1 and list(rows[0]) == bench_csv.COLUMNS
    r = rows[0]
    assert r["algo"] == "kernel" and r["precision"] == prec and r["batch-size"] == "2048"
    assert r["bs_position"] == ("bs_last" if bs_last else "bs_first")
    assert r["pattern"] == "[[6, 64, 64, 1], [1, 768, 192, 2]]"
    assert float(r["mean"]) > 0 and float(r["median"]) > 0


@pytest.mark.parametrize("prec", ["fp16", "fp8", "fp32"])
def test_cli_feed_forward_granularity_on_the_kernel_path(prec, tmp_path):
    """`--granularity ffn` with the reference's ViT-S patterns in its default layout (bs_last 0):
    up + bias + GELU and down + bias, both inside the kernels, against the dense reference."""
    out = tmp_path / "ffn.csv"
    argv = ["--saving-csv", str(out), "--granularity", "ffn", "--patterns_up"] + VIT_S_UP + ["--patterns_down"] + \
        VIT_S_DOWN + ["--algo", "kernel", "--device", "cuda", "--precision", prec, "--bs-last", "0",
                      "--batch-size", "1576", "--correctness", "--min-run-time", "0.02"]
    err = _cli(argv)
    assert err <= CLI_TOL[prec], (prec, err)
    (r,) = _rows(out)
    assert r["pattern"].startswith("ffn:") and r["algo"] == "kernel" and r["bs_position"] == "bs_first"
    # the same configuration again replaces its row instead of adding one
    _cli(argv)
    assert len(_rows(out)) == 1


@pytest.mark.parametrize("bs_last", [True, False])
@pytest.mark.parametrize("prec", ["fp32", "fp16", "fp8"])
def test_kernel_output_matches_get_dense_product(prec, bs_last):
    """KSLinear(algo='kernel').get_dense_product() @ x (ksmm_time.py:148-157) against the layer's
    own output; for e4m3 the dense product is that of the dequantised factors."""
    from ksmm_amd import KSLinear

    patterns = [(2, 64, 32, 2), (1, 96, 128, 2), (4, 16, 48, 1)]
    ws4 = seeded_weights(patterns, seed=61)
    dt = TORCH_DTYPE[prec]
    ksl = KSLinear(patterns, weights=ws4, bias=False, algo="kernel", dtype=dt, bs_last=bs_last, device="cuda")
    x = seeded_input(ksl.in_size, 520, bs_last, seed=62)
    dense = ksl.get_dense_product(torch.float32).cpu().double()
    assert dense.shape == (ksl.out_size, ksl.in_size)
    # the dense product is the oracle's dense form of the rounded factors
    wr = [round_to(w, prec)[0] for w in ws4]
    assert O.rel_fro_error(dense.numpy(), O.chain_dense(wr)) <= 1e-6
    if prec == "fp8":
        xr, xq, xs = round_to(x, prec)
        y = ksl(xq.cuda(), x_scale=xs)
    else:
        xr = round_to(x, prec)[0]
        y = ksl(x.to(dt).cuda())
    want = dense.numpy() @ xr if bs_last else xr @ dense.numpy().T
    assert O.rel_fro_error(y.float().cpu().numpy(), want) <= TOL[prec], (prec, bs_last)


def _table_sample():
    """Two rows (the smallest and the largest that fits the size cap) of the measured table per
    (family, sub-family, element types, layout)."""
    from ksmm_amd.kernel import tuned_table

    groups = {}
    for row in tuned_table():
        a, b, c, d, combo, bs_last, algo, variant = row
        if variant < 0:
            continue
        if a * max(b, c) * d > 8192:  # 25088 columns of that many features: at most 0.8 GB in fp32
            continue
        sub = (variant >> 24) & 15 if algo == 3 else (1 if variant >= 1000 else 0)
        groups.setdefault((algo, sub, combo, bs_last), []).append(row)
    picked = []
    for key in sorted(groups):
        rows = sorted(groups[key], key=lambda r: r[0] * r[1] * r[2] * r[3])
        picked.append(rows[0])
        if len(rows) > 1:
            picked.append(rows[-1])
    return picked


@pytest.mark.parametrize("combo", [0, 1, 2])
@pytest.mark.parametrize("bs_last", [1, 0])
def test_tuned_table_rows_of_every_family_at_full_batch(combo, bs_last):
    """Rows of every kernel family the measured table names (wave, rows, k-loop, weight-stationary,
    stream, grouped batch-size-first, GEMM and persistent GEMM tiles), small and large blocks, at
    the batch the table was measured at (25 088): the automatic choice must be the row's kernel
    and agree with the oracle on sampled batch columns."""
    from ksmm_amd import Kernel, generate_factor
    from ksmm_amd.kernel import query_tile

    prec = {0: "fp32", 1: "fp16", 2: "fp8"}[combo]
    dt = TORCH_DTYPE[prec]
    batch = 25088
    cols = sample_columns(batch, step=199)
    rows = [r for r in _table_sample() if r[4] == combo and r[5] == bs_last]
    assert len(rows) >= 2, rows
    seen = set()
    for a, b, c, d, _, _, algo, variant in rows:
        pattern = (a, b, c, d)
        tile = query_tile(batch, pattern, dt, None, bool(bs_last))
        assert tile == query_tile(batch, pattern, dt, None, bool(bs_last), algo, variant), (pattern, tile)
        (w4,) = seeded_weights([pattern], seed=71)
        x = seeded_input(a * c * d, batch, bool(bs_last), seed=72)
        wr, wq, ws = round_to(w4, prec)
        if prec == "fp8":
            xq, xs_t = __import__("ksmm_amd").quantize_fp8(x)
            xs = float(xs_t)
            xin, scale = xq.cuda(), ws * xs
            xsub = xq[:, cols] if bs_last else xq[cols, :]
            xr = xsub.to(torch.float32).double().numpy() * xs
            fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), dt, "cuda")
        else:
            xin, scale = x.to(dt).cuda(), 1.0
            xsub = xin[:, cols] if bs_last else xin[cols, :]
            xr = xsub.cpu().double().numpy()
            fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
        print("table row", pattern, prec, "bs_last" if bs_last else "bs_first", algo, hex(variant), flush=True)
        y = Kernel.forward(xin, fac, bool(bs_last), a, b, c, d, dtype=dt, scale=scale)
        torch.cuda.synchronize()
        ysub = (y[:, cols] if bs_last else y[cols, :]).float().cpu().numpy()
        z = O.ks_apply_einsum(wr, xr, bool(bs_last))
        err = O.rel_fro_error(ysub, z)
        assert err <= TOL[prec], (pattern, prec, bs_last, algo, hex(variant), err)
        assert bool(torch.isfinite(y.float()).all())
        seen.add((algo, (variant >> 24) & 15 if algo == 3 else 0))
        del x, xin, y, fac
    print("families covered", sorted(seen), flush=True)


@pytest.mark.parametrize("bs_last", [True, False])
@pytest.mark.parametrize("prec", ["fp16", "fp32"])
def test_kslinear_with_gradients_enabled_matches_the_chain_launcher(prec, bs_last):
    """A freshly built KSLinear(algo='kernel') called with gradients enabled takes the per-factor
    autograd path (bias and activation as PyTorch operations); it must give what the chain
    launcher gives under no_grad, and what the oracle gives, with and without bias / GELU."""
    from ksmm_amd import KSLinear

    patterns = [(2, 64, 32, 2), (1, 96, 128, 2)]
    ws4 = seeded_weights(patterns, seed=91)
    dt = TORCH_DTYPE[prec]
    for bias, act in ((False, None), (True, None), (True, "gelu")):
        ksl = KSLinear(patterns, weights=ws4, bias=bias, algo="kernel", dtype=dt, bs_last=bs_last, device="cuda",
                       act=act)
        x = seeded_input(ksl.in_size, 264, bs_last, seed=92)
        xin = x.to(dt).cuda()
        with torch.enable_grad():
            assert all(f.requires_grad for f in ksl.factors)
            y_grad = ksl(xin)
            assert y_grad.requires_grad
        with torch.no_grad():
            y_chain = ksl(xin)
        z = oracle_chain([round_to(w, prec)[0] for w in ws4], round_to(x, prec)[0], bs_last)
        if bias:
            bvec = ksl.bias.detach().double().cpu().numpy().reshape(-1)
            z = z + (bvec[:, None] if bs_last else bvec[None, :])
        if act:
            z = torch.nn.functional.gelu(torch.from_numpy(z)).numpy()
        for name, y in (("grad", y_grad), ("chain", y_chain)):
            err = O.rel_fro_error(y.detach().float().cpu().numpy(), z)
            assert err <= TOL[prec], (prec, bs_last, bias, act, name, err)
