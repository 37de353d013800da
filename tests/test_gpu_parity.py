"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Tolerances are relative Frobenius errors: fp32 1e-5, fp16 2e-3, fp8 5e-3
(fp8: oracle on the dequantised operands; the contract allows 5e-2)."""
import numpy as np
import pytest
import torch

from tests.util import (TOL, TORCH_DTYPE, oracle_chain, round_to, sample_columns, seeded_input,
                        seeded_weights)
from oracle import ks_oracle as O

pytestmark = pytest.mark.gpu

ALGO = {"auto": 0, "generic": 1, "wave": 2, "tile": 3}

SMALL_PATTERNS = [
    (2, 3, 5, 4), (1, 4, 3, 2), (3, 2, 2, 1), (1, 1, 1, 1), (4, 1, 3, 2),      # ragged
    (1, 16, 16, 1), (2, 16, 16, 3), (1, 48, 48, 16), (6, 64, 64, 1), (1, 16, 16, 64),
    (16, 16, 16, 4), (64, 16, 16, 1), (2, 32, 64, 2), (1, 64, 32, 4), (3, 48, 16, 2),
    (1, 96, 96, 2), (1, 128, 128, 1), (2, 192, 192, 1), (1, 256, 64, 2), (1, 80, 48, 1),
    (1, 17, 33, 2), (2, 16, 16, 16), (1, 64, 64, 4), (2, 48, 48, 8), (2, 64, 32, 2), (1, 128, 64, 4), (3, 32, 32, 8), (1, 256, 128, 2),
    (2, 48, 192, 2), (1, 64, 256, 2), (1, 192, 48, 3),
    (1, 64, 50, 3), (2, 32, 18, 1), (1, 128, 70, 2),                            # c not a multiple of the K tile
]
BATCHES = [1, 7, 64, 200, 1024]


def _run_factor(pattern, batch, prec, bs_last, algo, seed=0):
    from ksmm_amd import Kernel, generate_factor, _lib

    a, b, c, d = pattern
    (w4,) = seeded_weights([pattern], seed=seed)
    x = seeded_input(a * c * d, batch, bs_last, seed=seed + 1)
    wr, wq, ws = round_to(w4, prec)
    xr, xq, xs = round_to(x, prec)
    dt = TORCH_DTYPE[prec]
    if prec == "fp8":
        fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), dt, "cuda")
        xin = xq.cuda()
        scale = ws * xs
    else:
        fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
        xin = x.to(dt).cuda()
        scale = 1.0
    try:
        y = Kernel.forward(xin, fac, bs_last, a, b, c, d, dtype=dt, scale=scale, algo=ALGO[algo])
    except _lib.KsmmError as e:
        if e.status == -6 and algo != "auto" and algo != "generic":
            pytest.skip("family %s does not take this problem" % algo)
        raise
    torch.cuda.synchronize()
    z = O.ks_apply_einsum(wr, xr, bs_last)
    return y.float().cpu().numpy(), z


@pytest.mark.parametrize("algo", ["generic", "wave", "tile", "auto"])
@pytest.mark.parametrize("bs_last", [True, False])
@pytest.mark.parametrize("prec", ["fp32", "fp16", "fp8"])
def test_factor_small(prec, bs_last, algo):
    """All small patterns x batches for one (precision, layout, family): one test so the GPU
    process count stays at one and a failure names the case."""
    ran = 0
    for pattern in SMALL_PATTERNS:
        for batch in BATCHES:
            try:
                y, z = _run_factor(pattern, batch, prec, bs_last, algo)
            except pytest.skip.Exception:
                continue
            ran += 1
            err = O.rel_fro_error(y, z)
            assert y.shape == z.shape
            assert err <= TOL[prec], (pattern, batch, prec, bs_last, algo, err)
    print("test_factor_small", prec, bs_last, algo, "ran", ran, flush=True)
    # a family that starts refusing the shapes it is built for must not pass silently
    total = len(SMALL_PATTERNS) * len(BATCHES)
    floor = {"generic": total, "auto": total, "wave": 20 if bs_last else 10, "tile": 20 if bs_last else 8}[algo]
    assert ran >= floor, (prec, bs_last, algo, ran, floor)


def test_tile_bf_groups_of_blocks_forced():
    """Batch-size-first tile kernel on groups of DD neighbouring d_i out of a larger d (tile
    variant 3<<24 | i): every instance on shapes with d = DD, d a multiple of DD, several a_i,
    ragged batches, and the automatic choice with a bias, against the oracle."""
    from ksmm_amd import Kernel, generate_factor, _lib

    cases = [("fp16", (1, 128, 64, 16)), ("fp16", (2, 64, 32, 8)), ("fp16", (1, 64, 64, 24)), ("fp16", (1, 128, 32, 2)),
             ("fp16", (2, 64, 32, 4)), ("fp32", (1, 128, 32, 8)), ("fp32", (2, 64, 16, 12)), ("fp32", (1, 64, 32, 4)),
             ("fp32", (1, 128, 32, 2)), ("fp8", (1, 128, 64, 16)),
             # 5, 7 and 12 slabs of 16: whole and partial rounds of the two-slab register pipeline
             ("fp16", (1, 64, 80, 8)), ("fp16", (1, 192, 192, 16)), ("fp8", (2, 64, 112, 8)),
             ("fp32", (1, 64, 80, 8)), ("fp32", (1, 192, 192, 4)), ("fp32", (2, 64, 112, 12)),
             # d = 4 and 2 whole on the 8-wave instances (128-row tiles too)
             ("fp16", (1, 128, 48, 4)), ("fp16", (2, 256, 32, 2)), ("fp8", (2, 128, 32, 4)), ("fp8", (1, 128, 64, 2))]
    ran, strided = 0, 0
    for prec, pattern in cases:
        a, b, c, d = pattern
        dt = TORCH_DTYPE[prec]
        (w4,) = seeded_weights([pattern], seed=31)
        if prec == "fp8":  # e4m3 weights, fp16 input
            wr, wq, ws = round_to(w4, "fp8")
            fac, scale, x_dt, xprec = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), dt, "cuda"), ws, torch.float16, "fp16"
        else:
            wr = round_to(w4, prec)[0]
            fac, scale, x_dt, xprec = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda"), 1.0, dt, prec
        bias = (torch.rand(a * b * d, generator=torch.Generator().manual_seed(5)) - 0.5).to(x_dt)
        for batch in (520, 77):
            x = seeded_input(a * c * d, batch, False, seed=32)
            z = O.ks_apply_einsum(wr, round_to(x, xprec)[0], False)
            zb = z + bias.double().numpy()[None, :]
            for inst in list(range(40)) + list(range(53, 63)) + [69, 70]:
                try:
                    y = Kernel.forward(x.to(x_dt).cuda(), fac, False, a, b, c, d, scale=scale, algo=3,
                                       variant=(3 << 24) | inst)
                except _lib.KsmmError as e:
                    assert e.status == -6
                    continue
                ran += 1
                strided += d > 4 or (prec == "fp32" and d > 2 and d != 4)
                err = O.rel_fro_error(y.float().cpu().numpy(), z)
                assert err <= TOL[prec], (prec, pattern, batch, inst, err)
            # the automatic choice with the bias applied in the kernel
            y = Kernel.forward(x.to(x_dt).cuda(), fac, False, a, b, c, d, scale=scale, bias=bias.cuda())
            err = O.rel_fro_error(y.float().cpu().numpy(), zb)
            assert err <= TOL[prec], (prec, pattern, batch, "bias", err)
    print("tile_bf forced: ran", ran, "of which d > DD", strided, flush=True)
    # e4m3 input and weights (8-byte vectors of a group, decoded on their way to LDS)
    _forced_sweep([("fp8", False, (1, 128, 64, 16), 520), ("fp8", False, (2, 64, 80, 8), 77),
                   ("fp8", False, (1, 192, 192, 8), 1000), ("fp8", False, (1, 64, 32, 24), 203)],
                  [(3 << 24) | i for i in list(range(27, 41)) + [71]], 3, 9)
    # e4m3 input and weights, d = 2 or 4 whole (16-byte vectors of 8 or 4 k of every d_i)
    _forced_sweep([("fp8", False, (1, 256, 64, 2), 520), ("fp8", False, (2, 128, 96, 2), 77),
                   ("fp8", False, (1, 64, 128, 4), 203), ("fp8", False, (3, 32, 32, 4), 1000),
                   ("fp8", False, (1, 768, 192, 2), 264)],
                  [(3 << 24) | i for i in range(35, 41)] + [-1], 3, 14)
    # the same on 8 waves (instances 63..65)
    _forced_sweep([("fp8", False, (1, 256, 64, 2), 520), ("fp8", False, (2, 128, 96, 2), 77),
                   ("fp8", False, (1, 64, 128, 4), 203), ("fp8", False, (2, 128, 64, 4), 1000)],
                  [(3 << 24) | i for i in range(63, 66)], 3, 5)
    assert ran >= 40 and strided >= 12, (ran, strided)


def test_tile_bf_wide_groups_forced():
    """Batch-size-first tile kernel on 32 or 16 neighbouring blocks per workgroup (instances 41..52:
    slabs of 8 k, results staged through LDS): d whole and a multiple of the group, 32- and 64-row
    tiles, several a_i, ragged batches (the last batch tile partly empty, fewer rows than a tile),
    1 to 24 slabs; fp16, fp16 with e4m3 weights, e4m3 input and weights; with a bias."""
    from ksmm_amd import Kernel, generate_factor

    shapes = [((1, 64, 64, 32), 520), ((2, 64, 8, 32), 77), ((1, 32, 24, 64), 203), ((3, 96, 40, 32), 100),
              ((1, 64, 192, 16), 264), ((2, 128, 16, 48), 31), ((1, 192, 96, 64), 130), ((1, 64, 72, 128), 65)]
    variants = [(3 << 24) | i for i in range(41, 50)]
    for prec, min_ran in (("fp16", 14), ("hq", 14), ("fp8", 14)):
        _forced_sweep([(prec, False, p, n) for p, n in shapes], variants, 3, min_ran)
    # fp32: 16 or 8 blocks per workgroup (instances 50..52), 32- and 64-row tiles
    _forced_sweep([("fp32", False, p, n) for p, n in shapes + [((2, 64, 24, 8), 150), ((1, 96, 16, 16), 77)]],
                  [(3 << 24) | i for i in range(50, 53)], 3, 16)
    # fp32 groups of 4 on 128-row tiles (instances 66..68)
    _forced_sweep([("fp32", False, (1, 128, 48, 4), 520), ("fp32", False, (2, 256, 32, 8), 77),
                   ("fp32", False, (1, 128, 80, 12), 300)], [(3 << 24) | i for i in range(66, 69)], 3, 9)
    # the automatic choice with a bias (applied before the results are staged)
    from ksmm_amd.kernel import query_tile

    a, b, c, d = 1, 128, 48, 64
    batch = 4100
    pick = query_tile(batch, (a, b, c, d), torch.float16, torch.float16, False)
    assert pick["algo"] == 3 and pick["tile_d"] == 32 and pick["threads"] == 512, pick
    (w4,) = seeded_weights([(a, b, c, d)], seed=61)
    x = seeded_input(a * c * d, batch, False, seed=62)
    bias = (torch.rand(a * b * d, generator=torch.Generator().manual_seed(6)) - 0.5).half()
    fac = generate_factor(a, b, c, d, "kernel", w4, torch.float16, "cuda")
    z = O.ks_apply_einsum(round_to(w4, "fp16")[0], round_to(x, "fp16")[0], False) + bias.double().numpy()[None, :]
    y = Kernel.forward(x.half().cuda(), fac, False, a, b, c, d, bias=bias.cuda())
    err = O.rel_fro_error(y.float().cpu().numpy(), z)
    assert err <= TOL["fp16"], err


def test_wave_row_groups_forced():
    """fp32 wave instance for 32-row blocks forced on 64-row blocks (two row groups per block,
    variant 7 | tiles-per-wave << 8 | dealing << 16), with a_i, d_i > 1, ragged batches and a bias."""
    from ksmm_amd import Kernel, generate_factor, _lib
    from ksmm_amd.kernel import query_tile

    ran = 0
    for pattern in [(6, 64, 64, 1), (2, 64, 64, 3), (1, 32, 64, 2), (1, 96, 64, 2)]:
        a, b, c, d = pattern
        (w4,) = seeded_weights([pattern], seed=41)
        fac = generate_factor(a, b, c, d, "kernel", w4, torch.float32, "cuda")
        for batch in (1024, 200):
            x = seeded_input(a * c * d, batch, True, seed=42)
            z = O.ks_apply_einsum(w4.double().numpy(), x.double().numpy(), True)
            for variant in (7, 7 | (3 << 8), 7 | (2 << 8) | (1 << 16), 7 | (1 << 16 + 1)):
                t = query_tile(batch, pattern, torch.float32, None, True, algo=2, variant=variant)
                assert t["tile_m"] == 32, t
                y = Kernel.forward(x.cuda(), fac, True, a, b, c, d, algo=2, variant=variant)
                ran += 1
                assert O.rel_fro_error(y.cpu().numpy(), z) <= TOL["fp32"], (pattern, batch, variant)
    assert ran == 32


def test_gemm_kernels_forced():
    """Every instance of the direct-to-LDS GEMM sub-family (tile variant 4<<24 | i), forced on
    shapes with batch tails, several blocks per factor and d > 1."""
    from ksmm_amd import Kernel, generate_factor, _lib

    cases = [("fp16", True, (2, 256, 64, 3)), ("fp16", False, (2, 256, 64, 1)), ("fp16", False, (2, 256, 64, 2)),
             ("fp16", False, (1, 128, 128, 2)), ("fp32", True, (1, 256, 64, 2)), ("fp32", True, (2, 128, 32, 1)),
             # c not a multiple of the K tile (partial last slab), c below one K tile
             ("fp16", True, (2, 128, 70, 2)), ("fp16", True, (1, 64, 50, 3)), ("fp16", True, (1, 128, 18, 1)),
             ("fp32", True, (1, 128, 50, 2)), ("fp32", True, (2, 64, 18, 1)), ("fp32", True, (1, 64, 7, 2)),
             # b not a multiple of the tile (partly masked last TM-tile)
             ("fp16", True, (2, 96, 64, 3)), ("fp32", True, (1, 48, 48, 16)), ("fp32", True, (2, 80, 32, 2)),
             ("fp16", True, (1, 176, 96, 2))]
    ran = 0
    for prec, bs_last, pattern in cases:
        a, b, c, d = pattern
        for batch in (1000, 264):
            (w4,) = seeded_weights([pattern], seed=21)
            x = seeded_input(a * c * d, batch, bs_last, seed=22)
            dt = TORCH_DTYPE[prec]
            fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
            z = O.ks_apply_einsum(round_to(w4, prec)[0], round_to(x, prec)[0], bs_last)
            for inst in range(64):
                try:
                    y = Kernel.forward(x.to(dt).cuda(), fac, bs_last, a, b, c, d, algo=3, variant=(4 << 24) | inst)
                except _lib.KsmmError as e:
                    assert e.status == -6
                    continue
                ran += 1
                err = O.rel_fro_error(y.float().cpu().numpy(), z)
                assert err <= TOL[prec], (prec, bs_last, pattern, batch, inst, err)
    assert ran >= 24


def test_gemm_kernels_forced_e4m3():
    """The e4m3 instances of the GEMM sub-family (bytes straight into the fp8 MFMA): batch tails,
    several blocks, d > 1, c = 1, 2 and 3 slabs."""
    cases = [("fp8", True, (2, 256, 64, 3), 1008), ("fp8", True, (1, 128, 128, 2), 272),
             ("fp8", True, (2, 256, 192, 1), 528), ("fp8", True, (1, 256, 96, 2), 1024),
             ("fp8", True, (1, 128, 70, 2), 1008), ("fp8", True, (2, 256, 40, 1), 272), ("fp8", True, (1, 128, 9, 1), 64),
             ("fp8", True, (1, 192, 128, 2), 528), ("fp8", True, (2, 64, 72, 1), 1008),
             # partly masked last TM-tile
             ("fp8", True, (2, 96, 64, 3), 1008), ("fp8", True, (1, 48, 128, 4), 528)]
    _forced_sweep(cases, [(4 << 24) | i for i in range(21, 64)], 3, 26)


def _forced_sweep(cases, variants, algo, min_ran):
    """Every (case, variant) the family accepts must agree with the oracle; the others must be
    refused with KSMM_ERR_BAD_ALGO."""
    from ksmm_amd import Kernel, generate_factor, quantize_fp8, _lib

    ran = 0
    for prec, bs_last, pattern, batch in cases:
        a, b, c, d = pattern
        (w4,) = seeded_weights([pattern], seed=51)
        x = seeded_input(a * c * d, batch, bs_last, seed=52)
        if prec == "hq":  # fp16 activations, e4m3fn weights
            wq, ws = quantize_fp8(w4)
            fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), torch.float8_e4m3fn, "cuda")
            xin, scale, tol = x.half().cuda(), float(ws), TOL["fp16"]
            z = O.ks_apply_einsum((wq.to(torch.float32) * ws).double().numpy(), x.half().double().numpy(), bs_last)
        elif prec == "fp8":
            wr, wq, ws = round_to(w4, prec)
            xr, xq, xs = round_to(x, prec)
            fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), torch.float8_e4m3fn, "cuda")
            xin, scale, tol = xq.cuda(), ws * xs, TOL["fp8"]
            z = O.ks_apply_einsum(wr, xr, bs_last)
        else:
            dt = TORCH_DTYPE[prec]
            fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
            xin, scale, tol = x.to(dt).cuda(), 1.0, TOL[prec]
            z = O.ks_apply_einsum(round_to(w4, prec)[0], round_to(x, prec)[0], bs_last)
        for variant in variants:
            try:
                y = Kernel.forward(xin, fac, bs_last, a, b, c, d, scale=scale, algo=algo, variant=variant)
            except _lib.KsmmError as e:
                assert e.status == -6, (prec, bs_last, pattern, variant, e)
                continue
            ran += 1
            err = O.rel_fro_error(y.float().cpu().numpy(), z)
            assert err <= tol, (prec, bs_last, pattern, batch, hex(variant), err)
    assert ran >= min_ran, ran


def test_wave_instances_forced():
    """Every instance of the wave family (all four type combinations), one tile per wave and
    several, consecutive and round-robin tiles, with a ragged last tile."""
    shapes = [(2, 48, 48, 3), (2, 64, 64, 2), (3, 16, 16, 5), (2, 32, 32, 3), (1, 96, 96, 2), (2, 48, 192, 2),
              (1, 192, 48, 3)]
    cases = [(prec, True, p, 1040) for prec in ("fp32", "fp16", "hq", "fp8") for p in shapes]
    # tiles per wave / dealing: one tile, three consecutive, every n-th, balanced (automatic and 3
    # workgroups per block)
    variants = [inst | (it << 8) | (rr << 16) for inst in range(20)
                for it, rr in ((1, 0), (3, 0), (2, 1), (0, 2), (3, 2))]
    _forced_sweep(cases, variants, 2, 260)
    # the fp32 ring form (input rows through a per-wave LDS ring, stores spread over the next tile):
    # 1 .. 5 tiles per wave, 1 .. 8 waves per workgroup (bits 18-21), row groups of taller blocks,
    # batches of one vector, one tile, ragged last tiles
    ring_shapes = [(2, 48, 48, 3), (2, 64, 64, 2), (3, 16, 16, 5), (2, 32, 32, 3), (1, 96, 48, 2), (1, 128, 64, 2)]
    ring = [inst | (it << 8) | (w << 18) for inst in range(8, 19) for it in (0, 1, 2, 5) for w in (0, 1, 3, 8)]
    for batch in (4, 64, 1040, 8204):
        _forced_sweep([("fp32", True, p, batch) for p in ring_shapes], ring, 2, 100)


def test_row_kernel_instances_forced():
    """Every instance of the batch-size-first row kernel, full and ragged batch tiles."""
    shapes = [(2, 48, 48, 16), (1, 48, 48, 8), (2, 48, 48, 4), (1, 64, 64, 8), (2, 64, 64, 4), (1, 16, 16, 16),
              (3, 16, 16, 4), (2, 32, 32, 8),
              # all d blocks of an a_i in one workgroup, other group sizes and block shapes
              (1, 48, 48, 12), (2, 48, 48, 6), (1, 48, 48, 3), (2, 48, 48, 2), (1, 64, 64, 12), (1, 64, 64, 6),
              (2, 64, 64, 3), (1, 64, 64, 2), (1, 96, 96, 4), (2, 96, 96, 3), (1, 48, 192, 4), (1, 48, 192, 3),
              (2, 48, 192, 2), (1, 192, 48, 4), (1, 192, 48, 3), (1, 32, 32, 16),
              # d a multiple of the group: several workgroups per a_i, runs of DD floats
              (1, 48, 48, 32), (2, 48, 48, 24), (1, 64, 64, 16), (1, 16, 16, 64), (2, 96, 96, 8), (1, 192, 48, 16)]
    cases = [("fp32", False, p, batch) for p in shapes for batch in (512, 203)]
    # (143..157: the instances whose LDS tiles are split into one plane per d_i)
    _forced_sweep(cases, [1000 + i for i in list(range(32)) + list(range(97, 110)) + list(range(143, 160))], 2, 120)
    # fp16: the same design with 16-byte vectors of 8 halves (batch a multiple of nothing special)
    shapes16 = [(2, 48, 48, 16), (1, 48, 48, 8), (2, 48, 48, 4), (1, 48, 48, 12), (1, 48, 48, 6), (2, 48, 48, 2),
                (1, 64, 64, 16), (1, 64, 64, 8), (2, 64, 64, 3), (1, 96, 96, 8), (1, 96, 96, 3), (1, 48, 192, 8),
                (1, 48, 192, 4), (2, 192, 48, 8), (1, 192, 48, 3), (1, 16, 16, 16), (1, 32, 32, 8), (1, 128, 128, 4),
                (1, 48, 48, 32), (2, 48, 48, 24), (1, 64, 64, 64), (1, 16, 16, 64), (1, 192, 48, 16)]
    cases = [("fp16", False, p, batch) for p in shapes16 for batch in (512, 203)]
    _forced_sweep(cases, [1000 + i for i in list(range(25, 61)) + list(range(107, 125))], 2, 50)
    # e4m3: 16-byte vectors of 16 elements
    cases = [("fp8", False, p, batch) for p in shapes16 for batch in (512, 203)]
    _forced_sweep(cases, [1000 + i for i in list(range(61, 97)) + list(range(125, 143))], 2, 40)
    # three 128 x 128 blocks per workgroup (fp32: two waves per d_i), 16 x 16 blocks in groups of four
    late = [(2, 128, 128, 3), (1, 128, 128, 3), (3, 16, 16, 4), (16, 16, 16, 4), (1, 128, 128, 4), (2, 128, 128, 2),
            (1, 128, 128, 8)]
    for prec in ("fp32", "fp16", "fp8"):
        _forced_sweep([(prec, False, p, batch) for p in late for batch in (512, 203)], [1000 + i for i in list(range(158, 172)) + list(range(222, 240))], 2,
                      4 if prec == "fp32" else 16)
    # d = 1: groups of consecutive a_i (16 x 16 and 32 x 32 blocks), every group size that divides a
    ag = [(64, 16, 16, 1), (48, 16, 16, 1), (12, 16, 16, 1), (6, 16, 16, 1), (3, 16, 16, 1), (16, 32, 32, 1),
          (4, 32, 32, 1), (6, 32, 32, 1), (3, 32, 32, 1), (12, 64, 64, 1), (6, 64, 64, 1), (3, 64, 64, 1),
          (4, 48, 48, 1), (2, 48, 48, 1), (1, 48, 48, 1), (4, 96, 96, 1), (2, 96, 96, 1)]
    for prec in ("fp32", "fp16", "fp8"):
        _forced_sweep([(prec, False, p, batch) for p in ag for batch in (512, 203)], [1000 + i for i in range(167, 222)],
                      2, 60)
        # and as the automatic choice
        _forced_sweep([(prec, False, p, 1000) for p in ag], [-1], 0, len(ag))


def test_tile_subfamilies_forced():
    """Stream, weight-stationary, k-loop and batch-size-first (d > 1) tiles: every instance on
    shapes it can take."""
    cases = []
    for prec in ("fp16", "hq"):
        for bs_last in (True, False):
            for p in [(2, 64, 64, 1), (3, 128, 128, 1), (2, 192, 192, 1)]:
                cases.append((prec, bs_last, p, 1000))
    cases += [("fp32", True, (2, 64, 64, 1), 1000), ("fp32", True, (1, 128, 128, 1), 1000)]
    _forced_sweep(cases, [(2 << 24) | i for i in range(32)], 3, 24)                      # stream
    kcases = [("fp16", True, (2, 128, 64, 2), 520), ("fp16", False, (2, 128, 64, 1), 520),
              ("fp32", True, (1, 128, 64, 3), 520), ("fp32", False, (2, 64, 32, 1), 520),
              ("fp8", True, (2, 128, 64, 2), 528), ("hq", False, (1, 256, 128, 1), 520),
              ("fp16", True, (2, 96, 64, 2), 520), ("fp8", True, (1, 96, 96, 3), 528), ("fp32", True, (1, 96, 48, 2), 520),
              # b neither a multiple of the tile nor of the 16-byte vector
              ("fp16", True, (2, 70, 64, 2), 520), ("fp16", False, (2, 77, 64, 1), 520), ("fp32", True, (1, 45, 48, 3), 520),
              ("fp32", False, (1, 130, 32, 1), 520), ("fp8", True, (1, 50, 64, 2), 528), ("fp8", False, (2, 200, 64, 1), 528),
              ("fp16", True, (1, 449, 64, 1), 264)]
    _forced_sweep(kcases, [(0 << 24) | i for i in range(90)], 3, 52)                     # k-loop
    wcases = [("fp32", True, (2, 64, 64, 2), 520), ("fp32", False, (2, 96, 96, 1), 520),
              ("fp16", True, (2, 64, 64, 2), 520), ("fp16", False, (3, 64, 64, 1), 520),
              ("fp8", True, (2, 64, 64, 1), 528), ("hq", False, (2, 96, 96, 1), 520)]
    _forced_sweep(wcases, [(1 << 24) | i for i in range(64)], 3, 6)                      # weight-stationary
    bcases = [("fp16", False, (2, 128, 64, 2), 520), ("fp16", False, (1, 64, 64, 4), 520),
              ("fp32", False, (2, 64, 32, 2), 520), ("hq", False, (1, 128, 128, 2), 520)]
    _forced_sweep(bcases, [(3 << 24) | i for i in range(16)], 3, 4)                      # d > 1 tiles


def test_generic_kernel_forms_forced():
    """One thread per output (variant 0) and the 16-byte vector form for small blocks (variant 1,
    batch-size-last): blocks of a few elements with large d, b above one chunk of 8 outputs."""
    cases = [(prec, True, p, batch) for prec in ("fp32", "fp16", "fp8")
             for p in [(1, 2, 4, 112), (3, 1, 2, 40), (64, 7, 1, 1), (1, 14, 28, 16), (2, 16, 32, 8), (1, 20, 3, 5)]
             for batch in (64, 1040)]
    cases += [("fp16", False, (1, 2, 4, 112), 64), ("fp32", True, (1, 2, 4, 112), 7)]
    _forced_sweep(cases, [0, 1], 1, 70)


def test_tuned_table_rows_match_oracle():
    """A sample of the measured table's rows (every element type and layout), run through the
    automatic choice at a batch that consults the table, against the oracle; the tile the
    library reports must be the row's."""
    from ksmm_amd import Kernel, generate_factor
    from ksmm_amd.kernel import query_tile, tuned_table

    rows = [r for r in tuned_table() if r[0] * r[1] * r[2] * r[3] <= 1 << 16]
    assert len(rows) >= 40
    prec_of = {0: "fp32", 1: "fp16", 2: "fp8"}
    batch = 8192
    ran = {}
    for a, b, c, d, combo, bs_last, algo, variant in rows[::max(1, len(rows) // 40)]:
        prec = prec_of[combo]
        dt = TORCH_DTYPE[prec]
        pattern = (a, b, c, d)
        tile = query_tile(batch, pattern, dt, None, bool(bs_last))
        assert tile == query_tile(batch, pattern, dt, None, bool(bs_last), algo, variant)
        (w4,) = seeded_weights([pattern], seed=11)
        x = seeded_input(a * c * d, batch, bool(bs_last), seed=12)
        wr, wq, ws = round_to(w4, prec)
        xr, xq, xs = round_to(x, prec)
        if prec == "fp8":
            fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), dt, "cuda")
            xin, scale = xq.cuda(), ws * xs
        else:
            fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
            xin, scale = x.to(dt).cuda(), 1.0
        print("tuned row", pattern, prec, bs_last, algo, hex(variant), flush=True)
        y = Kernel.forward(xin, fac, bool(bs_last), a, b, c, d, dtype=dt, scale=scale)
        torch.cuda.synchronize()
        z = O.ks_apply_einsum(wr, xr, bool(bs_last))
        err = O.rel_fro_error(y.float().cpu().numpy(), z)
        assert err <= TOL[prec], (pattern, prec, bs_last, algo, hex(variant), err)
        ran[(combo, bs_last)] = ran.get((combo, bs_last), 0) + 1
    assert len(ran) >= 4, ran


def test_fp16_input_fp8_weight_factor():
    """Chain intermediate type: fp16 activations times e4m3fn weights."""
    from ksmm_amd import Kernel, generate_factor, quantize_fp8

    for pattern in [(16, 16, 16, 4), (64, 16, 16, 1), (2, 3, 5, 4), (1, 64, 64, 2)]:
        for bs_last in (True, False):
            a, b, c, d = pattern
            (w4,) = seeded_weights([pattern], seed=3)
            x = seeded_input(a * c * d, 200, bs_last, seed=4)
            wq, ws = quantize_fp8(w4)
            fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), torch.float8_e4m3fn, "cuda")
            y = Kernel.forward(x.half().cuda(), fac, bs_last, a, b, c, d, scale=float(ws))
            z = O.ks_apply_einsum(wq.double().numpy() * float(ws), x.half().double().numpy(), bs_last)
            assert y.dtype == torch.float16
            assert O.rel_fro_error(y.float().cpu().numpy(), z) <= TOL["fp16"], (pattern, bs_last)


CONFIGS = {
    # name: (patterns, precision, layouts, weight bound or None)
    "C1_readme_fp32": ([(6, 64, 64, 1), (1, 768, 192, 2)], "fp32", [True], None),
    "C2_48x48_d16_fp32": ([(1, 48, 48, 16)], "fp32", [True, False], None),
    "C3_192x192_fp16": ([(4, 192, 192, 1)], "fp16", [True, False], None),
    "C4_vit_b_up_fp16": ([(12, 64, 64, 1), (1, 1536, 384, 2)], "fp16", [False], None),
    "C5_butterfly_fp8": ([(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)], "fp8", [True], 0.25),
}
FULL_BATCH = 25088


@pytest.mark.parametrize("name", list(CONFIGS))
def test_config_full_batch(name):
    """The five benchmark configurations at B = 25088 through KSLinear(algo='kernel').  The
    oracle is evaluated on a sample of batch columns (columns are independent)."""
    from ksmm_amd import KSLinear

    patterns, prec, layouts, bound = CONFIGS[name]
    ws4 = seeded_weights(patterns, seed=0, bound=bound)
    in_size = patterns[0][0] * patterns[0][2] * patterns[0][3]
    for bs_last in layouts:
        x = seeded_input(in_size, FULL_BATCH, bs_last, seed=1)
        ksl = KSLinear(patterns, weights=ws4, bias=False, algo="kernel", dtype=TORCH_DTYPE[prec],
                       bs_last=bs_last, device="cuda")
        if prec == "fp8":
            xr, xq, xs = round_to(x, prec)
            y = ksl(xq.cuda(), x_scale=xs)
            wr = [round_to(w, prec)[0] for w in ws4]
        else:
            xr = round_to(x, prec)[0]
            y = ksl(x.to(TORCH_DTYPE[prec]).cuda())
            wr = [round_to(w, prec)[0] for w in ws4]
        torch.cuda.synchronize()
        cols = sample_columns(FULL_BATCH)
        z = oracle_chain(wr, xr, bs_last, cols)
        yh = y.float().cpu().numpy()
        ys = yh[:, cols] if bs_last else yh[cols, :]
        err = O.rel_fro_error(ys, z)
        assert np.isfinite(yh).all()
        assert err <= TOL[prec], (name, bs_last, err)
        # size-independent property on the full output: linearity in x (fp32/fp16 only; the
        # fp8 path re-quantises its input so it is checked through its scale instead)
        if prec == "fp8":
            y2 = ksl(xq.cuda(), x_scale=2 * xs)
            assert O.rel_fro_error(y2.float().cpu().numpy(), 2 * yh) <= 2e-3


@pytest.mark.parametrize("prec", ["fp8", "fp16"])
def test_fused_radix16_chain_matches_unfused_and_oracle(prec):
    """The LDS-resident fused chain (all factors b = c = 16) against the factor-by-factor launch
    and the oracle, on 2-, 3- and 4-factor chains and ragged batch sizes."""
    from ksmm_amd import KSLinear

    chains = [[(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)],
              [(4, 16, 16, 4), (16, 16, 16, 1)],
              [(1, 16, 16, 32), (2, 16, 16, 16), (8, 16, 16, 4), (32, 16, 16, 1)],
              [(64, 16, 16, 1), (1, 16, 16, 64)]]
    for patterns in chains:
        n_feat = patterns[0][0] * 16 * patterns[0][3]
        # (16400 columns: more chunks than workgroups and not a multiple of them, i.e. the launch
        # that cuts the batch into even contiguous ranges with a partial last chunk)
        for batch in (16, 80, 1000 if prec == "fp16" else 1008, 4096 + 48, 16400):
            ws4 = seeded_weights(patterns, seed=31, bound=0.25)
            x = seeded_input(n_feat, batch, True, seed=32)
            outs = {}
            for fuse in (True, False):
                ksl = KSLinear(patterns, weights=ws4, bias=False, algo="kernel", dtype=TORCH_DTYPE[prec],
                               bs_last=True, device="cuda", fuse=fuse)
                if prec == "fp8":
                    xr, xq, xs = round_to(x, prec)
                    outs[fuse] = ksl(xq.cuda(), x_scale=xs).float().cpu().numpy()
                else:
                    xr = round_to(x, prec)[0]
                    outs[fuse] = ksl(x.half().cuda()).float().cpu().numpy()
            wr = [round_to(w, prec)[0] for w in ws4]
            z = oracle_chain(wr, xr, True)
            assert O.rel_fro_error(outs[True], z) <= TOL[prec], (patterns, batch, "fused")
            assert O.rel_fro_error(outs[False], z) <= TOL[prec], (patterns, batch, "unfused")
            assert O.rel_fro_error(outs[True], outs[False]) <= 2e-3, (patterns, batch)


@pytest.mark.parametrize("prec", ["fp32", "fp16", "fp8"])
def test_bs_first_strided_blocks_take_the_transposed_route(prec):
    """Batch-size-first factors with d > 1 and no kernel of their own: the library asks for a
    workspace, runs them in batch-size-last layout between two transposes, and agrees with the
    oracle and with the generic kernel; so does a whole chain (KSLinear), fused or not."""
    import ctypes
    from ksmm_amd import Kernel, KSLinear, generate_factor, _lib
    from ksmm_amd.kernel import dtype_code, query_tile

    lib = _lib.load()
    dt = TORCH_DTYPE[prec]
    for pattern, batch in [((1, 192, 192, 16), 512), ((2, 128, 128, 8), 328), ((4, 64, 64, 8), 1000),
                           ((1, 96, 96, 6), 77), ((2, 64, 256, 8), 256), ((1, 192, 192, 12), 1001),
                           ((2, 128, 128, 6), 3)]:
        a, b, c, d = pattern
        ydt = torch.float16 if prec == "fp8" else dt
        need = lib.ksmm_factor_workspace(batch, a, b, c, d, dtype_code(dt), dtype_code(dt), dtype_code(ydt), 0)
        if batch % 16 == 0:
            assert lib.ksmm_factor_workspace(batch, a, b, c, d, dtype_code(dt), dtype_code(dt), dtype_code(ydt), 1) == 0
        y, z = _run_factor(pattern, batch, prec, False, "auto")
        assert O.rel_fro_error(y, z) <= TOL[prec], (pattern, batch)
        direct = query_tile(batch, pattern, dt, dt, False)["algo"] != 1   # e.g. the fp32 row kernel
        # batch-size-last kernel (the transposed copy has rows padded to 16 columns)
        twin = query_tile((batch + 15) // 16 * 16, pattern, dt, dt, True)["algo"] != 1
        if direct or not twin:
            assert need == 0, pattern
            continue
        assert need > 0, pattern
        # too small a workspace is an error, not a silent fallback
        (w4,) = seeded_weights([pattern], seed=0)
        fac = generate_factor(a, b, c, d, "kernel", w4 if prec != "fp8" else round_to(w4, prec)[1].float(), dt, "cuda")
        xin = torch.zeros(batch, a * c * d, device="cuda").to(dt)
        out = torch.empty(batch, a * b * d, device="cuda", dtype=ydt)
        small = torch.empty(256, dtype=torch.uint8, device="cuda")
        rc = lib.ksmm_factor_forward_ws(xin.data_ptr(), fac.data_ptr(), out.data_ptr(), batch, a, b, c, d,
                                        dtype_code(dt), dtype_code(dt), dtype_code(ydt), 0, 1.0,
                                        small.data_ptr(), 256, None)
        assert rc == -9
    # chains: butterfly (fused between the transposes) and a mixed one
    for patterns, batch in [([(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)], 400),
                            ([(2, 64, 64, 8), (16, 64, 64, 1)], 264),
                            ([(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)], 203),
                            ([(2, 128, 128, 6), (12, 128, 128, 1)], 77)]:
        if prec == "fp32" and patterns[0][1] == 16:
            continue
        ws4 = seeded_weights(patterns, seed=41, bound=0.25)
        n_in = patterns[0][0] * patterns[0][2] * patterns[0][3]
        x = seeded_input(n_in, batch, False, seed=42)
        ksl = KSLinear(patterns, weights=ws4, bias=False, algo="kernel", dtype=dt, bs_last=False, device="cuda")
        if prec == "fp8":
            xr, xq, xs = round_to(x, prec)
            y = ksl(xq.cuda(), x_scale=xs).float().cpu().numpy()
        else:
            xr = round_to(x, prec)[0]
            y = ksl(x.to(dt).cuda()).float().cpu().numpy()
        z = oracle_chain([round_to(w, prec)[0] for w in ws4], xr, False)
        assert O.rel_fro_error(y, z) <= TOL[prec], (patterns, batch)


@pytest.mark.parametrize("prec", ["fp32", "fp16", "fp8"])
def test_unaligned_batch_runs_on_padded_rows(prec):
    """Batch-size-last with a batch that is not a multiple of the 16-byte vector: with the
    workspace the library asks for, the factor runs on rows padded to 16 columns with the kernel
    of the padded batch (not the one-thread-per-output kernel), and agrees with the oracle; so do
    whole chains (KSLinear), fused or not.  Without a workspace the slow kernel still answers."""
    from ksmm_amd import Kernel, KSLinear, generate_factor, _lib
    from ksmm_amd.kernel import dtype_code, query_tile

    lib = _lib.load()
    dt = TORCH_DTYPE[prec]
    ydt = torch.float16 if prec == "fp8" else dt
    for pattern, batch in [((1, 48, 48, 16), 25087), ((6, 64, 64, 1), 2003), ((1, 768, 192, 2), 1001),
                           ((4, 192, 192, 1), 4099), ((64, 16, 16, 1), 333), ((2, 3, 5, 4), 77),
                           ((1, 128, 70, 2), 203), ((1, 48, 48, 16), 7)]:
        a, b, c, d = pattern
        need = lib.ksmm_factor_workspace(batch, a, b, c, d, dtype_code(dt), dtype_code(dt), dtype_code(ydt), 1)
        assert need > 0, (pattern, batch)
        assert query_tile(batch, pattern, dt, dt, True)["algo"] == 1
        padded = query_tile((batch + 15) // 16 * 16, pattern, dt, dt, True)
        assert padded["algo"] != 1 or padded["variant"] == 1, pattern
        y, z = _run_factor(pattern, batch, prec, True, "auto")
        assert y.shape == z.shape
        if batch > 4096:
            cols = sample_columns(batch)
            y, z = y[:, cols], z[:, cols]
        assert O.rel_fro_error(y, z) <= TOL[prec], (pattern, batch)
        # the same call without a workspace: the one-thread-per-output kernel, same result
        if batch <= 2048:
            y1, _ = _run_factor(pattern, batch, prec, True, "generic")
            assert O.rel_fro_error(y1, z) <= TOL[prec], (pattern, batch)
    for patterns, batch in [([(6, 64, 64, 1), (1, 768, 192, 2)], 2003),
                            ([(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)], 1001)]:
        if prec == "fp32" and patterns[0][1] == 16:
            continue
        ws4 = seeded_weights(patterns, seed=51, bound=0.25)
        n_in = patterns[0][0] * patterns[0][2] * patterns[0][3]
        x = seeded_input(n_in, batch, True, seed=52)
        bias = torch.linspace(-1, 1, patterns[-1][0] * patterns[-1][1] * patterns[-1][3])
        for fuse in (True, False):
            ksl = KSLinear(patterns, weights=ws4, bias=True, algo="kernel", dtype=dt, bs_last=True, device="cuda")
            ksl.fuse = fuse
            with torch.no_grad():
                ksl.bias.copy_(bias.to(ksl.bias.dtype).reshape(ksl.bias.shape))
                if prec == "fp8":
                    xr, xq, xs = round_to(x, prec)
                    y = ksl(xq.cuda(), x_scale=xs).float().cpu().numpy()
                else:
                    xr = round_to(x, prec)[0]
                    y = ksl(x.to(dt).cuda()).float().cpu().numpy()
            z = oracle_chain([round_to(w, prec)[0] for w in ws4], xr, True)
            z = z + ksl.bias.detach().float().cpu().double().numpy().reshape(-1, 1)
            assert y.shape == z.shape
            assert O.rel_fro_error(y, z) <= TOL[prec], (patterns, batch, fuse)


def test_layouts_agree_full_batch():
    """bs_last result == transposed bs_first result (same weights, fp32, C2 at full batch)."""
    from ksmm_amd import KSLinear

    patterns = [(1, 48, 48, 16)]
    ws4 = seeded_weights(patterns, seed=5)
    x = seeded_input(768, FULL_BATCH, False, seed=6)
    k_first = KSLinear(patterns, weights=ws4, bias=False, algo="kernel", dtype=torch.float32,
                       bs_last=False, device="cuda")
    k_last = KSLinear(patterns, weights=ws4, bias=False, algo="kernel", dtype=torch.float32,
                      bs_last=True, device="cuda")
    y1 = k_first(x.cuda())
    y2 = k_last(x.t().contiguous().cuda())
    assert O.rel_fro_error(y2.t().cpu().numpy(), y1.cpu().numpy()) <= 2e-6


def test_linearity_full_batch():
    from ksmm_amd import KSLinear

    patterns = [(6, 64, 64, 1), (1, 768, 192, 2)]
    ws4 = seeded_weights(patterns, seed=7)
    ksl = KSLinear(patterns, weights=ws4, bias=False, algo="kernel", dtype=torch.float32,
                   bs_last=True, device="cuda")
    x = seeded_input(384, FULL_BATCH, True, seed=8).cuda()
    z = seeded_input(384, FULL_BATCH, True, seed=9).cuda()
    lhs = ksl(2 * x - 3 * z)
    rhs = 2 * ksl(x) - 3 * ksl(z)
    assert O.rel_fro_error(lhs.cpu().numpy(), rhs.cpu().numpy()) <= 1e-5


def test_kernel_matches_dense_and_bmm_algos():
    """The README comparison (scripts/example.py:19-23): kernel vs dense vs bmm, same weights,
    bias off, on the device."""
    from ksmm_amd import KSLinear

    patterns = [(6, 64, 64, 1), (1, 768, 192, 2)]
    ws4 = seeded_weights(patterns, seed=10)
    x = seeded_input(384, 1024, True, seed=11).cuda()
    ys = {}
    for algo in ("kernel", "dense", "bmm", "einsum"):
        ksl = KSLinear(patterns, weights=ws4, bias=False, algo=algo, dtype=torch.float32,
                       bs_last=True, device="cuda")
        ys[algo] = ksl(x).detach().double().cpu().numpy()
    for algo in ("dense", "bmm", "einsum"):
        assert O.rel_fro_error(ys["kernel"], ys[algo]) <= 1e-5, algo


def test_bias_and_nd_input():
    from ksmm_amd import KSLinear

    patterns = [(2, 16, 16, 2)]
    ws4 = seeded_weights(patterns, seed=12)
    for bs_last in (False, True):
        kk = KSLinear(patterns, weights=ws4, bias=True, algo="kernel", dtype=torch.float32,
                      bs_last=bs_last, device="cuda")
        kd = KSLinear(patterns, weights=ws4, bias=True, algo="dense", dtype=torch.float32,
                      bs_last=bs_last, device="cuda")
        with torch.no_grad():
            kd.bias.copy_(kk.bias)
        x = torch.randn(64, 5, 3, device="cuda") if bs_last else torch.randn(5, 3, 64, device="cuda")
        y, z = kk(x), kd(x)
        assert y.shape == z.shape == ((64, 5, 3) if bs_last else (5, 3, 64))
        assert O.rel_fro_error(y.detach().cpu().numpy(), z.detach().cpu().numpy()) <= 1e-5


def test_current_stream_is_used():
    """Launches go to torch's current stream: work queued on a side stream is ordered after
    the producer on that stream without a device-wide sync."""
    from ksmm_amd import Kernel, generate_factor

    pattern = (1, 48, 48, 16)
    (w4,) = seeded_weights([pattern], seed=13)
    fac = generate_factor(*pattern, "kernel", w4, torch.float32, "cuda")
    s = torch.cuda.Stream()
    x = torch.zeros(768, 4096, device="cuda")
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        x.normal_()                      # producer on s
        y = Kernel.forward(x, fac, True, *pattern)
    s.synchronize()
    z = O.ks_apply_einsum(w4.double().numpy(), x.double().cpu().numpy(), True)
    assert O.rel_fro_error(y.cpu().numpy(), z) <= 1e-5


def _gelu64(v):
    from scipy.special import erf

    return 0.5 * v * (1.0 + erf(v / np.sqrt(2.0)))


EPILOGUE_CASES = [
    # pattern, batch: chosen so that the automatic choice visits every kernel family
    ((1, 48, 48, 16), 1040), ((6, 64, 64, 1), 520), ((2, 192, 192, 1), 520), ((1, 256, 64, 2), 520),
    ((2, 3, 5, 4), 203), ((1, 96, 48, 2), 520), ((3, 16, 16, 4), 528), ((1, 192, 192, 16), 264),
    ((2, 128, 70, 1), 520), ((1, 2, 4, 112), 64), ((2, 77, 64, 1), 520), ((1, 128, 128, 1), 1024),
    # enough batch tiles for the direct-to-LDS GEMM tiles (d = 2 and d = 1 epilogues differ)
    ((2, 256, 64, 2), 8192), ((2, 256, 64, 1), 8192),
]


@pytest.mark.parametrize("bs_last", [True, False])
@pytest.mark.parametrize("prec", ["fp32", "fp16", "fp8"])
def test_bias_and_gelu_in_the_kernel_epilogue(prec, bs_last):
    """y = gelu(scale * K x + bias) computed inside the kernels against the float64 oracle
    (bias and GELU applied to the oracle's product), bias only and bias + GELU; the families the
    automatic choice used are collected and must include every one that exists for the layout."""
    from ksmm_amd import Kernel, generate_factor
    from ksmm_amd.kernel import query_tile

    dt = TORCH_DTYPE[prec]
    out_dt = torch.float16 if prec == "fp8" else dt
    seen = set()
    for pattern, batch in EPILOGUE_CASES:
        a, b, c, d = pattern
        (w4,) = seeded_weights([pattern], seed=61)
        x = seeded_input(a * c * d, batch, bs_last, seed=62)
        g = torch.Generator().manual_seed(63)
        bias = (torch.rand(a * b * d, generator=g) - 0.5).to(out_dt)
        wr, wq, ws = round_to(w4, prec)
        xr, xq, xs = round_to(x, prec)
        if prec == "fp8":
            fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), dt, "cuda")
            xin, scale = xq.cuda(), ws * xs
        else:
            fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
            xin, scale = x.to(dt).cuda(), 1.0
        t = query_tile(batch, pattern, dt, None, bs_last)
        seen.add((t["algo"], t["variant"] >> 24 if t["algo"] == 3 else (t["variant"] >= 1000 if t["algo"] == 2 else t["variant"])))
        z = O.ks_apply_einsum(wr, xr, bs_last)
        bz = bias.double().numpy()
        zb = z + (bz[:, None] if bs_last else bz[None, :])
        for act, want in ((None, zb), ("gelu", _gelu64(zb))):
            y = Kernel.forward(xin, fac, bs_last, a, b, c, d, scale=scale, bias=bias.cuda(), act=act)
            err = O.rel_fro_error(y.float().cpu().numpy(), want)
            assert err <= TOL[prec], (pattern, batch, prec, bs_last, act, t, err)
        # activation without a bias
        y = Kernel.forward(xin, fac, bs_last, a, b, c, d, scale=scale, act="gelu")
        assert O.rel_fro_error(y.float().cpu().numpy(), _gelu64(z)) <= TOL[prec], (pattern, prec, bs_last)
    print("families seen", prec, bs_last, sorted(seen), flush=True)
    assert len(seen) >= (4 if bs_last else 3), seen
    if bs_last or prec == "fp16":
        assert (3, 4) in seen, seen  # the GEMM tiles' bias/activation instantiation ran


@pytest.mark.parametrize("prec", ["fp16", "fp8"])
def test_kslinear_bias_gelu_chain(prec):
    """KSLinear(bias=True, act='gelu', algo='kernel') against the same layer with algo='dense' (which
    adds the bias and applies F.gelu in PyTorch) and against the float64 oracle: the two-factor
    ViT up-projection shape in batch-size-first layout and the fused radix-16 chain."""
    from ksmm_amd import KSLinear

    for patterns, bs_last, batch in [([(12, 64, 64, 1), (1, 1536, 384, 2)], False, 392),
                                     ([(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)], True, 1008),
                                     ([(6, 64, 64, 1), (1, 768, 192, 2)], True, 520)]:
        if prec == "fp8" and patterns[0][1] == 64 and not bs_last:
            continue  # e4m3 batch-size-first with d = 2 runs on the transposed route: covered above
        ws4 = seeded_weights(patterns, seed=71, bound=0.25 if patterns[0][1] == 16 else None)
        n_in = patterns[0][0] * patterns[0][2] * patterns[0][3]
        x = seeded_input(n_in, batch, bs_last, seed=72)
        dt = TORCH_DTYPE[prec]
        kk = KSLinear(patterns, weights=ws4, bias=True, algo="kernel", dtype=dt, bs_last=bs_last, device="cuda",
                      act="gelu")
        bz = kk.bias.detach().double().cpu().numpy().reshape(-1)
        if prec == "fp8":
            xr, xq, xs = round_to(x, prec)
            y = kk(xq.cuda(), x_scale=xs).float().cpu().numpy()
        else:
            xr = round_to(x, prec)[0]
            y = kk(x.to(dt).cuda()).float().cpu().numpy()
        z = oracle_chain([round_to(w, prec)[0] for w in ws4], xr, bs_last)
        want = _gelu64(z + (bz[:, None] if bs_last else bz[None, :]))
        assert O.rel_fro_error(y, want) <= TOL[prec], (patterns, prec)


BACKWARD_CASES = [
    # pattern, batch: MFMA weight-gradient tiles of 16, 32, 48 and 64, ragged b / c, d > 1, odd batch
    ((1, 48, 48, 16), 1040), ((6, 64, 64, 1), 520), ((2, 3, 5, 4), 203), ((1, 96, 48, 2), 264), ((3, 16, 16, 4), 528),
    ((1, 256, 64, 2), 520), ((2, 77, 64, 1), 520), ((1, 17, 33, 2), 64), ((2, 32, 32, 3), 1000), ((1, 192, 192, 16), 264),
    # fp16: the 128 x 128 tiles of the GEMM-shaped weight gradient (several tiles per block, d > 1, ragged last slab)
    ((1, 256, 128, 2), 520), ((2, 128, 128, 1), 1000), ((1, 128, 256, 3), 264), ((1, 384, 128, 1), 4168),
]


@pytest.mark.parametrize("bs_last", [True, False])
@pytest.mark.parametrize("prec", ["fp32", "fp16"])
def test_factor_backward_matches_oracle(prec, bs_last):
    """ksmm_factor_backward_input / _weight through Kernel.backward against the float64 adjoints
    (oracle.ks_backward) on the values the device holds."""
    from ksmm_amd import Kernel, generate_factor
    from ksmm_amd.layer import from_kernel_format_to_abcd

    dt = TORCH_DTYPE[prec]
    tol = {"fp32": 2e-5, "fp16": 2e-3}[prec]
    for pattern, batch in BACKWARD_CASES:
        a, b, c, d = pattern
        (w4,) = seeded_weights([pattern], seed=91)
        x = seeded_input(a * c * d, batch, bs_last, seed=92)
        dy = seeded_input(a * b * d, batch, bs_last, seed=93)
        fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
        gi, gf = Kernel.backward(dy.to(dt).cuda(), x.to(dt).cuda(), fac, bs_last, a, b, c, d)
        torch.cuda.synchronize()
        dx, dw = O.ks_backward(round_to(w4, prec)[0], round_to(x, prec)[0], round_to(dy, prec)[0], bs_last)
        assert gi.shape == x.shape and gf.shape == fac.shape
        assert O.rel_fro_error(gi.float().cpu().numpy(), dx) <= tol, (pattern, batch, prec, bs_last, "dX")
        got_dw = from_kernel_format_to_abcd(gf.float().cpu(), pattern).numpy()
        assert O.rel_fro_error(got_dw, dw) <= tol, (pattern, batch, prec, bs_last, "dW")


@pytest.mark.parametrize("bs_last", [True, False])
def test_weight_gradient_is_bit_reproducible(bs_last):
    """The weight gradient reduces over the batch in per-split partial sums that a finish kernel
    adds in a fixed order (no atomics): repeated calls on the same inputs, at a batch large enough
    for many splits, give the same bits, and agree with the oracle."""
    from ksmm_amd import Kernel, generate_factor
    from ksmm_amd.layer import from_kernel_format_to_abcd

    for prec, pattern, batch in [("fp32", (1, 48, 48, 16), 25088), ("fp16", (2, 64, 96, 3), 8200), ("fp32", (3, 20, 12, 2), 4099),
                                 ("fp16", (1, 256, 128, 2), 8200)]:
        a, b, c, d = pattern
        dt = TORCH_DTYPE[prec]
        (w4,) = seeded_weights([pattern], seed=101)
        x = seeded_input(a * c * d, batch, bs_last, seed=102).to(dt).cuda()
        dy = seeded_input(a * b * d, batch, bs_last, seed=103).to(dt).cuda()
        fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
        runs = [Kernel.backward(dy, x, fac, bs_last, a, b, c, d, need_input=False)[1] for _ in range(4)]
        torch.cuda.synchronize()
        for g in runs[1:]:
            assert torch.equal(g.view(torch.uint8), runs[0].view(torch.uint8)), (prec, pattern, bs_last)
        _, dw = O.ks_backward(round_to(w4, prec)[0], x.float().cpu().double().numpy(), dy.float().cpu().double().numpy(), bs_last)
        got = from_kernel_format_to_abcd(runs[0].float().cpu(), pattern).numpy()
        assert O.rel_fro_error(got, dw) <= {"fp32": 2e-5, "fp16": 2e-3}[prec], (prec, pattern, bs_last)


def test_kslinear_trains_through_the_kernel_path():
    """Autograd through KSLinear(algo='kernel') (two factors, bias, GELU) against the same layer
    with algo='dense': output, input gradient, bias gradient and the gradient of every factor
    (compared as 4-D weights)."""
    from ksmm_amd import KSLinear
    from ksmm_amd.layer import from_kernel_format_to_abcd

    patterns = [(6, 64, 64, 1), (1, 768, 192, 2)]
    ws4 = seeded_weights(patterns, seed=95)
    with torch.enable_grad():
        kk = KSLinear(patterns, weights=ws4, bias=True, algo="kernel", dtype=torch.float32, bs_last=True, device="cuda",
                      act="gelu")
        ke = KSLinear(patterns, weights=ws4, bias=True, algo="einsum", dtype=torch.float32, bs_last=True, device="cuda",
                      act="gelu")
        with torch.no_grad():
            ke.bias.copy_(kk.bias)
        x1 = seeded_input(384, 328, True, seed=96).cuda().requires_grad_(True)
        x2 = x1.detach().clone().requires_grad_(True)
        g = seeded_input(1536, 328, True, seed=97).cuda()
        y1, y2 = kk(x1), ke(x2)
        (y1 * g).sum().backward()
        (y2 * g).sum().backward()
    rel = lambda u, v: O.rel_fro_error(u.detach().double().cpu().numpy(), v.detach().double().cpu().numpy())
    assert rel(y1, y2) <= 1e-5
    assert rel(x1.grad, x2.grad) <= 2e-5
    assert rel(kk.bias.grad, ke.bias.grad) <= 2e-5
    for fk, fe, p in zip(kk.factors, ke.factors, patterns):
        assert rel(from_kernel_format_to_abcd(fk.grad, p), fe.grad) <= 2e-5, p


def test_persistent_gemm_walks_several_tiles_per_workgroup():
    """The persistent batch-size-first GEMM instances (loads and stores issued by different waves,
    the slab stream running on across tile boundaries) on problems with about three tiles per
    workgroup, a ragged last batch tile and c = 3 slabs: the whole output against the ordinary
    GEMM instance of the same tile (same summation order: equal up to nothing), sampled rows
    against the oracle, and the bias + GELU epilogue."""
    from ksmm_amd import Kernel, generate_factor, _lib
    from ksmm_amd.kernel import variant_id

    batch = 20008
    ran = 0
    for pattern in [(1, 512, 96, 2), (2, 512, 96, 1), (3, 256, 64, 2)]:
        a, b, c, d = pattern
        (w4,) = seeded_weights([pattern], seed=101)
        x = seeded_input(a * c * d, batch, False, seed=102)
        fac = generate_factor(a, b, c, d, "kernel", w4, torch.float16, "cuda")
        xin = x.half().cuda()
        ref = Kernel.forward(xin, fac, False, a, b, c, d, algo=0, variant=-3)
        rows = sample_columns(batch, step=389)
        z = O.ks_apply_einsum(round_to(w4, "fp16")[0], round_to(x, "fp16")[0][rows], False)
        assert O.rel_fro_error(ref.float().cpu().numpy()[rows], z) <= TOL["fp16"]
        for inst in range(32, 64):
            try:
                variant_id(3, (4 << 24) | inst, 1, False)
            except _lib.KsmmError:
                continue
            try:
                y = Kernel.forward(xin, fac, False, a, b, c, d, algo=3, variant=(4 << 24) | inst)
            except _lib.KsmmError as e:
                assert e.status == -6
                continue
            torch.cuda.synchronize()
            ran += 1
            assert torch.isfinite(y).all(), (pattern, inst)
            err = ((y.float() - ref.float()).norm() / ref.float().norm()).item()
            assert err <= 1e-6, (pattern, inst, err)
    assert ran >= 7, ran
    # bias + GELU on the persistent kernel (its epilogue is an instantiation of its own): forced
    # instances take no epilogue, so a problem with three tiles per CU, where the heuristic picks
    # the persistent form by itself
    from ksmm_amd.kernel import query_tile

    pattern, batch = (1, 512, 96, 2), 49152
    a, b, c, d = pattern
    t = query_tile(batch, pattern, torch.float16, None, False)
    assert t["algo"] == 3 and (t["variant"] >> 24) == 4 and t["grid"] == 256, t
    (w4,) = seeded_weights([pattern], seed=103)
    x = seeded_input(a * c * d, batch, False, seed=104)
    fac = generate_factor(a, b, c, d, "kernel", w4, torch.float16, "cuda")
    bias = (torch.rand(a * b * d, generator=torch.Generator().manual_seed(7)) - 0.5).half()
    rows = sample_columns(batch, step=911)
    z = O.ks_apply_einsum(round_to(w4, "fp16")[0], round_to(x, "fp16")[0][rows], False)
    zb = z + bias.double().numpy()[None, :]
    import scipy.special

    zg = 0.5 * zb * (1.0 + scipy.special.erf(zb / np.sqrt(2.0)))
    for act, want in ((None, zb), ("gelu", zg)):
        y = Kernel.forward(x.half().cuda(), fac, False, a, b, c, d, bias=bias.cuda(), act=act)
        assert O.rel_fro_error(y.float().cpu().numpy()[rows], want) <= TOL["fp16"], act


def test_persistent_gemm_batch_size_last():
    """The persistent batch-size-last GEMM instances (fp16 and fp32) on problems with two to five
    tiles per workgroup, d > 1, several a_i, a ragged last batch tile and 2-4 K slabs: the whole
    output against the automatic choice, sampled columns against the oracle."""
    from ksmm_amd import Kernel, generate_factor, _lib
    from ksmm_amd.kernel import query_tile

    batch = 20008
    ran = 0
    for prec, pattern in [("fp16", (1, 512, 96, 2)), ("fp16", (2, 256, 64, 3)), ("fp32", (2, 512, 64, 2)),
                          ("fp32", (1, 768, 48, 3)), ("fp32", (1, 48, 48, 16)), ("fp16", (2, 96, 64, 3)),
                          ("fp32", (3, 80, 32, 4))]:
        a, b, c, d = pattern
        dt = TORCH_DTYPE[prec]
        (w4,) = seeded_weights([pattern], seed=111)
        x = seeded_input(a * c * d, batch, True, seed=112)
        fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
        xin = x.to(dt).cuda()
        ref = Kernel.forward(xin, fac, True, a, b, c, d)
        cols = sample_columns(batch, step=389)
        z = O.ks_apply_einsum(round_to(w4, prec)[0], round_to(x, prec)[0][:, cols], True)
        assert O.rel_fro_error(ref.float().cpu().numpy()[:, cols], z) <= TOL[prec]
        for inst in range(32, 64):
            try:
                t = query_tile(batch, pattern, dt, None, True, algo=3, variant=(4 << 24) | inst)
            except _lib.KsmmError:
                continue  # no such instance, or one that does not fit
            if t["grid"] not in (256, 512):
                continue  # one workgroup per tile: not a persistent instance (those run 1 or 2 per CU)
            y = Kernel.forward(xin, fac, True, a, b, c, d, algo=3, variant=(4 << 24) | inst)
            torch.cuda.synchronize()
            ran += 1
            assert torch.isfinite(y).all(), (prec, pattern, inst)
            err = ((y.float() - ref.float()).norm() / ref.float().norm()).item()
            assert err <= (1e-3 if prec == "fp16" else 2e-6), (prec, pattern, inst, err)
            assert O.rel_fro_error(y.float().cpu().numpy()[:, cols], z) <= TOL[prec], (prec, pattern, inst)
    assert ran >= 20, ran
    # the e4m3 instances (the persistent ones are the last of the table), whole output against the oracle
    _forced_sweep([("fp8", True, (1, 512, 128, 2), 20016), ("fp8", True, (2, 96, 128, 3), 20016)],
                  [(4 << 24) | i for i in range(39, 64)], 3, 8)
    # bias + GELU (an instantiation of its own), reached through the automatic choice: three
    # tiles per CU make the heuristic take the persistent form
    import scipy.special

    for prec, pattern, batch in [("fp16", (1, 512, 96, 2), 49152), ("fp32", (2, 256, 64, 3), 32772),
                                 ("fp16", (2, 192, 64, 3), 49160)]:
        a, b, c, d = pattern
        dt = TORCH_DTYPE[prec]
        t = query_tile(batch, pattern, dt, None, True)
        assert t["algo"] == 3 and (t["variant"] >> 24) == 4 and t["grid"] in (256, 512), t
        (w4,) = seeded_weights([pattern], seed=113)
        x = seeded_input(a * c * d, batch, True, seed=114)
        fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
        bias = torch.from_numpy(np.random.default_rng(115).standard_normal(a * b * d).astype(np.float32)).to(dt)
        cols = sample_columns(batch, step=997)
        z = O.ks_apply_einsum(round_to(w4, prec)[0], round_to(x, prec)[0][:, cols], True)
        zb = z + bias.double().numpy()[:, None]
        zg = 0.5 * zb * (1.0 + scipy.special.erf(zb / np.sqrt(2.0)))
        for act, want in ((None, zb), ("gelu", zg)):
            y = Kernel.forward(x.to(dt).cuda(), fac, True, a, b, c, d, bias=bias.cuda(), act=act)
            assert O.rel_fro_error(y.float().cpu().numpy()[:, cols], want) <= TOL[prec], (prec, act)


def test_measurement_probes():
    """The measurement aids of the benchmark (libksmm_bench.so, not part of the drop-in ABI): the
    tile copy and the streaming copy must reproduce their input exactly (ragged last batch tile,
    several blocks, every supported tile width; a size that is not a multiple of a round) and
    refuse what they cannot hold; the matrix-core probe must report the flops it was asked to
    perform."""
    import ctypes

    from ksmm_amd import _lib, bench_lib
    from ksmm_amd.kernel import dtype_code

    lib = bench_lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    a, rows, d, batch = 2, 48, 3, 1000  # 4000-byte rows: 250 vectors, ragged for every tile width
    x = torch.randn(a * rows * d, batch, device="cuda")
    for tile_bytes in (16, 256, 1024, 4096):
        y = torch.zeros_like(x)
        _lib.check(lib.ksbench_tilecopy_probe(x.data_ptr(), y.data_ptr(), batch * 4, a, rows, d, tile_bytes, stream))
        torch.cuda.synchronize()
        assert torch.equal(x, y), tile_bytes
    assert lib.ksbench_tilecopy_probe(x.data_ptr(), y.data_ptr(), batch * 4, a, 49, d, 4096, stream) == -2  # 49 rows of 4 KB
    assert lib.ksbench_tilecopy_probe(x.data_ptr(), y.data_ptr(), batch * 4, a, rows, d, 48, stream) == -2  # not a power of two
    for wgs in (1, 7, 512):
        y = torch.zeros_like(x)
        _lib.check(lib.ksbench_stream_copy(x.data_ptr(), y.data_ptr(), x.numel() * 4, wgs, stream))
        torch.cuda.synchronize()
        assert torch.equal(x, y), wgs
    assert lib.ksbench_stream_copy(x.data_ptr(), y.data_ptr(), 24, 8, stream) == -9  # not whole vectors
    out = torch.empty(lib.ksbench_mfma_probe_bytes(), dtype=torch.uint8, device="cuda")
    flops = ctypes.c_double(0.0)
    _lib.check(lib.ksbench_mfma_probe(dtype_code(torch.float16), 10, 1, out.data_ptr(), out.numel(), ctypes.byref(flops), stream))
    torch.cuda.synchronize()
    assert flops.value == 16 * 2.0 * 32 * 32 * 16 * 10 * 256 * 8


def test_auto_dispatch_at_larger_batches():
    """The automatic choice at batches where the persistent GEMM tiles, the masked last TM-tile,
    the pipelined batch-size-first tiles and the measured table take over (the small-batch
    tests above stay below their thresholds): sampled batch entries against the oracle, and
    the families that are expected to run must be the ones that do."""
    from ksmm_amd import Kernel, generate_factor
    from ksmm_amd.kernel import query_tile

    cases = [  # (prec, bs_last, pattern, batch)
        ("fp16", True, (3, 192, 64, 4), 33000), ("fp32", True, (2, 192, 64, 3), 33000),
        ("fp16", True, (1, 96, 384, 6), 25088), ("fp32", True, (2, 452, 64, 1), 18004),
        ("fp8", True, (2, 192, 128, 3), 33008), ("fp8", True, (1, 96, 128, 8), 25088),
        ("fp16", False, (1, 192, 192, 16), 9000), ("fp16", False, (2, 64, 64, 64), 9000),
        ("fp32", False, (1, 192, 192, 8), 9000), ("fp32", False, (3, 64, 64, 16), 25088),
        ("fp16", False, (1, 1536, 384, 2), 25088), ("fp32", True, (1, 768, 192, 2), 25088),
        ("fp16", True, (4, 192, 192, 1), 25088), ("fp32", True, (6, 64, 64, 1), 25088),
        ("fp16", True, (1, 512, 128, 2), 12296), ("fp32", False, (3, 64, 64, 64), 4104),
        # big 16-bit blocks with d = 4 in batch-size-first: the transposed route (algo 1 here)
        ("fp16", False, (1, 512, 512, 4), 4100), ("fp16", False, (1, 1024, 256, 4), 4096),
        # batch-size-last batches off the vector: the padded-rows route
        ("fp16", True, (4, 192, 192, 1), 25083), ("fp32", True, (1, 768, 192, 2), 9001),
    ]
    seen = set()
    for prec, bs_last, pattern, batch in cases:
        a, b, c, d = pattern
        dt = TORCH_DTYPE[prec]
        t = query_tile(batch, pattern, dt, None, bs_last)
        seen.add((t["algo"], t["variant"] >> 24 if t["algo"] == 3 else -1, t["grid"] in (256, 512)))
        print("auto", prec, bs_last, pattern, batch, t["algo"], hex(t["variant"]), t["grid"], flush=True)
        (w4,) = seeded_weights([pattern], seed=201)
        x = seeded_input(a * c * d, batch, bs_last, seed=202)
        wr, wq, ws = round_to(w4, prec)
        xr, xq, xs = round_to(x, prec)
        if prec == "fp8":
            fac = generate_factor(a, b, c, d, "kernel", wq.to(torch.float32), dt, "cuda")
            xin, scale = xq.cuda(), ws * xs
        else:
            fac = generate_factor(a, b, c, d, "kernel", w4, dt, "cuda")
            xin, scale = x.to(dt).cuda(), 1.0
        y = Kernel.forward(xin, fac, bs_last, a, b, c, d, dtype=dt, scale=scale)
        torch.cuda.synchronize()
        assert torch.isfinite(y).all(), (prec, bs_last, pattern, batch)
        idx = sample_columns(batch, step=211)
        xs_ = xr[:, idx] if bs_last else xr[idx]
        z = O.ks_apply_einsum(wr, xs_, bs_last)
        got = y.float().cpu().numpy()
        got = got[:, idx] if bs_last else got[idx]
        err = O.rel_fro_error(got, z)
        assert err <= TOL[prec], (prec, bs_last, pattern, batch, t, err)
    # persistent GEMM tiles (one or two workgroups per CU) and the batch-size-first tile kernels ran
    assert (3, 4, True) in seen and any(s[0] == 3 and s[1] == 3 for s in seen), seen
