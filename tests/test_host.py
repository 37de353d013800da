"""CPU-only checks of the host side: the C ABI loads and exports every declared symbol, its
argument validation returns the documented codes, and KSLinear's host logic mirrors the
reference's error behaviour.  No GPU call is made."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import ks_oracle as O
from tests.util import seeded_input, seeded_weights

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(lib):
    from ksmm_amd import _lib

    header = open(os.path.join(ROOT, "include", "ksmm_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ksmm_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.ksmm_version() == 2


def test_struct_layout_matches_header():
    from ksmm_amd import _lib

    assert ctypes.sizeof(_lib.KsmmTile) == 40
    assert ctypes.sizeof(_lib.KsmmFactorDesc) == 32


@pytest.mark.parametrize("args,code", [
    ((25088, 1, 48, 48, 16, 0, 0, 0, 1), 0),
    ((25088, 1, 48, 48, 16, 1, 1, 1, 0), 0),
    ((25088, 1, 16, 16, 64, 2, 2, 1, 1), 0),
    ((25088, 16, 16, 16, 4, 1, 2, 1, 1), 0),
    ((25088, 0, 48, 48, 16, 0, 0, 0, 1), -2),
    ((25088, 1, 48, -1, 16, 0, 0, 0, 1), -2),
    ((0, 1, 48, 48, 16, 0, 0, 0, 1), -3),
    ((25088, 1, 48, 48, 16, 0, 1, 0, 1), -4),      # f32 x with f16 w
    ((25088, 1, 48, 48, 16, 2, 2, 2, 1), -4),      # fp8 output is not provided
    ((25088, 1, 48, 48, 16, 7, 0, 0, 1), -4),
    ((1 << 20, 1, 4096, 4096, 1, 0, 0, 0, 1), -5),
    ((2, 1 << 15, 1 << 15, 1 << 15, 1 << 15, 0, 0, 0, 1), -5),
])
def test_validate_codes(lib, args, code):
    assert lib.ksmm_validate(*args) == code
    assert lib.ksmm_strerror(code)


def test_strerror_distinct(lib):
    msgs = {lib.ksmm_strerror(c) for c in range(0, -12, -1)}
    assert len(msgs) == 12
    assert lib.ksmm_strerror(-99) == b"unknown ksmm status"


def test_query_tile_host_only(lib):
    from ksmm_amd import query_tile

    for prec in (torch.float32, torch.float16, torch.float8_e4m3fn):
        for bs_last in (True, False):
            for pattern in [(1, 48, 48, 16), (4, 192, 192, 1), (1, 17, 33, 2), (64, 16, 16, 1)]:
                t = query_tile(25088, pattern, prec, bs_last=bs_last)
                assert t["algo"] in (1, 2, 3) and t["threads"] > 0 and t["grid"] > 0
                assert t["lds_bytes"] <= 160 * 1024
    # the generic family takes anything
    assert query_tile(3, (1, 17, 33, 2), torch.float32, algo=1)["algo"] == 1


def test_forward_rejects_bad_arguments_without_gpu(lib):
    # null pointers and aliasing are detected before any launch
    f = lib.ksmm_factor_forward
    assert f(None, None, None, 8, 1, 2, 2, 1, 0, 0, 0, 1, 1.0, None) == -1
    assert f(4096, 8192, 4096, 8, 1, 2, 2, 1, 0, 0, 0, 1, 1.0, None) == -11
    assert f(4096, 8192, 4096 + 32, 8, 1, 2, 2, 1, 0, 0, 0, 1, 1.0, None) == -11
    assert lib.ksmm_factor_forward_algo(4096, 8192, 1 << 20, 8, 1, 2, 2, 1, 0, 0, 0, 1, 1.0, 99, -1,
                                        None) == -6


def test_chain_argument_checks(lib):
    from ksmm_amd import _lib

    d = (_lib.KsmmFactorDesc * 2)()
    for i, p in enumerate([(2, 3, 5, 4), (3, 6, 4, 2)]):
        d[i].w = 4096
        d[i].a, d[i].b, d[i].c, d[i].d = p
        d[i].w_dtype, d[i].scale = 0, 1.0
    need = lib.ksmm_chain_workspace(d, 2, 100, 0)
    assert need == 2 * ((24 * 100 * 4 + 255) // 256 * 256)
    assert lib.ksmm_chain_workspace(d, 1, 100, 0) == 0
    assert lib.ksmm_chain_workspace(d, 0, 100, 0) == -10
    # (fake, non-overlapping device addresses: every check below fails before anything is launched)
    x, y, ws = 1 << 20, 2 << 20, 3 << 20
    assert lib.ksmm_chain_forward(d, 2, x, y, None, 0, 100, 0, 0, 1, 1, None) == -9
    # overlapping tensors are refused: y inside x, workspace inside y, misaligned workspace
    assert lib.ksmm_chain_forward(d, 2, x, x + 256, ws, need, 100, 0, 0, 1, 1, None) == -11
    assert lib.ksmm_chain_forward(d, 2, x, y, y + 512, need, 100, 0, 0, 1, 1, None) == -11
    assert lib.ksmm_chain_forward(d, 2, x, y, ws + 4, need, 100, 0, 0, 1, 1, None) == -9
    ep = _lib.KsmmEpilogue(None, 7)
    import ctypes
    assert lib.ksmm_chain_forward_ep(d, 2, x, y, ws, need, 100, 0, 0, 1, 1, ctypes.byref(ep), None) == -12
    # the static-scratch entry point refuses chains that need more than its fixed array
    assert lib.ksmm_static_scratch_bytes() == 32 << 20
    assert lib.ksmm_chain_workspace_layout(d, 2, 1 << 20, 0, 0, 1) > lib.ksmm_static_scratch_bytes()
    assert lib.ksmm_chain_forward_static(d, 2, x, 1 << 40, 1 << 20, 0, 0, 1, 1, None, None) == -9
    # chains that take the transposed (batch-size-first, strided blocks) or the padded-rows route
    # (batch-size-last, batch off the vector) ask for more than ksmm_chain_workspace(): with less
    # they are refused, like ksmm_factor_forward_ws, instead of falling back to a slow kernel
    t = (_lib.KsmmFactorDesc * 1)()
    t[0].w, t[0].w_dtype, t[0].scale = 4096, 1, 1.0
    t[0].a, t[0].b, t[0].c, t[0].d = 1, 192, 192, 12
    big = lib.ksmm_chain_workspace_layout(t, 1, 1024, 1, 1, 0)
    assert big > 0 and lib.ksmm_chain_workspace(t, 1, 1024, 1) == 0
    x2, y2, ws2 = 1 << 30, 2 << 30, 3 << 30
    assert lib.ksmm_chain_forward(t, 1, x2, y2, None, 0, 1024, 1, 1, 0, 1, None) == -9
    assert lib.ksmm_chain_forward(t, 1, x2, y2, ws2, big - 256, 1024, 1, 1, 0, 1, None) == -9
    t[0].a, t[0].b, t[0].c, t[0].d = 1, 48, 48, 16
    pad = lib.ksmm_chain_workspace_layout(t, 1, 1003, 1, 1, 1)
    assert pad > 0
    assert lib.ksmm_chain_forward(t, 1, x2, y2, ws2, pad - 256, 1003, 1, 1, 1, 1, None) == -9
    d[1].c = 5  # 3*5*2 = 30 != 24
    assert lib.ksmm_chain_forward(d, 2, x, y, ws, need, 100, 0, 0, 1, 1, None) == -8
    assert lib.ksmm_chain_forward(d, 17, x, y, ws, need, 100, 0, 0, 1, 1, None) == -10


def test_kslinear_constructor_contract():
    from ksmm_amd import KSLinear

    with pytest.raises(Exception, match="kernel expects device='cuda'"):
        KSLinear([(1, 2, 2, 1)], algo="kernel", device="cpu")      # interface.py:163-164
    with pytest.raises(AssertionError):
        KSLinear([(1, 2, 2, 1)], algo="nope")                      # interface.py:141-148
    with pytest.raises(AssertionError):
        KSLinear([(1, 2, 2)], algo="dense")                        # interface.py:149-150
    with pytest.raises(AssertionError):
        KSLinear([(1, 2, 2, 1)], weights=[None, None], algo="dense")  # interface.py:170
    k = KSLinear([(2, 3, 5, 4), (3, 6, 4, 2)], algo="bmm", dtype=torch.float32, bs_last=True)
    assert (k.in_size, k.out_size, k.num_mat, k.algo, k.bs_last, k.vsize) == (40, 36, 2, "bmm", True, 4)
    assert k.bias.shape == (36, 1)                                  # interface.py:186-189
    assert KSLinear([(2, 3, 5, 4)], algo="dense", dtype=torch.float32).bias.shape == (24,)
    assert [tuple(f.shape) for f in k.factors] == [(8, 3, 5), (6, 6, 4)]
    assert "in_size=40, out_size=36, num_mat=2" in repr(k)


@pytest.mark.parametrize("algo", ["dense", "bmm", "einsum"])
@pytest.mark.parametrize("bs_last", [True, False])
def test_kslinear_torch_algos_match_oracle(algo, bs_last):
    from ksmm_amd import KSLinear

    patterns = [(2, 3, 5, 4), (3, 6, 4, 2)]
    ws = seeded_weights(patterns, seed=0)
    x = seeded_input(40, 9, bs_last, seed=1)
    k = KSLinear(patterns, weights=ws, bias=False, algo=algo, dtype=torch.float32, bs_last=bs_last)
    y = k(x).detach().numpy()
    z = O.chain_apply([w.double().numpy() for w in ws], x.double().numpy(), bs_last)
    assert O.rel_fro_error(y, z) <= 1e-6
    kd = k.get_dense_product().double().numpy()
    assert abs(kd - O.chain_dense([w.double().numpy() for w in ws])).max() <= 1e-6


def test_generate_factor_layouts_match_oracle():
    from ksmm_amd import generate_factor

    p = (2, 3, 5, 4)
    (w4,) = seeded_weights([p], seed=2)
    w = w4.numpy()
    assert (generate_factor(*p, "kernel", w4, torch.float32).numpy() == O.pack_kernel_format(w)).all()
    assert (generate_factor(*p, "bmm", w4, torch.float32).numpy() == O.pack_bmm_format(w)).all()
    assert (generate_factor(*p, "dense", w4, torch.float32).numpy() == O.ks_dense(w)).all()
    f = generate_factor(*p, "kernel", None, torch.float32)
    assert f.shape == (40, 3) and f.abs().max() <= 1 / 5 ** 0.5


def test_nd_input_and_bias_cpu():
    from ksmm_amd import KSLinear

    k = KSLinear([(2, 3, 5, 4)], algo="bmm", dtype=torch.float32, bs_last=False, bias=True)
    x = torch.randn(4, 6, 40)
    y = k(x)
    assert y.shape == (4, 6, 24)
    z = torch.nn.functional.linear(x, k.get_dense_product(), k.bias)
    assert torch.allclose(y, z, atol=1e-5)
    kl = KSLinear([(2, 3, 5, 4)], algo="einsum", dtype=torch.float32, bs_last=True, bias=True)
    xl = torch.randn(40, 4, 6)
    yl = kl(xl)
    assert yl.shape == (24, 4, 6)
    zl = (kl.get_dense_product() @ xl.reshape(40, -1) + kl.bias).reshape(24, 4, 6)
    assert torch.allclose(yl, zl, atol=1e-5)


def test_fp8_torch_algos_use_dequantised_operands():
    from ksmm_amd import KSLinear, quantize_fp8

    patterns = [(1, 16, 16, 4), (4, 16, 16, 1)]
    ws = seeded_weights(patterns, seed=3, bound=0.25)
    x = seeded_input(64, 11, True, seed=4)
    k = KSLinear(patterns, weights=ws, bias=False, algo="dense", dtype=torch.float8_e4m3fn, bs_last=True)
    y = k(x).detach().double().numpy()
    wd = []
    for w in ws:
        q, s = O.fp8_quantize(w.numpy())
        wd.append(O.fp8_dequantize(q, s).reshape(w.shape))
    xq, xs = O.fp8_quantize(x.numpy())
    z = O.chain_apply(wd, O.fp8_dequantize(xq, xs).reshape(x.shape), True)
    assert O.rel_fro_error(y, z) <= 1e-6
    q, s = quantize_fp8(x)
    assert (q.view(torch.uint8).numpy() == xq).all() and abs(float(s) - float(xs)) < 1e-12


def test_kernel_forward_host_checks():
    from ksmm_amd import Kernel

    x = torch.zeros(4, 8)
    w = torch.zeros(8, 2)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):   # kernel.cpp:19
        Kernel.forward(x, w, False, 1, 2, 8, 1)


def test_workspace_queries_need_no_gpu():
    """ksmm_factor_workspace / ksmm_chain_workspace_layout are host-only: 0 for problems with a
    kernel of their own, room for the transposed operands for batch-size-first d > 1 blocks."""
    import ctypes
    from ksmm_amd import _lib

    lib = _lib.load()
    F16 = _lib.KSMM_F16
    assert lib.ksmm_factor_workspace(1024, 4, 192, 192, 1, F16, F16, F16, 0) == 0
    assert lib.ksmm_factor_workspace(1024, 1, 192, 192, 16, F16, F16, F16, 1) == 0
    need = lib.ksmm_factor_workspace(1024, 1, 192, 192, 16, F16, F16, F16, 0)
    assert need == 2 * (192 * 16 * 1024 * 2)
    assert lib.ksmm_factor_workspace(0, 1, 192, 192, 16, F16, F16, F16, 0) == -3
    descs = (_lib.KsmmFactorDesc * 2)()
    for i, (a, b, c, d) in enumerate([(2, 192, 192, 8), (16, 192, 192, 1)]):
        descs[i].w = 0
        descs[i].a, descs[i].b, descs[i].c, descs[i].d = a, b, c, d
        descs[i].w_dtype = F16
        descs[i].scale = 1.0
    plain = lib.ksmm_chain_workspace(descs, 2, 512, F16)
    assert lib.ksmm_chain_workspace_layout(descs, 2, 512, F16, F16, 1) == plain
    assert lib.ksmm_chain_workspace_layout(descs, 2, 512, F16, F16, 0) == 3 * (3072 * 512 * 2)


def test_gelu_constants_of_the_kernel_epilogue():
    """The epilogue's GELU (gelu_erf in ksmm_common.h) is x * Phi(x) with erfc by Abramowitz &
    Stegun 7.1.26 and the formula's factors folded into its constants.  The constants are read
    from the header and the same arithmetic, in float32, is compared with the erf form of
    torch.nn.functional.gelu evaluated in float64 (the ViT feed-forward's activation,
    src/ksmm_py/model/vit.py:416-431): a wrong or mis-folded constant fails this."""
    import math
    import os
    import re

    import torch

    src = open(os.path.join(os.path.dirname(__file__), "..", "ksmm_amd", "csrc", "ksmm_common.h")).read()
    body = src[src.index("float gelu_erf(float x)"):]
    body = body[:body.index("\n}\n")]
    k, p, a5, a4, a3, a2, a1 = [np.float32(v) for v in re.findall(r"(-?\d+\.\d{6,})f", body)]
    assert abs(float(k) - math.sqrt(math.log2(math.e) / 2)) < 1e-7
    x = np.concatenate([np.linspace(-12, 12, 240001), [0.0, -0.0, 1e-20, -1e-20, 60.0, -60.0]]).astype(np.float32)
    ax = np.abs(x)
    z = ax * k
    t = np.float32(1) / (p * z + np.float32(1))
    poly = a5 * t + a4
    for coef in (a3, a2, a1):
        poly = poly * t + coef
    got = np.maximum(x, np.float32(0)) - ax * ((poly * t) * np.exp2(-(z * z)))
    want = torch.nn.functional.gelu(torch.from_numpy(x).double()).numpy()
    assert got.dtype == np.float32
    assert np.abs(got - want).max() <= 5e-7
    assert np.linalg.norm(got - want) <= 1e-7 * np.linalg.norm(want)


def test_unaligned_batch_asks_for_room_for_padded_rows():
    """Batch-size-last rows are `batch` elements long; when that is not a multiple of the
    16-byte vector the library asks for room for the input and the output with rows padded to a
    multiple of 16 columns (the reference refuses shapes without hyper-parameters,
    kernel.py:241-244).  Aligned batches, and batch-size-first, ask for nothing."""
    from ksmm_amd import _lib

    lib = _lib.load()
    F32, F16, F8 = _lib.KSMM_F32, _lib.KSMM_F16, _lib.KSMM_FP8_E4M3
    pad = lambda n: (n + 255) // 256 * 256
    for a, b, c, d in [(1, 48, 48, 16), (6, 64, 64, 1), (1, 768, 192, 2)]:
        assert lib.ksmm_factor_workspace(25088, a, b, c, d, F32, F32, F32, 1) == 0
        assert lib.ksmm_factor_workspace(25092, a, b, c, d, F32, F32, F32, 1) == 0      # 4 floats
        assert lib.ksmm_factor_workspace(25087, a, b, c, d, F32, F32, F32, 0) == 0
        assert lib.ksmm_factor_workspace(25087, a, b, c, d, F32, F32, F32, 1) == \
            pad(a * c * d * 25088 * 4) + pad(a * b * d * 25088 * 4)
        assert lib.ksmm_factor_workspace(25090, a, b, c, d, F16, F16, F16, 1) == \
            pad(a * c * d * 25104 * 2) + pad(a * b * d * 25104 * 2)
        assert lib.ksmm_factor_workspace(25096, a, b, c, d, F16, F16, F16, 1) == 0      # 8 halves
        assert lib.ksmm_factor_workspace(25090, a, b, c, d, F8, F8, F16, 1) == \
            pad(a * c * d * 25104) + pad(a * b * d * 25104 * 2)
    descs = (_lib.KsmmFactorDesc * 2)()
    for i, (a, b, c, d) in enumerate([(6, 64, 64, 1), (1, 768, 192, 2)]):
        descs[i].w = 0
        descs[i].a, descs[i].b, descs[i].c, descs[i].d = a, b, c, d
        descs[i].w_dtype = F32
        descs[i].scale = 1.0
    assert lib.ksmm_chain_workspace_layout(descs, 2, 2000, F32, F32, 1) == lib.ksmm_chain_workspace(descs, 2, 2000, F32)
    assert lib.ksmm_chain_workspace_layout(descs, 2, 2003, F32, F32, 1) == \
        pad(384 * 2016 * 4) + 2 * pad(1536 * 2016 * 4)
    assert lib.ksmm_chain_workspace_layout(descs, 2, 2003, F32, F32, 0) == lib.ksmm_chain_workspace(descs, 2, 2003, F32)


def test_tuned_table_is_sorted_and_every_row_names_a_kernel_that_fits():
    """The measured table (the counterpart of the reference's *.best files, kernel.py:151-257):
    keys strictly ascending (binary search), every row a forced instance that takes the problem
    at the batch it was measured on, and the automatic choice follows it there, not below 8192."""
    from ksmm_amd.kernel import query_tile, tuned_table

    rows = tuned_table()
    keys = [r[:6] for r in rows]
    assert keys == sorted(keys) and len(set(keys)) == len(keys)
    dts = {0: torch.float32, 1: torch.float16, 2: torch.float8_e4m3fn}
    for a, b, c, d, combo, bs_last, algo, variant in rows:
        assert combo in dts and algo in (2, 3) and variant >= 0
        forced = query_tile(25088, (a, b, c, d), dts[combo], None, bool(bs_last), algo, variant)
        auto = query_tile(25088, (a, b, c, d), dts[combo], None, bool(bs_last))
        assert auto == forced, (a, b, c, d, combo, bs_last)
        small = query_tile(4096, (a, b, c, d), dts[combo], None, bool(bs_last))
        heur = query_tile(4096, (a, b, c, d), dts[combo], None, bool(bs_last), variant=-3)
        assert small == heur


def test_wave_row_group_instance_only_when_named():
    """The fp32 wave instance for 32-row blocks takes row groups of a 64- or 96-row block when it
    is forced (or named by a table row); the heuristics keep whole blocks per wave."""
    from ksmm_amd import _lib
    from ksmm_amd.kernel import query_tile

    f32 = torch.float32
    forced = query_tile(25088, (6, 64, 64, 1), f32, None, True, algo=2, variant=7)
    assert forced["tile_m"] == 32 and forced["tile_k"] == 64
    whole = query_tile(25088, (6, 64, 64, 1), f32, None, True, algo=2, variant=-1)
    assert whole["tile_m"] == 64 and (whole["variant"] & 0xff) != 7
    assert forced["grid"] >= whole["grid"]  # twice the waves for the same tiles per wave or fewer
    assert query_tile(25088, (2, 96, 64, 3), f32, None, True, algo=2, variant=7)["tile_m"] == 32
    with pytest.raises(_lib.KsmmError):   # 48 rows are not a multiple of 32
        query_tile(25088, (1, 48, 64, 2), f32, None, True, algo=2, variant=7)
    with pytest.raises(_lib.KsmmError):   # other c
        query_tile(25088, (1, 64, 32, 2), f32, None, True, algo=2, variant=7)


def test_every_pattern_shape_class_has_a_kernel_family():
    """Host-only view of the dispatch for the shape classes of the reference's pattern list that
    used to end on the one-thread-per-output kernel: b not a multiple of 16, c not a multiple of the
    K tile, blocks of a few elements, batch-size-first blocks with d > 1."""
    from ksmm_amd import _lib
    from ksmm_amd.kernel import dtype_code, query_tile

    lib = _lib.load()
    f16, f32, f8 = torch.float16, torch.float32, torch.float8_e4m3fn
    B = 25088
    for dt in (f32, f16, f8):
        for bs_last in (True, False):  # ragged b, d = 1: tiles with a partial last TM-tile
            t = query_tile(B, (64, 460, 64, 1), dt, None, bs_last, variant=-3)
            if bs_last and dt == f32:
                # rows of whole 16-byte vectors (460 floats): the persistent GEMM tiles with a masked last TM-tile
                assert t["algo"] == 3 and (t["variant"] >> 24) == 4 and t["grid"] == 512 and t["tile_m"] == 64, (dt, t)
            else:  # k-loop tiles
                assert t["algo"] == 3 and t["grid"] >= 64 * 98 * 4, (dt, bs_last, t)
        t = query_tile(B, (1, 448, 910, 32), dt, None, True, variant=-3)       # c = 910: partial K slab
        assert t["algo"] == 3 and (t["variant"] >> 24) == 4, (dt, t)
        t = query_tile(B, (1, 2, 4, 7168), dt, None, True, variant=-3)         # tiny block: vector form
        assert (t["algo"], t["variant"]) == (1, 1), (dt, t)
        assert query_tile(B + 1, (1, 2, 4, 7168), dt, None, True, variant=-3)["variant"] == 0   # odd batch
        t = query_tile(B, (1, 48, 48, 32), dt, None, False, variant=-3)        # rows kernel, groups of 16 d_i
        assert t["algo"] == 2 and t["variant"] >= 1000 and t["tile_d"] == 16, (dt, t)
    t = query_tile(B, (1, 768, 192, 16), f8, None, True, variant=-3)           # e4m3 GEMM tiles
    assert t["algo"] == 3 and (t["variant"] >> 24) == 4
    # batch-size-first, big blocks, d a multiple of the 16-byte vector: groups of d_i on the tile_bf kernel
    t = query_tile(B, (1, 192, 192, 16), f16, None, False, variant=-3)
    assert t["algo"] == 3 and (t["variant"] >> 24) == 3 and t["tile_d"] == 8, t
    assert lib.ksmm_factor_workspace(B, 1, 192, 192, 16, dtype_code(f16), dtype_code(f16), dtype_code(f16), 0) == 0
    t = query_tile(B, (1, 128, 128, 8), f32, None, False, variant=-3)
    assert t["algo"] == 3 and (t["variant"] >> 24) == 3 and t["tile_d"] == 4, t
    # fp32 groups out of a large d, and d that is not a multiple of the vector: transposed route
    assert query_tile(B, (1, 256, 256, 32), f32, None, False, variant=-3)["algo"] == 1
    assert query_tile(B, (1, 192, 192, 12), f16, None, False, variant=-3)["algo"] == 1
    assert lib.ksmm_factor_workspace(B, 1, 192, 192, 12, dtype_code(f16), dtype_code(f16), dtype_code(f16), 0) > 0


def test_tuner_emit_keeps_one_sorted_row_per_key_above_the_threshold(tmp_path):
    """ksmm_amd.tune.emit: rows only where the measured winner beats the heuristic by more than
    3 %, one per (pattern, types, layout), sorted for the library's binary search."""
    from ksmm_amd.tune import emit

    def entry(p, prec, bs_last, auto, best, algo=3, variant=5):
        return {"pattern": list(p), "prec": prec, "bs_last": bs_last, "auto_us": auto, "best_us": best,
                "algo": algo, "variant": variant}

    entries = [entry((2, 64, 64, 1), "fp16", True, 10.0, 9.0, 2, 0),
               entry((1, 48, 48, 16), "fp32", True, 10.0, 9.9),            # within 3 %: dropped
               entry((1, 48, 48, 16), "fp32", False, 10.0, 8.0, 2, 1000),
               entry((2, 64, 64, 1), "fp16", True, 10.0, 8.5, 2, 1),        # duplicate key: the faster one
               entry((4, 64, 64, 1), "fp16", True, 10.0, 5.0, 3, 5),        # a kernel that does not take it: dropped
               entry((1, 16, 16, 4), "fp8", True, None, None, 0, -1)]       # nothing measured
    path = tmp_path / "t.inc"
    assert emit(entries, str(path), 25088) == 2
    rows = [l for l in path.read_text().splitlines() if l.startswith("{")]
    # rows name the kernel by stable instance id and parameter, not by table position
    from ksmm_amd.kernel import variant_from_id, variant_id

    assert rows[0].startswith("{1, 48, 48, 16, 0, 0, 2, %du, %d}" % variant_id(2, 1000, 0, False))
    assert rows[1].startswith("{2, 64, 64, 1, 1, 1, 2, %du, %d}" % variant_id(2, 1, 1, True))
    # an id recorded at measuring time wins over the (positional) variant when it still names a
    # kernel with the recorded tile; a stale variant alone must not be trusted
    iid, par = variant_id(2, 1, 1, True)
    moved = dict(entry((2, 64, 64, 1), "fp16", True, 10.0, 8.0, 2, 0), id=iid, param=par,
                 tile={"tile_m": 64, "tile_n": 128, "tile_k": 64, "tile_d": 1, "threads": 256})
    assert emit([moved], str(path), 25088) == 1
    row = [l for l in path.read_text().splitlines() if l.startswith("{")][0]
    assert row.startswith("{2, 64, 64, 1, 1, 1, 2, %du, %d}" % (iid, par))
    assert variant_from_id(2, iid, par, 1, True) == 1


def test_tuner_best_files_have_the_reference_columns(tmp_path):
    """ksmm_amd.tune.emit_best: `batch a b c d <kernel> ms std mse` per pattern, one file per
    element type and layout, named like the reference's *.best files."""
    from ksmm_amd.tune import emit_best

    e = {"pattern": [1, 48, 48, 16], "prec": "fp32", "bs_last": True, "batch": 25088, "auto_us": 35.0,
         "auto_mean_us": 35.5, "auto_std_us": 0.2, "auto_mse": 1e-14, "bound_us": 19.3, "best_us": 34.0,
         "best_mean_us": 34.2, "best_std_us": 0.1, "algo": 2, "variant": 0x700, "id": 12345, "param": 7,
         "mse": 2e-14, "tile": {"tile_m": 48, "tile_n": 64, "tile_k": 48, "tile_d": 1, "threads": 256},
         "auto_tile": {"algo": 2, "tile_m": 48, "tile_n": 64, "tile_k": 48, "tile_d": 1, "threads": 256}}
    slow = dict(e, pattern=[2, 64, 64, 1], best_us=40.0)      # the heuristic choice is the faster one
    written = emit_best([e, slow], str(tmp_path))
    assert written == {"kernel_bs_last_float.best": 2}
    lines = (tmp_path / "kernel_bs_last_float.best").read_text().splitlines()
    assert lines[0].startswith("# batch a b c d family instance_id parameter")
    f = lines[1].split()
    from ksmm_amd.kernel import variant_id

    iid, par = variant_id(2, 0x700, 0, True)   # ids come from (family, variant) with the library at hand
    assert f[:8] == ["25088", "1", "48", "48", "16", "wave", str(iid), str(par)] and par == 7
    assert float(f[13]) == pytest.approx(0.0342) and float(f[14]) == pytest.approx(0.0001) and float(f[15]) == 2e-14
    g = lines[2].split()
    assert g[:8] == ["25088", "2", "64", "64", "1", "wave", "0", "0"] and float(g[13]) == pytest.approx(0.0355)


def test_instance_ids_are_unique_and_round_trip(lib):
    """Every instance of every family has its own id inside the set a table row is resolved in
    (family x element types x layout), and (id, parameter) -> variant -> (id, parameter) is the
    identity; every row of the compiled table still names an instance of this build."""
    from ksmm_amd import _lib
    from ksmm_amd.kernel import tuned_table, variant_from_id, variant_id
    from ksmm_amd.tune import candidates, kloop_candidates

    for combo in (0, 1, 2, 3):
        for bs_last in (True, False):
            seen = {}
            for algo, variant in candidates(bs_last, combo) + kloop_candidates(combo, bs_last) + [(1, 0), (1, 1)]:
                iid, par = variant_id(algo, variant, combo, bs_last)
                assert variant_from_id(algo, iid, par, combo, bs_last) == variant, (combo, bs_last, algo, hex(variant))
                key = (algo, iid)
                inst = variant & 0xff if algo != 2 or bs_last else (variant - 1000) & 0x3ff
                sub = (variant >> 24) if algo == 3 else 0
                assert seen.setdefault(key, (sub, inst)) == (sub, inst), ("id collision", combo, bs_last, key)
    rows = tuned_table(full=True)
    assert len(rows) >= 700
    assert all(r[9] >= 0 for r in rows), [r for r in rows if r[9] < 0][:3]
    with pytest.raises(_lib.KsmmError):
        variant_from_id(3, 12345, 0, 1, True)


def test_kernel_format_converters_match_oracle():
    """from_kernel_format_to_dense / from_bmm_format_to_dense / from_abcd_to_dense on asymmetric
    patterns against the oracle's dense form (interface.py:75-113)."""
    from ksmm_amd.layer import (from_abcd_to_dense, from_bmm_format_to_dense, from_kernel_format_to_abcd,
                                from_kernel_format_to_dense, generate_factor)

    for pattern in [(2, 3, 5, 4), (3, 2, 2, 1), (1, 4, 3, 2), (2, 6, 4, 3)]:
        a, b, c, d = pattern
        w4 = torch.arange(a * b * c * d, dtype=torch.float64).reshape(a, b, c, d) + 1
        dense = O.ks_dense(w4.numpy())
        fk = generate_factor(a, b, c, d, "kernel", w4, torch.float64, "cpu")
        assert fk.shape == (a * d * c, b)
        assert torch.equal(from_kernel_format_to_abcd(fk, pattern), w4)
        assert np.array_equal(from_kernel_format_to_dense(fk, pattern).numpy(), dense)
        fb = generate_factor(a, b, c, d, "bmm", w4, torch.float64, "cpu")
        assert np.array_equal(from_bmm_format_to_dense(fb, pattern).numpy(), dense)
        assert np.array_equal(from_abcd_to_dense(w4).numpy(), dense)


def test_get_dense_product_of_a_kernel_format_layer_on_cpu_tensors():
    """get_dense_product() reads the kernel-format parameters: build the layer's parameters by
    hand (algo='kernel' itself needs a device) and compare with the oracle's chain product."""
    from ksmm_amd import KSLinear, generate_factor

    patterns = [(2, 3, 5, 4), (3, 6, 4, 2)]
    ws4 = seeded_weights(patterns, seed=9)
    ksl = KSLinear(patterns, weights=ws4, bias=False, algo="einsum", dtype=torch.float64)
    # swap in kernel-format storage: the dense product must not change
    want = O.chain_dense([w.double().numpy() for w in ws4])
    assert np.allclose(ksl.get_dense_product().numpy(), want, rtol=0, atol=1e-12)
    ksl.algo = "kernel"
    for i, (p, w) in enumerate(zip(patterns, ws4)):
        ksl.factors[i] = torch.nn.Parameter(generate_factor(*p, "kernel", w, torch.float64, "cpu"))
    assert np.allclose(ksl.get_dense_product().numpy(), want, rtol=0, atol=1e-12)


def test_wave_family_refuses_offsets_beyond_32_bits(lib):
    """The wave kernels address rows with 32-bit per-lane byte offsets; the largest one formed
    on the output side is (12*d*B + B) elements.  (1,16,16,4096) fp32 at B = 25088 passes the
    shape check but would wrap: the family must refuse it (another family takes it)."""
    from ksmm_amd.kernel import query_tile
    from ksmm_amd import _lib

    assert lib.ksmm_validate(25088, 1, 16, 16, 4096, 0, 0, 0, 1) == 0
    with pytest.raises(_lib.KsmmError) as e:
        query_tile(25088, (1, 16, 16, 4096), torch.float32, None, True, algo=_lib.ALGO_WAVE)
    assert e.value.status == -6
    assert query_tile(25088, (1, 16, 16, 4096), torch.float32, None, True)["algo"] != _lib.ALGO_WAVE
    # just below the limit the family still takes the shape: 12*d*B*4 + 4*B < 2^32
    assert query_tile(25088, (1, 16, 16, 3500), torch.float32, None, True, algo=_lib.ALGO_WAVE)["algo"] == 2
    # 16-bit outputs: 24*d*B + 2*B bytes stays below 2^32 for every shape the 2^31-element limit lets in
    assert query_tile(25088, (1, 16, 16, 5300), torch.float16, None, True, algo=_lib.ALGO_WAVE)["algo"] == 2


def test_row_kernel_variants_round_trip(lib):
    """What ksmm_query_tile reports for the batch-size-first row kernels can be forced back to
    the same tile, for every element type (the instance field holds every index)."""
    from ksmm_amd.kernel import query_tile
    from ksmm_amd import _lib

    seen = set()
    for dt in (torch.float32, torch.float16, torch.float8_e4m3fn):
        for pattern in [(1, 48, 48, 8), (1, 48, 48, 16), (2, 64, 64, 4), (1, 96, 96, 4), (1, 192, 48, 3),
                        (1, 48, 192, 4), (1, 64, 64, 16), (1, 48, 48, 2)]:
            t = query_tile(25088, pattern, dt, None, False, algo=_lib.ALGO_WAVE)
            assert t["variant"] >= 1000
            again = query_tile(25088, pattern, dt, None, False, algo=_lib.ALGO_WAVE, variant=t["variant"])
            assert again == t, (dt, pattern, t, again)
            seen.add(t["variant"] - 1000)
    assert max(seen) >= 128  # instances beyond the old 7-bit field are reachable
    # an index outside the table is refused, not aliased to another instance
    with pytest.raises(_lib.KsmmError):
        query_tile(25088, (1, 48, 48, 8), torch.float32, None, False, algo=_lib.ALGO_WAVE, variant=1000 + 1000)


def test_unaligned_tensors_are_refused_by_forced_families(lib):
    """Pointer checks happen before any launch: a forced vector family refuses tensors that do
    not start on a 16-byte boundary (the automatic choice would run the scalar kernel)."""
    f = lib.ksmm_factor_forward_algo
    assert f(4096 + 4, 1 << 20, 2 << 20, 64, 1, 16, 16, 1, 0, 0, 0, 1, 1.0, 2, -1, None) == -6
    assert f(4096, (1 << 20) + 8, 2 << 20, 64, 1, 16, 16, 1, 0, 0, 0, 1, 1.0, 3, -1, None) == -6


def test_bench_csv_writes_the_reference_schema_and_replaces_rows(tmp_path, capsys):
    """python -m ksmm_amd.bench_csv: the reference's CSV columns (ksmm_time.py:61-67), one row per
    configuration (a second run of the same configuration replaces its row), --correctness
    prints the relative error against the dense product, and the feed-forward granularity."""
    import csv

    from ksmm_amd import bench_csv

    out = tmp_path / "res" / "t.csv"
    base = ["--saving-csv", str(out), "--device", "cpu", "--precision", "fp32", "--batch-size", "16",
            "--min-run-time", "0.01"]
    bench_csv.main(base + ["--patterns", "2,3,5,4", "3,6,4,2", "--algo", "bmm", "--bs-last", "1", "--correctness"])
    printed = capsys.readouterr().out
    err = float(re.search(r"Relative error = ([0-9.e+-]+)", printed).group(1))
    assert err < 1e-5
    bench_csv.main(base + ["--patterns", "2,3,5,4", "3,6,4,2", "--algo", "bmm", "--bs-last", "1"])      # same key
    bench_csv.main(base + ["--patterns", "2,3,5,4", "3,6,4,2", "--algo", "einsum", "--bs-last", "0"])
    bench_csv.main(base + ["--granularity", "ffn", "--patterns_up", "2,6,4,1", "--patterns_down", "2,4,6,1",
                           "--algo", "dense", "--correctness"])
    assert float(re.search(r"Relative error = ([0-9.e+-]+)", capsys.readouterr().out).group(1)) < 1e-5
    rows = list(csv.DictReader(open(out)))
    assert list(rows[0].keys()) == ["pattern", "batch-size", "algo", "bs_position", "precision", "vsize",
                                    "device_name", "mean", "median", "iqr", "times"]
    assert len(rows) == 3
    assert rows[0]["pattern"] == "[[2, 3, 5, 4], [3, 6, 4, 2]]" and rows[0]["bs_position"] == "bs_last"
    assert rows[1]["algo"] == "einsum" and rows[1]["bs_position"] == "bs_first"
    assert rows[2]["pattern"].startswith("ffn:") and float(rows[2]["median"]) > 0
    # a file without the expected columns is refused, as the reference does
    bad = tmp_path / "bad.csv"
    bad.write_text("a,b\n1,2\n")
    with pytest.raises(ValueError):
        bench_csv.main(["--saving-csv", str(bad), "--device", "cpu", "--patterns", "2,3,5,4", "--algo", "bmm",
                        "--min-run-time", "0.01"])
