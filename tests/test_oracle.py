"""Pins the CPU oracle.  The reference ships no golden vectors for this path, so each
oracle function is checked against the five-loop definition on asymmetric patterns, against
special cases that reduce to library routines, and against closed forms."""
import numpy as np
import pytest

from oracle import c_oracle
from oracle import ks_oracle as O

ASYM = [(2, 3, 5, 4), (3, 2, 2, 1), (1, 4, 3, 2), (2, 6, 4, 3), (1, 1, 1, 1), (4, 1, 3, 2)]


def _rand(pattern, n, seed=0):
    a, b, c, d = pattern
    rng = np.random.default_rng(seed)
    w4 = rng.integers(-4, 5, size=(a, b, c, d)).astype(np.float64)
    x = rng.integers(-4, 5, size=(a * c * d, n)).astype(np.float64)
    return w4, x


@pytest.mark.parametrize("pattern", ASYM)
@pytest.mark.parametrize("bs_last", [True, False])
def test_algorithms_match_definition(pattern, bs_last):
    w4, x = _rand(pattern, 7)
    xin = x if bs_last else x.T.copy()
    z = O.ks_apply_loops(w4, xin, bs_last)
    for fn in (O.ks_apply_dense, O.ks_apply_bmm, O.ks_apply_einsum):
        np.testing.assert_array_equal(fn(w4, xin, bs_last), z)  # integer data: exact
    wk = O.pack_kernel_format(w4)
    np.testing.assert_array_equal(O.ks_apply_kernel_format(wk, pattern, xin, bs_last), z)
    np.testing.assert_array_equal(c_oracle.factor(xin, wk, pattern, bs_last), z)
    np.testing.assert_array_equal(
        c_oracle.factor(xin.astype(np.float32), wk.astype(np.float32), pattern, bs_last), z)


@pytest.mark.parametrize("pattern", ASYM)
def test_layouts(pattern):
    a, b, c, d = pattern
    w4, _ = _rand(pattern, 1, seed=1)
    wk = O.pack_kernel_format(w4)
    wb = O.pack_bmm_format(w4)
    kd = O.ks_dense(w4)
    assert wk.shape == (a * d * c, b) and wb.shape == (a * d, b, c)
    for ai in range(a):
        for bi in range(b):
            for ci in range(c):
                for di in range(d):
                    v = w4[ai, bi, ci, di]
                    assert wk[(ai * d + di) * c + ci, bi] == v
                    assert wb[ai * d + di, bi, ci] == v
                    assert kd[(ai * b + bi) * d + di, (ai * c + ci) * d + di] == v
    assert np.count_nonzero(kd) <= a * b * c * d
    np.testing.assert_array_equal(O.unpack_kernel_format(wk, pattern), w4)


def test_dense_support_is_kronecker():
    # all-ones weights: K == I_a (x) 1_{b x c} (x) I_d   (interface.py:120-122)
    a, b, c, d = 2, 3, 5, 4
    k = O.ks_dense(np.ones((a, b, c, d)))
    ref = np.kron(np.eye(a), np.kron(np.ones((b, c)), np.eye(d)))
    np.testing.assert_array_equal(k, ref)


def test_special_case_plain_linear():
    rng = np.random.default_rng(2)
    w = rng.standard_normal((6, 5))
    x = rng.standard_normal((5, 9))
    np.testing.assert_allclose(O.ks_apply_einsum(w[None, :, :, None], x, True), w @ x, rtol=1e-13)
    np.testing.assert_allclose(O.ks_apply_bmm(w[None, :, :, None], x.T.copy(), False), x.T @ w.T,
                               rtol=1e-13)


def test_special_case_block_diagonal():
    rng = np.random.default_rng(3)
    a, b, c = 3, 4, 2
    w = rng.standard_normal((a, b, c))
    x = rng.standard_normal((a * c, 5))
    ref = np.concatenate([w[i] @ x[i * c:(i + 1) * c] for i in range(a)], axis=0)
    for fn in (O.ks_apply_dense, O.ks_apply_bmm, O.ks_apply_einsum):
        np.testing.assert_allclose(fn(w[..., None], x, True), ref, rtol=1e-13, atol=1e-13)


def test_special_case_kron_identity():
    rng = np.random.default_rng(4)
    b, c, d = 3, 4, 5
    w = rng.standard_normal((b, c))
    w4 = np.broadcast_to(w[None, :, :, None], (1, b, c, d)).copy()
    np.testing.assert_allclose(O.ks_dense(w4), np.kron(w, np.eye(d)), rtol=0, atol=0)
    x = rng.standard_normal((c * d, 6))
    np.testing.assert_allclose(O.ks_apply_bmm(w4, x, True), np.kron(w, np.eye(d)) @ x, rtol=1e-12,
                               atol=1e-12)


def test_special_case_elementwise_scale():
    rng = np.random.default_rng(5)
    a, d = 3, 4
    s = rng.standard_normal((a, 1, 1, d))
    x = rng.standard_normal((a * d, 5))
    np.testing.assert_allclose(O.ks_apply_einsum(s, x, True), s.reshape(-1, 1) * x, rtol=1e-14)


def test_all_ones_sums_c_inputs():
    a, b, c, d = 2, 3, 4, 2
    rng = np.random.default_rng(6)
    x = rng.standard_normal((a * c * d, 3))
    y = O.ks_apply_bmm(np.ones((a, b, c, d)), x, True).reshape(a, b, d, 3)
    ref = x.reshape(a, c, d, 3).sum(axis=1)
    for bi in range(b):
        np.testing.assert_allclose(y[:, bi], ref, rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("bs_last", [True, False])
def test_chain_order_and_dense_product(bs_last):
    # non-square chain: order matters, sizes 2*5*4=40 -> 24 -> 36
    p0, p1 = (2, 3, 5, 4), (3, 6, 4, 2)
    rng = np.random.default_rng(7)
    w0 = rng.standard_normal(p0)
    w1 = rng.standard_normal(p1)
    x = rng.standard_normal((40, 5))
    xin = x if bs_last else x.T.copy()
    y = O.chain_apply([w0, w1], xin, bs_last)
    kd = O.chain_dense([w0, w1])
    assert kd.shape == (36, 40)
    ref = kd @ x
    np.testing.assert_allclose(y if bs_last else y.T, ref, rtol=1e-12, atol=1e-12)
    ref2 = O.ks_dense(w1) @ (O.ks_dense(w0) @ x)
    np.testing.assert_allclose(ref, ref2, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("log2n", [3, 6, 10])
def test_butterfly_chain_is_walsh_hadamard(log2n):
    ws = O.hadamard_butterfly_weights(log2n)
    n = 2 ** log2n
    if log2n <= 6:
        np.testing.assert_array_equal(O.chain_dense(ws), O.sylvester_hadamard(log2n))
    rng = np.random.default_rng(8)
    x = rng.integers(-3, 4, size=(n, 4)).astype(np.float64)
    y = O.chain_apply(ws, x, True, apply=O.ks_apply_bmm)
    np.testing.assert_array_equal(y, O.sylvester_hadamard(log2n) @ x)


def test_radix16_chain_config5_is_kron_product():
    # the 3-factor 1024 chain of the fp8 configuration with H_16 blocks equals the product of
    # explicit Kronecker products (H16 (x) I64) ... applied right to left
    h16 = O.sylvester_hadamard(4)
    pats = [(1, 16, 16, 64), (16, 16, 16, 4), (64, 16, 16, 1)]
    ws = [np.broadcast_to(h16[None, :, :, None], p).copy() for p in pats]
    rng = np.random.default_rng(9)
    x = rng.integers(-3, 4, size=(1024, 3)).astype(np.float64)
    y = O.chain_apply(ws, x, True)
    k0 = np.kron(h16, np.eye(64))
    k1 = np.kron(np.eye(16), np.kron(h16, np.eye(4)))
    k2 = np.kron(np.eye(64), h16)
    np.testing.assert_array_equal(y, k2 @ (k1 @ (k0 @ x)))


def test_linearity_and_layout_transpose():
    p = (2, 3, 5, 4)
    rng = np.random.default_rng(10)
    w4 = rng.standard_normal(p)
    x = rng.standard_normal((40, 6))
    z = rng.standard_normal((40, 6))
    f = lambda t: O.ks_apply_bmm(w4, t, True)
    np.testing.assert_allclose(f(2 * x - 3 * z), 2 * f(x) - 3 * f(z), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.ks_apply_bmm(w4, x.T.copy(), False), f(x).T, rtol=1e-13, atol=1e-13)


def test_e4m3fn_table_matches_torch():
    import torch

    tab = O.e4m3fn_decode_table()
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).to(torch.float64).numpy()
    assert np.array_equal(np.isnan(tab), np.isnan(ref))
    np.testing.assert_array_equal(tab[~np.isnan(tab)], ref[~np.isnan(ref)])
    assert np.nanmax(tab) == 448.0


def test_e4m3fn_encode_matches_torch():
    import torch

    rng = np.random.default_rng(11)
    v = np.concatenate([rng.standard_normal(20000) * 60, rng.uniform(-448, 448, 20000),
                        O.e4m3fn_decode_table()[:0x7F],           # exact points
                        (O.e4m3fn_decode_table()[:0x7E] + O.e4m3fn_decode_table()[1:0x7F]) / 2,  # ties
                        np.array([0.0, -0.0, 1e-9, -1e-9, 2.0 ** -10, 448.0, -448.0])]).astype(np.float32)
    v = v[np.abs(v) <= 448]
    ours = O.e4m3fn_encode(v)
    ref = torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(ours, ref)


def test_fp8_quantize_roundtrip():
    rng = np.random.default_rng(12)
    t = rng.standard_normal(5000).astype(np.float32)
    q, s = O.fp8_quantize(t)
    back = O.fp8_dequantize(q, s)
    assert np.max(np.abs(back - t) / np.maximum(np.abs(t), float(s) * 2.0 ** -6)) <= 2.0 ** -4 + 1e-6
    assert abs(float(s) - np.max(np.abs(t)) / 448) < 1e-9


def test_torch_bmm_restatement_matches():
    import torch

    for p in ASYM:
        for bs_last in (True, False):
            w4, x = _rand(p, 5, seed=13)
            xin = x if bs_last else x.T.copy()
            wb = torch.from_numpy(O.pack_bmm_format(w4))
            y = O.torch_bmm_forward(wb, torch.from_numpy(xin), p, bs_last).numpy()
            np.testing.assert_array_equal(y, O.ks_apply_loops(w4, xin, bs_last))


def test_rel_fro_error_closed_forms():
    """The metric every parity assertion rests on, on values that can be worked out by hand."""
    z = np.array([[3.0, 4.0], [0.0, 0.0]])                 # ||z|| = 5
    assert O.rel_fro_error(z, z) == 0.0
    assert O.rel_fro_error(z + np.array([[0.0, 0.0], [0.3, 0.4]]), z) == pytest.approx(0.1, rel=1e-12)
    assert O.rel_fro_error(1.01 * z, z) == pytest.approx(0.01, rel=1e-9)      # relative: scale-free
    assert O.rel_fro_error(np.zeros_like(z), z) == pytest.approx(1.0, rel=1e-12)
    # not symmetric: the second argument is the reference
    assert O.rel_fro_error(z, 2 * z) == pytest.approx(0.5, rel=1e-12)
    assert O.rel_fro_error(2 * z, z) == pytest.approx(1.0, rel=1e-12)


@pytest.mark.parametrize("tol_name", ["fp32", "fp16", "fp8"])
def test_checker_fails_on_plausible_mistakes(tol_name):
    """Negative controls: the mistakes a kernel is likely to make must exceed every tolerance
    class, i.e. the parity tests can fail.  One swapped pair of weight blocks, one transposed
    block, one wrong d index, one dropped k term, one stale output row."""
    from tests.util import TOL

    tol = TOL[tol_name]
    pattern = (2, 48, 48, 16)
    a, b, c, d = pattern
    w4, x = _rand(pattern, 64, seed=5)
    z = O.ks_apply_einsum(w4, x, True)
    bad = {}
    w = w4.copy(); w[[0, 1]] = w[[1, 0]]; bad["swapped a blocks"] = O.ks_apply_einsum(w, x, True)
    w = w4.copy(); w[0, :, :, 3] = w4[0, :, :, 3].T; bad["one transposed block"] = O.ks_apply_einsum(w, x, True)
    w = w4.copy(); w[:, :, :, 5] = w4[:, :, :, 6]; bad["wrong d index"] = O.ks_apply_einsum(w, x, True)
    w = w4.copy(); w[:, :, c - 1, :] = 0; bad["dropped last k term"] = O.ks_apply_einsum(w, x, True)
    y = z.copy(); y[17] = 0; bad["one of 1536 output rows missing"] = y
    y = z.copy(); y[:, 63] = z[:, 62]; bad["one of 64 columns stale"] = y
    for name, y in bad.items():
        assert O.rel_fro_error(y, z) > tol, (name, O.rel_fro_error(y, z), tol)
    # and rounding of the size the storage types produce stays inside
    noise = {"fp32": 2.0 ** -24, "fp16": 2.0 ** -11, "fp8": 2.0 ** -11}[tol_name]
    rng = np.random.default_rng(0)
    y = z * (1 + noise * rng.uniform(-1, 1, z.shape))
    assert O.rel_fro_error(y, z) <= tol


@pytest.mark.parametrize("bs_last", [True, False])
@pytest.mark.parametrize("pattern", [(2, 3, 5, 4), (1, 4, 3, 2), (3, 2, 2, 1)])
def test_backward_matches_autograd_on_the_dense_form(pattern, bs_last):
    """ks_backward against torch autograd through the explicit dense matrix (float64): dX is
    K^T dY, dW is the gradient of the dense matrix read back on the factor's support; and a
    central finite difference of one weight and one input entry."""
    import torch

    a, b, c, d = pattern
    w4, x = _rand(pattern, 7, seed=3)
    if not bs_last:
        x = x.T.copy()
    rng = np.random.default_rng(4)
    dy = rng.standard_normal((a * b * d, 7)) if bs_last else rng.standard_normal((7, a * b * d))
    dx, dw = O.ks_backward(w4, x, dy, bs_last)
    with torch.enable_grad():
        K = torch.tensor(O.ks_dense(w4), requires_grad=True)
        xt = torch.tensor(x, requires_grad=True)
        y = K @ xt if bs_last else xt @ K.T
        (y * torch.tensor(dy)).sum().backward()
    assert np.allclose(dx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)
    # dense gradient -> (a,b,c,d): entry ((i*b+j)*d+l, (i*c+k)*d+l)
    gK = K.grad.numpy()
    want = np.zeros_like(w4)
    for i in range(a):
        for j in range(b):
            for k in range(c):
                for l in range(d):
                    want[i, j, k, l] = gK[(i * b + j) * d + l, (i * c + k) * d + l]
    assert np.allclose(dw, want, rtol=1e-12, atol=1e-12)
    f = lambda w, xx: float((O.ks_apply_einsum(w, xx, bs_last) * dy).sum())
    eps = 1e-6
    wp, wm = w4.copy(), w4.copy()
    wp[a - 1, b - 1, 0, d - 1] += eps
    wm[a - 1, b - 1, 0, d - 1] -= eps
    assert (f(wp, x) - f(wm, x)) / (2 * eps) == pytest.approx(dw[a - 1, b - 1, 0, d - 1], rel=1e-6)
    xp, xm = x.copy(), x.copy()
    idx = (1, 2) if bs_last else (2, 1)
    xp[idx] += eps
    xm[idx] -= eps
    assert (f(w4, xp) - f(w4, xm)) / (2 * eps) == pytest.approx(dx[idx], rel=1e-6)
