"""CPU oracle for the Kronecker-sparse (KS) hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it is the checker used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``.  It restates, in numpy float64 (plus one torch restatement of the
``bmm`` data movement used as the timed CPU baseline), what the reference computes
on the path ``KSLinear(algo=...)`` -> per-factor product -> factor chain.

A KS factor with pattern ``(a, b, c, d)`` has the 4-D weight ``W[a, b, c, d]`` and maps

    y[a_i, b_i, d_i, n] = sum_{c_i} W[a_i, b_i, c_i, d_i] * x[a_i, c_i, d_i, n]

with input feature index ``(a_i*c + c_i)*d + d_i`` and output feature index
``(a_i*b + b_i)*d + d_i``.

Reference statements restated here (file:line under the reference tree):
  * dense form                      src/ksmm_py/layer/kronecker_sparse/interface.py:108-113
  * kernel weight format (a*d*c,b)  src/ksmm_py/layer/kronecker_sparse/interface.py:65-69, 75-86
  * bmm weight format (a*d,b,c)     src/ksmm_py/layer/kronecker_sparse/interface.py:31-36
  * bmm forward, both layouts       src/ksmm_py/layer/bmm/forward_bmm.py:38-69
  * einsum forward                  src/ksmm_py/layer/kronecker_sparse/interface.py:254-264, 332-342
  * dense forward                   src/ksmm_py/layer/kronecker_sparse/interface.py:252-253, 330-331
  * chain order / dense product     src/ksmm_py/layer/kronecker_sparse/interface.py:193-345, 434-436
  * stand-alone CPU triple loop     src/ksmm_cu/src/template_sparse_mm.cu:813-842
  * error metric                    scripts/example.py:22-23, src/ksmm_py/benchmark/ksmm_time.py:163

How each function is pinned (see tests/test_oracle.py): the reference ships no golden
vectors for this path, so every function is checked against the five-loop definition
``ks_apply_loops`` on asymmetric patterns, against special cases that reduce to library
routines (``np.kron``, block-diagonal matmul, plain matmul, elementwise scale, all-ones
weights), against the Walsh-Hadamard closed form for the butterfly chain, and against
each other (dense == bmm == einsum == kernel-format).  The fp8 decode table is checked
exhaustively against ``torch.float8_e4m3fn``.  No function here is "parity unpinned".
"""
from __future__ import annotations

import math

import numpy as np

# ----------------------------------------------------------------------------------------
# definition (tiny cases only): the five nested loops
# ----------------------------------------------------------------------------------------

def ks_apply_loops(w4, x, bs_last):
    """y = K x straight from the support I_a (x) 1_{b x c} (x) I_d, pure Python loops.

    ``w4``: (a, b, c, d); ``x``: (a*c*d, n) if ``bs_last`` else (n, a*c*d).
    Follows the definition in interface.py:120-122 and the index walk of
    template_sparse_mm.cu:813-842.  Use only on tiny inputs.
    """
    w4 = np.asarray(w4, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    a, b, c, d = w4.shape
    xt = x if bs_last else x.T
    n = xt.shape[1]
    assert xt.shape[0] == a * c * d
    y = np.zeros((a * b * d, n), dtype=np.float64)
    for ai in range(a):
        for bi in range(b):
            for di in range(d):
                row = (ai * b + bi) * d + di
                for ci in range(c):
                    col = (ai * c + ci) * d + di
                    wv = w4[ai, bi, ci, di]
                    for ni in range(n):
                        y[row, ni] += wv * xt[col, ni]
    return y if bs_last else y.T


# ----------------------------------------------------------------------------------------
# storage layouts
# ----------------------------------------------------------------------------------------

def ks_dense(w4):
    """Dense (a*b*d, a*c*d) matrix of a factor given as (a,b,c,d).

    K[(a_i*b+b_i)*d+d_i, (a_i*c+c_i)*d+d_i] = W[a_i,b_i,c_i,d_i]
    (interface.py:108-113: diag_embed over d, permute, block_diag over a).
    """
    w4 = np.asarray(w4)
    a, b, c, d = w4.shape
    k = np.zeros((a, b, d, a, c, d), dtype=w4.dtype)
    ai = np.arange(a)
    di = np.arange(d)
    # k[ai, :, di, ai, :, di] = w4[ai, :, :, di]
    for i in ai:
        for j in di:
            k[i, :, j, i, :, j] = w4[i, :, :, j]
    return k.reshape(a * b * d, a * c * d)


def pack_kernel_format(w4):
    """(a,b,c,d) -> (a*d*c, b): element (a_i,b_i,c_i,d_i) at row (a_i*d+d_i)*c+c_i, col b_i.

    interface.py:69 (``weights.permute(0, 3, 2, 1).reshape(a*d*c, b)``).
    """
    w4 = np.asarray(w4)
    a, b, c, d = w4.shape
    return np.ascontiguousarray(np.transpose(w4, (0, 3, 2, 1)).reshape(a * d * c, b))


def unpack_kernel_format(wk, pattern):
    """Inverse of :func:`pack_kernel_format` (interface.py:78)."""
    a, b, c, d = pattern
    wk = np.asarray(wk)
    assert wk.shape == (a * d * c, b)
    return np.ascontiguousarray(np.transpose(wk.reshape(a, d, c, b), (0, 3, 2, 1)))


def pack_bmm_format(w4):
    """(a,b,c,d) -> (a*d, b, c) (interface.py:35-36: ``permute(0,3,1,2).view(a*d,b,c)``)."""
    w4 = np.asarray(w4)
    a, b, c, d = w4.shape
    return np.ascontiguousarray(np.transpose(w4, (0, 3, 1, 2)).reshape(a * d, b, c))


# ----------------------------------------------------------------------------------------
# the three CPU algorithms of the reference, restated in numpy
# ----------------------------------------------------------------------------------------

def ks_apply_dense(w4, x, bs_last):
    """``F.linear(x, K)`` / ``K @ x`` (interface.py:252-253, 330-331)."""
    k = ks_dense(np.asarray(w4, dtype=np.float64))
    x = np.asarray(x, dtype=np.float64)
    return k @ x if bs_last else x @ k.T


def ks_apply_bmm(w4, x, bs_last):
    """The permute -> batched matmul -> permute scheme of forward_bmm.py:38-69."""
    w4 = np.asarray(w4, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    a, b, c, d = w4.shape
    wb = pack_bmm_format(w4)  # (a*d, b, c)
    if bs_last:
        n = x.shape[1]
        xs = np.transpose(x.reshape(a, c, d, n), (0, 2, 1, 3)).reshape(a * d, c, n)
        out = np.matmul(wb, xs)  # (a*d, b, n)
        return np.transpose(out.reshape(a, d, b, n), (0, 2, 1, 3)).reshape(a * b * d, n)
    n = x.shape[0]
    xs = np.transpose(x.reshape(n, a, c, d), (0, 1, 3, 2)).reshape(n, a * d, c)
    xs = np.transpose(xs, (1, 0, 2))  # (a*d, n, c)
    out = np.matmul(xs, np.transpose(wb, (0, 2, 1)))  # (a*d, n, b)
    out = np.transpose(out, (1, 0, 2)).reshape(n, a, d, b)
    return np.transpose(out, (0, 1, 3, 2)).reshape(n, a * b * d)


def ks_apply_einsum(w4, x, bs_last):
    """``"... a c d, a b c d -> ... a b d"`` (interface.py:254-264, 332-342)."""
    w4 = np.asarray(w4, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    a, b, c, d = w4.shape
    if bs_last:
        n = x.shape[1]
        return np.einsum("acdn,abcd->abdn", x.reshape(a, c, d, n), w4).reshape(a * b * d, n)
    n = x.shape[0]
    return np.einsum("nacd,abcd->nabd", x.reshape(n, a, c, d), w4).reshape(n, a * b * d)


def ks_apply_kernel_format(wk, pattern, x, bs_last):
    """Product taking the weight in kernel format (a*d*c, b), as ``Kernel.forward`` does."""
    return ks_apply_einsum(unpack_kernel_format(wk, pattern), x, bs_last)


# ----------------------------------------------------------------------------------------
# chain
# ----------------------------------------------------------------------------------------

def chain_apply(w4_list, x, bs_last, apply=ks_apply_einsum):
    """Apply factors in list order: ``patterns[0]`` is the right-most factor and acts first
    (interface.py:193-345, README.md:37)."""
    out = np.asarray(x, dtype=np.float64)
    for w4 in w4_list:
        out = apply(w4, out, bs_last)
    return out


def chain_dense(w4_list):
    """K_L ... K_1 with K_1 = ks_dense(w4_list[0]) (interface.py:434-436)."""
    dense = ks_dense(np.asarray(w4_list[0], dtype=np.float64))
    for w4 in w4_list[1:]:
        dense = ks_dense(np.asarray(w4, dtype=np.float64)) @ dense
    return dense


def ks_backward(w4, x, dy, bs_last):
    """Adjoints of y = K x for one factor, float64: (dX, dW4) with
    dX[a,c,d,n] = sum_b W[a,b,c,d] dY[a,b,d,n]  (= K^T dY, the dense form of interface.py:108-113
    transposed) and dW[a,b,c,d] = sum_n dY[a,b,d,n] X[a,c,d,n].  The reference has no backward
    pass of its own (kernel.py:319-329, forward_bmm.py:12-15)."""
    w4 = np.asarray(w4, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    a, b, c, d = w4.shape
    if not bs_last:
        x, dy = x.T, dy.T
    n = x.shape[1]
    x4, dy4 = x.reshape(a, c, d, n), dy.reshape(a, b, d, n)
    dx = np.einsum("abdn,abcd->acdn", dy4, w4).reshape(a * c * d, n)
    dw = np.einsum("abdn,acdn->abcd", dy4, x4)
    return (dx if bs_last else dx.T), dw


def rel_fro_error(y, z):
    """||y - z||_F / ||z||_F with z the oracle (scripts/example.py:22-23)."""
    y = np.asarray(y, dtype=np.float64)
    z = np.asarray(z, dtype=np.float64)
    return float(np.linalg.norm(y - z) / np.linalg.norm(z))


# ----------------------------------------------------------------------------------------
# fp8 e4m3fn (OCP) helpers.  The reference has no working fp8 path through PyTorch
# (kernel.cu:66-82 is a no-op); the contract here is: e4m3fn x and W, per-tensor fp32
# scales, fp32 accumulate, fp16 output.  The oracle works on the *dequantised* operands.
# ----------------------------------------------------------------------------------------

def e4m3fn_decode_table():
    """All 256 e4m3fn code points as float64 (NaN for 0x7f / 0xff).

    1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; max finite 448.
    """
    tab = np.empty(256, dtype=np.float64)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            tab[code] = np.nan
        elif e == 0:
            tab[code] = s * (m / 8.0) * 2.0 ** (-6)
        else:
            tab[code] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return tab


def e4m3fn_encode(v):
    """Round-to-nearest-even encode of finite values with |v| <= 448 into e4m3fn codes."""
    v = np.asarray(v, dtype=np.float64)
    tab = e4m3fn_decode_table()
    pos = tab[:0x7F]  # 0 .. 448, ascending
    mag = np.abs(v)
    assert np.all(mag <= 448.0 * (1 + 2.0 ** -4)), "value out of e4m3fn range"
    hi = np.searchsorted(pos, mag, side="left").clip(0, len(pos) - 1)
    lo = (hi - 1).clip(0, None)
    dlo = mag - pos[lo]
    dhi = pos[hi] - mag
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((hi & 1) == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(pos[hi] == mag, hi, code).astype(np.uint8)
    return np.where(np.signbit(v), code | 0x80, code).astype(np.uint8)


def fp8_quantize(t):
    """Per-tensor scale ``s = amax/448`` then e4m3fn encode of ``t/s``.

    The division is carried out in float32, as the device-side caller does with torch.
    Returns (codes uint8, scale float32).
    """
    t32 = np.asarray(t, dtype=np.float32)
    amax = float(np.max(np.abs(t32)))
    scale = np.float32(amax / 448.0) if amax > 0 else np.float32(1.0)
    q = e4m3fn_encode((t32 / scale).astype(np.float32))
    return q, scale


def fp8_dequantize(codes, scale):
    return e4m3fn_decode_table()[np.asarray(codes, dtype=np.uint8)] * float(scale)


# ----------------------------------------------------------------------------------------
# torch restatement of the reference's CPU ``bmm`` algorithm: this is the *timed CPU
# baseline* (forward_bmm.py:38-69: permute -> contiguous -> torch.bmm -> permute).
# ----------------------------------------------------------------------------------------

def torch_bmm_forward(w_bmm, x, pattern, bs_last):
    """``w_bmm``: torch tensor (a*d, b, c); ``x``: (a*c*d, n) or (n, a*c*d)."""
    import torch

    a, b, c, d = pattern
    if bs_last:
        n = x.shape[1]
        xs = x.reshape(a, c, d, n).transpose(1, 2).reshape(a * d, c, n).contiguous()
        out = torch.empty(a * d, b, n, dtype=x.dtype)
        torch.bmm(w_bmm, xs, out=out)
        return out.reshape(a, d, b, n).transpose(1, 2).reshape(a * b * d, n)
    n = x.shape[0]
    xs = x.reshape(n, a, c, d).transpose(-1, -2).reshape(n, a * d, c).contiguous().transpose(0, 1)
    out = torch.empty(n, a * d, b, dtype=x.dtype).transpose(0, 1)
    torch.bmm(xs, w_bmm.transpose(-1, -2), out=out)
    return out.transpose(0, 1).reshape(n, a, d, b).transpose(-1, -2).reshape(n, a * b * d)


def torch_bmm_chain(w_bmm_list, x, patterns, bs_last):
    out = x
    for w, p in zip(w_bmm_list, patterns):
        out = torch_bmm_forward(w, out, p, bs_last)
    return out


# ----------------------------------------------------------------------------------------
# closed forms used to pin the oracle
# ----------------------------------------------------------------------------------------

def hadamard_butterfly_weights(log2n):
    """Weights of the radix-2 butterfly chain whose product is the Sylvester-Hadamard
    matrix H_{2^L} (no permutation needed for this ordering).

    Factor l (l = 0 .. L-1, applied in list order) has pattern (2^(L-1-l), 2, 2, 2^l) and
    every 2x2 block equal to [[1, 1], [1, -1]]: its dense form is I (x) H_2 (x) I, and the
    product of the L commuting terms is H_2^{(x) L}.
    """
    h2 = np.array([[1.0, 1.0], [1.0, -1.0]])
    out = []
    for l in range(log2n):
        a, d = 2 ** (log2n - 1 - l), 2 ** l
        w4 = np.broadcast_to(h2[None, :, :, None], (a, 2, 2, d)).copy()
        out.append(w4)
    return out


def sylvester_hadamard(log2n):
    h = np.array([[1.0]])
    h2 = np.array([[1.0, 1.0], [1.0, -1.0]])
    for _ in range(log2n):
        h = np.kron(h2, h)
    return h
