"""Shared helpers for the parity tests (CPU side: oracle; GPU side: C ABI through ksmm_amd)."""
import math

import numpy as np
import torch

from oracle import ks_oracle as O

# Relative Frobenius error vs the oracle.  The contract asks for 1e-5 / 2e-3 / 5e-2; the e4m3 path
# multiplies exactly decoded operands with fp32 accumulation and rounds once to fp16, so its real
# error is that of fp16 storage (a few 1e-4) and the tests hold it to 5e-3: one wrong output row
# or column in a thousand would not pass.
TOL = {"fp32": 1e-5, "fp16": 2e-3, "fp8": 5e-3}
TORCH_DTYPE = {"fp32": torch.float32, "fp16": torch.float16, "fp8": torch.float8_e4m3fn}


def seeded_weights(patterns, seed=0, bound=None):
    """4-D weights U(-1/sqrt(c), 1/sqrt(c)) (or +-bound) per factor, float32, from a seed."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for (a, b, c, d) in patterns:
        s = bound if bound is not None else 1.0 / math.sqrt(c)
        out.append((torch.rand(a, b, c, d, generator=g) * 2 - 1) * s)
    return out


def seeded_input(in_size, batch, bs_last, seed=1):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, in_size, generator=g)
    return x.t().contiguous() if bs_last else x


def round_to(t, prec):
    """Value of ``t`` after the storage rounding of ``prec``, as float64 numpy; for fp8 also
    returns the codes and the per-tensor scale."""
    if prec == "fp32":
        return t.to(torch.float32).numpy().astype(np.float64), None, None
    if prec == "fp16":
        return t.to(torch.float16).to(torch.float32).numpy().astype(np.float64), None, None
    from ksmm_amd import quantize_fp8

    q, s = quantize_fp8(t)
    return q.to(torch.float32).numpy().astype(np.float64) * float(s), q, float(s)


def sample_columns(batch, step=97, edge=8):
    """Batch indices checked at full size: both edges plus a stride through the middle."""
    idx = set(range(min(edge, batch))) | set(range(max(0, batch - edge), batch))
    idx |= set(range(0, batch, step))
    return np.array(sorted(idx))


def oracle_chain(w4_list_rounded, x_rounded, bs_last, cols=None):
    """float64 oracle on (optionally a subset of) batch columns."""
    if cols is not None:
        x_rounded = x_rounded[:, cols] if bs_last else x_rounded[cols, :]
    return O.chain_apply(w4_list_rounded, x_rounded, bs_last, apply=O.ks_apply_einsum)
