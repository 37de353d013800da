"""Algorithmic work and MI355X roofline of one KS factor.

bytes = B*a*c*d*s_in + B*a*b*d*s_out + a*b*c*d*s_w      flops = 2*B*a*b*c*d
Peaks: HBM3E 8 TB/s; dense matrix fp32 157.3 TFLOP/s, fp16 2516.6, fp8 5033.2.
"""
import torch

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"fp32": 157.3, "fp16": 2516.6, "fp8": 5033.2}
ELEM = {torch.float32: 4, torch.float16: 2, torch.float8_e4m3fn: 1}


def factor_work(batch, pattern, x_dtype, w_dtype, y_dtype):
    a, b, c, d = pattern
    nbytes = batch * a * c * d * ELEM[x_dtype] + batch * a * b * d * ELEM[y_dtype] + a * b * c * d * ELEM[w_dtype]
    return nbytes, 2 * batch * a * b * c * d


def factor_roofline(batch, pattern, x_dtype, w_dtype, y_dtype, seconds):
    """Which roof bounds the factor and what fraction of it ``seconds`` per launch reaches.

    The matrix peak used is the one of the operand types: fp32 for fp32, fp8 when input and
    weights are both e4m3fn (the GEMM tiles feed the bytes to the fp8 MFMA; the small-block
    kernels decode to fp16 first, for which this peak is the stricter price), fp16 otherwise."""
    nbytes, flops = factor_work(batch, pattern, x_dtype, w_dtype, y_dtype)
    fp8 = torch.float8_e4m3fn
    prec = "fp32" if x_dtype == torch.float32 else "fp8" if (x_dtype == fp8 and w_dtype == fp8) else "fp16"
    t_hbm = nbytes / (HBM_PEAK_GBS * 1e9)
    t_mfma = flops / (MFMA_PEAK_TFLOPS[prec] * 1e12)
    gbs = nbytes / seconds / 1e9
    tfs = flops / seconds / 1e12
    if t_hbm >= t_mfma:
        roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": gbs / HBM_PEAK_GBS}
    else:
        roof = {"bound": "mfma", "achieved": tfs, "peak": MFMA_PEAK_TFLOPS[prec], "unit": "TFLOP/s",
                "frac": tfs / MFMA_PEAK_TFLOPS[prec]}
    roof.update({"bytes": nbytes, "flops": flops, "gbs": gbs, "tflops": tfs,
                 "floor_us": max(t_hbm, t_mfma) * 1e6})
    return roof
