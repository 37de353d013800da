"""``KSLinear``: Kronecker-sparse linear layer with the reference's constructor and attributes
(src/ksmm_py/layer/kronecker_sparse/interface.py:116-191), whose ``algo='kernel'`` runs the
hand-written gfx950 kernels of libksmm_hip.so.

Scope: the ``kernel`` path and the three dense-equivalent PyTorch paths it is compared with
(``dense``, ``bmm``, ``einsum``).  The ``sparse``/``bsr`` back-ends of the reference are torch
sparse formats unrelated to the kernel and are not provided.

A factor with pattern (a, b, c, d) has support I_a (x) 1_{b x c} (x) I_d; its weights are a
4-D tensor (a, b, c, d).  ``patterns[0]`` is the right-most factor: it is applied first.
"""
import math

import torch
import torch.nn.functional as F
from torch import nn

ALGOS = ("dense", "einsum", "kernel", "bmm")
FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


def quantize_fp8(t):
    """Per-tensor symmetric quantisation to e4m3fn: returns (codes, scale) with
    ``t ~= codes.float() * scale`` and ``scale = amax / 448``."""
    t32 = t.detach().to(torch.float32)
    amax = t32.abs().max()
    scale = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
    return (t32 / scale).to(FP8), scale


def from_abcd_to_dense(w4):
    """(a,b,c,d) -> dense (a*b*d, a*c*d): K[(i*b+j)*d+l, (i*c+k)*d+l] = w4[i,j,k,l]
    (interface.py:108-113)."""
    a, b, c, d = w4.shape
    eye = torch.eye(d, dtype=w4.dtype, device=w4.device)
    blocks = w4.unsqueeze(-1) * eye  # (a, b, c, d, d'): zero unless d == d'
    blocks = blocks.permute(0, 1, 3, 2, 4).reshape(a, b * d, c * d)
    return torch.block_diag(*blocks.unbind(0))


def from_kernel_format_to_abcd(factor, pattern):
    """(a*d*c, b) -> (a,b,c,d) (inverse of interface.py:69)."""
    a, b, c, d = pattern
    return factor.reshape(a, d, c, b).permute(0, 3, 2, 1)


def from_kernel_format_to_dense(factor, pattern):
    """interface.py:75-86."""
    return from_abcd_to_dense(from_kernel_format_to_abcd(factor, pattern).contiguous())


def from_bmm_format_to_dense(factor, pattern):
    """(a*d, b, c) or (a, d, b, c) -> dense (interface.py:89-105)."""
    a, b, c, d = pattern
    return from_abcd_to_dense(factor.reshape(a, d, b, c).permute(0, 2, 3, 1).contiguous())


def generate_factor(a, b, c, d, algo, weights=None, dtype=torch.float16, device="cpu"):
    """Storage of one factor in the layout ``algo`` consumes (interface.py:16-72).

    kernel: (a*d*c, b)   bmm: (a*d, b, c)   einsum: (a, b, c, d)   dense: (a*b*d, a*c*d).
    Random initialisation is U(-1/sqrt(c), 1/sqrt(c)) on the 4-D weights for every algo
    (the reference's ``dense`` branch draws a fully dense matrix when ``weights`` is None,
    interface.py:62; that is not reproduced).
    """
    assert algo in ALGOS, "algo must be one of %s" % (ALGOS,)
    if weights is None:
        s = 1.0 / math.sqrt(c)
        weights = torch.empty(a, b, c, d).uniform_(-s, s)
    assert tuple(weights.shape) == (a, b, c, d)
    if algo == "kernel":
        f = weights.permute(0, 3, 2, 1).reshape(a * d * c, b)
    elif algo == "bmm":
        f = weights.permute(0, 3, 1, 2).reshape(a * d, b, c)
    elif algo == "einsum":
        f = weights
    else:
        f = from_abcd_to_dense(weights)
    return f.to(dtype).to(device).contiguous()


def bmm_bs_first(x, w_kron, pattern):
    """forward_bmm.py:38-52."""
    a, b, c, d = pattern
    lead = x.shape[:-1]
    n = x.numel() // (a * c * d)
    xs = x.reshape(n, a, c, d).transpose(-1, -2).reshape(n, a * d, c).contiguous().transpose(0, 1)
    out = torch.bmm(xs, w_kron.transpose(-1, -2))  # (a*d, n, b)
    return out.transpose(0, 1).reshape(n, a, d, b).transpose(-1, -2).reshape(*lead, a * b * d)


def bmm_bs_last(x, w_kron, pattern):
    """forward_bmm.py:55-69."""
    a, b, c, d = pattern
    lead = x.shape[1:]
    n = x.numel() // (a * c * d)
    xs = x.reshape(a, c, d, n).transpose(1, 2).reshape(a * d, c, n).contiguous()
    out = torch.bmm(w_kron, xs)  # (a*d, b, n)
    return out.reshape(a, d, b, n).transpose(1, 2).reshape(a * b * d, *lead)


class KSLinear(nn.Module):
    """Drop-in for the reference's ``KSLinear`` on the ``kernel``/``dense``/``bmm``/``einsum``
    algorithms.

    ``algo='kernel'`` has two modes.  Without gradients (``torch.no_grad()``, which is how the
    reference runs it, utils.py:6-8, or when neither the input nor a factor requires a gradient)
    the whole layer is one call of the chain launcher: intermediates in a workspace or in LDS,
    bias and activation inside the last factor's kernel.  With gradients enabled and trainable
    factors (the state of a freshly built layer, ``eval()`` included) it runs factor by factor
    through an autograd function that keeps the intermediates for the backward pass, and bias
    and activation are PyTorch operations; both modes compute the same function.

    Beyond the reference's signature: ``fuse`` lets the chain launcher keep intermediates in
    LDS where it has a kernel for the chain, and ``act='gelu'`` applies GELU (erf form) after
    the bias, as the feed-forward block of the reference's ViT does between its two
    projections (src/ksmm_py/model/vit.py:416-431).  With ``algo='kernel'`` the bias and the
    activation are applied to the fp32 accumulator inside the last factor's kernel instead of
    in a pass of their own (interface.py:457-466).

    ``dtype=torch.float8_e4m3fn`` (kernel only on the device): weights are quantised per
    tensor to e4m3fn with an fp32 scale, the input is quantised on entry unless it already
    is e4m3fn (then pass ``x_scale``), accumulation is fp32 and the result is fp16.  With
    the PyTorch algorithms the same dtype stores the *dequantised* weights in fp32, which is
    what the kernel result is compared with.
    """

    def __init__(self, patterns, weights=None, bias=True, algo="dense", dtype=torch.float16,
                 bs_last=False, vsize=4, device="cpu", fuse=True, act=None):
        super().__init__()
        assert act in (None, "gelu"), "act must be None or 'gelu'"
        self.act = act
        assert algo in ("sparse", "bsr") + ALGOS
        if algo in ("sparse", "bsr"):
            raise NotImplementedError("algo=%r is outside the kernel path provided here" % algo)
        for pattern in patterns:
            assert len(pattern) == 4
        self.in_size = patterns[0][0] * patterns[0][2] * patterns[0][3]
        self.out_size = patterns[-1][0] * patterns[-1][1] * patterns[-1][3]
        self.algo = algo
        self.num_mat = len(patterns)
        self.patterns = [tuple(int(v) for v in p) for p in patterns]
        self.dtype = dtype
        self.bs_last = bs_last
        self.vsize = vsize
        self.weights = weights
        self.device = device
        self.fuse = fuse
        if str(device) == "cpu" and algo == "kernel":
            raise Exception("kernel expects device='cuda'.")
        if self.weights is None:
            self.weights = [None] * len(self.patterns)
        assert len(self.weights) == len(self.patterns)

        self.out_dtype = torch.float16 if dtype == FP8 else dtype
        params, scales = [], []
        for p, w in zip(self.patterns, self.weights):
            if dtype == FP8:
                w4 = generate_factor(*p, "einsum", w, torch.float32, "cpu")
                q4, s = quantize_fp8(w4)
                if algo == "kernel":
                    f = generate_factor(*p, "kernel", q4.to(torch.float32), FP8, device)
                else:
                    f = generate_factor(*p, algo, q4.to(torch.float32) * s, torch.float32, device)
                scales.append(float(s))
            else:
                f = generate_factor(*p, algo, w, dtype, device)
                scales.append(1.0)
            params.append(nn.Parameter(f, requires_grad=f.dtype != FP8))
        self.factors = nn.ParameterList(params)
        self.w_scales = scales

        if bias:
            bound = 1 / math.sqrt(self.in_size)
            shape = (self.out_size, 1) if bs_last else (self.out_size,)
            self.bias = nn.Parameter(
                torch.empty(*shape, device=device).uniform_(-bound, bound).to(self.out_dtype))
        else:
            self.register_parameter("bias", None)

    # -- chain -------------------------------------------------------------------------------
    def _kernel_chain(self, x, x_scale):
        from .kernel import Kernel

        if torch.is_grad_enabled() and self.dtype != FP8 and (
                x.requires_grad or any(f.requires_grad for f in self.factors)):
            # training: factor by factor through the autograd function (intermediates are kept for
            # the weight gradients); bias and activation stay PyTorch ops so that autograd sees them
            from .kernel import KSFactorFunction

            out = x
            for f, p in zip(self.factors, self.patterns):
                out = KSFactorFunction.apply(out, f, self.bs_last, p)
            if self.bias is not None:
                out = out + self.bias
            return F.gelu(out) if self.act == "gelu" else out
        scales = list(self.w_scales)
        if self.dtype == FP8:
            if x.dtype != FP8:
                x, s = quantize_fp8(x)
                x_scale = float(s)
            scales[0] *= 1.0 if x_scale is None else float(x_scale)
        if self.fuse or self.num_mat > 1:
            return Kernel.chain_forward(x, list(self.factors), self.patterns, self.bs_last,
                                        scales=scales, fuse=self.fuse, bias=self.bias, act=self.act)
        a, b, c, d = self.patterns[0]
        return Kernel.forward(x, self.factors[0], self.bs_last, a, b, c, d, dtype=self.dtype,
                              vsize=self.vsize, scale=scales[0], bias=self.bias, act=self.act)

    def forward_bs_first(self, output, x_scale=None):
        if self.algo == "kernel":
            return self._kernel_chain(output, x_scale)
        for factor, (a, b, c, d) in zip(self.factors, self.patterns):
            if self.algo == "bmm":
                output = bmm_bs_first(output, factor, (a, b, c, d))
            elif self.algo == "dense":
                output = F.linear(output, factor)
            else:
                lead = output.shape[:-1]
                output = torch.einsum("nacd,abcd->nabd", output.reshape(-1, a, c, d), factor)
                output = output.reshape(*lead, a * b * d)
        return output

    def forward_bs_last(self, output, x_scale=None):
        if self.algo == "kernel":
            return self._kernel_chain(output, x_scale)
        for factor, (a, b, c, d) in zip(self.factors, self.patterns):
            if self.algo == "bmm":
                output = bmm_bs_last(output, factor, (a, b, c, d))
            elif self.algo == "dense":
                output = torch.matmul(factor, output)
            else:
                lead = output.shape[1:]
                output = torch.einsum("acdn,abcd->abdn", output.reshape(a, c, d, -1), factor)
                output = output.reshape(a * b * d, *lead)
        return output

    def forward(self, tensor, x_scale=None):
        output = self.pre_process(tensor)
        if self.dtype == FP8 and self.algo != "kernel":
            # PyTorch algorithms work on the dequantised input in fp32
            if output.dtype == FP8:
                output = output.to(torch.float32) * (1.0 if x_scale is None else float(x_scale))
            else:
                q, s = quantize_fp8(output)
                output = q.to(torch.float32) * s
        if self.bs_last:
            output = self.forward_bs_last(output, x_scale)
        else:
            output = self.forward_bs_first(output, x_scale)
        return self.post_process(tensor, output)

    # -- helpers -----------------------------------------------------------------------------
    def get_dense_product(self, dtype=None):
        """Dense matrix of the whole layer, K_L ... K_1 (interface.py:363-437), multiplied in the
        factors' own type like the reference does, or in ``dtype`` when one is given (e4m3
        factors are dequantised to fp32 first either way)."""
        mats = []
        for factor, pattern, s in zip(self.factors, self.patterns, self.w_scales):
            f = factor.detach()
            if f.dtype == FP8:
                f = f.to(torch.float32) * s
            if dtype is not None:
                f = f.to(dtype)
            if self.algo == "bmm":
                mats.append(from_bmm_format_to_dense(f, pattern))
            elif self.algo == "kernel":
                mats.append(from_kernel_format_to_dense(f, pattern))
            elif self.algo == "einsum":
                mats.append(from_abcd_to_dense(f))
            else:
                mats.append(f)
        dense = mats[0]
        for m in mats[1:]:
            dense = torch.matmul(m, dense)
        return dense

    def pre_process(self, tensor):
        """interface.py:439-449: fold every non-feature axis into the batch."""
        if self.bs_last:
            return tensor.view(tensor.size(0), -1)
        return tensor.view(-1, tensor.size(-1))

    def post_process(self, tensor, output):
        """interface.py:451-467: bias, then restore the caller's batch axes.  The kernel path
        has added the bias (and applied the activation) in its last factor already."""
        if self.algo != "kernel":
            if self.bias is not None:
                output = output + self.bias
            if self.act == "gelu":
                output = F.gelu(output)
        if self.bs_last:
            return output.view(self.out_size, *tensor.shape[1:])
        return output.view(*tensor.shape[:-1], self.out_size)

    def extra_repr(self):
        return "in_size={}, out_size={}, num_mat={}, patterns={}, algo={}, bias={}".format(
            self.in_size, self.out_size, self.num_mat, self.patterns, self.algo,
            self.bias is not None)
