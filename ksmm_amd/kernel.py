"""``Kernel.forward``: the per-factor entry point ``KSLinear(algo='kernel')`` calls.

Same positional signature as the reference's
``Kernel.forward(input, factor, bs_last, a, b, c, d, dtype, vsize)``
(src/ksmm_py/layer/kronecker_sparse/kernel.py:61-73).  Instead of rewriting ``.cuh`` files
and JIT-compiling per (pattern, batch), it calls the prebuilt C ABI (include/ksmm_hip.h)
with raw device pointers on the current PyTorch stream.
"""
import ctypes

import torch

from . import _lib

_DTYPES = {
    torch.float32: _lib.KSMM_F32,
    torch.float16: _lib.KSMM_F16,
    torch.float8_e4m3fn: _lib.KSMM_FP8_E4M3,
}


def dtype_code(dt):
    try:
        return _DTYPES[dt]
    except KeyError:
        # kernel.cu:123-125: assert(0 && "Unsupported data type")
        raise AssertionError("Unsupported data type %s" % (dt,))


def _check_input(t, name):
    # kernel.cpp:19-23
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def _stream_ptr(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


_ACTS = {None: _lib.ACT_NONE, "none": _lib.ACT_NONE, "gelu": _lib.ACT_GELU}


def _epilogue(bias, act, out_size, out_dtype, device):
    """ctypes epilogue (or None) for a bias vector of ``out_size`` values and an activation name."""
    if act not in _ACTS:
        raise ValueError("act must be one of %s" % sorted(k for k in _ACTS if k))
    if bias is None and _ACTS[act] == _lib.ACT_NONE:
        return None, None
    ep = _lib.KsmmEpilogue()
    ep.act = _ACTS[act]
    keep = None
    if bias is not None:
        keep = bias.detach().reshape(-1)
        assert keep.numel() == out_size, "bias must hold one value per output feature"
        if keep.dtype != out_dtype or keep.device != device or not keep.is_contiguous():
            keep = keep.to(device=device, dtype=out_dtype).contiguous()
        ep.bias = keep.data_ptr()
    else:
        ep.bias = None
    return ep, keep


class Kernel:
    """Namespace with the reference's static-method calling convention (forward only)."""

    @staticmethod
    def forward(input, factor, bs_last, a, b, c, d, dtype=None, vsize=4, scale=1.0,
                algo=_lib.ALGO_AUTO, variant=-1, out=None, workspace=None, bias=None, act=None):
        """y = K x for one factor.

        ``input``: (a*c*d, batch) if ``bs_last`` else (batch, a*c*d); ``factor``: kernel
        format (a*d*c, b).  ``dtype`` is accepted for signature compatibility: the element
        types are taken from the tensors.  ``vsize`` is accepted and ignored (vector widths
        are part of the tile table).  fp8 inputs/weights produce an fp16 result scaled by
        ``scale``.  Batch-size-first factors with d > 1 that have no kernel of their own run
        in batch-size-last layout between two transposes; the scratch tensor for that is
        allocated here unless ``workspace`` (uint8, large enough) is passed.  ``bias`` (one
        value per output feature) and ``act`` ("gelu") are applied to the fp32 accumulator
        inside the kernel: y = act(scale * acc + bias).
        """
        lib = _lib.load()
        _check_input(input, "input")
        _check_input(factor, "factor")
        bs_last = bool(bs_last)
        in_size = a * c * d
        out_size = a * b * d
        # kernel.cpp:38-42
        assert input.dim() == 2 and factor.dim() == 2
        assert in_size == input.size(0 if bs_last else 1)
        assert factor.size(0) == input.size(0 if bs_last else 1)
        assert b == factor.size(1)
        batch = input.size(1 if bs_last else 0)
        xd, wd = dtype_code(input.dtype), dtype_code(factor.dtype)
        out_dtype = torch.float16 if wd == _lib.KSMM_FP8_E4M3 else input.dtype
        shape = (out_size, batch) if bs_last else (batch, out_size)
        if out is None:
            out = torch.empty(shape, dtype=out_dtype, device=input.device)
        else:
            assert out.shape == shape and out.dtype == out_dtype and out.is_contiguous()
        yd = dtype_code(out_dtype)
        ep, _keep = _epilogue(bias, act, out_size, out_dtype, input.device)
        if ep is not None and not (algo == _lib.ALGO_AUTO and variant == -1):
            raise ValueError("bias/act go with the automatic kernel choice")
        with torch.cuda.device(input.device):
            if algo == _lib.ALGO_AUTO and variant == -1:
                need = lib.ksmm_factor_workspace(batch, a, b, c, d, xd, wd, yd, int(bs_last))
                if need < 0:
                    _lib.check(int(need))
                if need > 0 and (workspace is None or workspace.numel() * workspace.element_size() < need):
                    workspace = torch.empty(need, dtype=torch.uint8, device=input.device)
                rc = lib.ksmm_factor_forward_ep(
                    input.data_ptr(), factor.data_ptr(), out.data_ptr(), batch, a, b, c, d, xd, wd, yd,
                    int(bs_last), float(scale), ctypes.byref(ep) if ep is not None else None,
                    workspace.data_ptr() if need > 0 else None,
                    workspace.numel() * workspace.element_size() if need > 0 else 0, _stream_ptr(input))
            else:
                rc = lib.ksmm_factor_forward_algo(
                    input.data_ptr(), factor.data_ptr(), out.data_ptr(), batch, a, b, c, d, xd, wd, yd,
                    int(bs_last), float(scale), int(algo), int(variant), _stream_ptr(input))
        _lib.check(rc)
        return out

    @staticmethod
    def backward(grad_output, input, factor, bs_last, a, b, c, d, scale=1.0, need_input=True, need_weight=True,
                 workspace=None):
        """(grad_input, grad_factor) of ``forward(input, factor, bs_last, a, b, c, d, scale=scale)``
        for fp32 / fp16 tensors: grad_input = scale * K^T grad_output on the forward kernels (the
        factor with pattern (a, c, b, d) and transposed blocks), grad_factor in kernel format
        (a*d*c, b) from a reduction over the batch.  The reference's ``Kernel.backward``
        (kernel.py:319-329) refers to an undefined symbol; this is the adjoint of its forward."""
        lib = _lib.load()
        for t, name in ((grad_output, "grad_output"), (input, "input"), (factor, "factor")):
            _check_input(t, name)
        bs_last = bool(bs_last)
        assert input.dtype == factor.dtype == grad_output.dtype and input.dtype in (torch.float32, torch.float16)
        batch = input.size(1 if bs_last else 0)
        assert input.size(0 if bs_last else 1) == a * c * d and grad_output.size(0 if bs_last else 1) == a * b * d
        assert grad_output.size(1 if bs_last else 0) == batch and tuple(factor.shape) == (a * c * d, b)
        dt = dtype_code(input.dtype)
        need = lib.ksmm_factor_backward_workspace(batch, a, b, c, d, dt, int(bs_last))
        if need < 0:
            _lib.check(int(need))
        if workspace is None or workspace.numel() * workspace.element_size() < need:
            workspace = torch.empty(need, dtype=torch.uint8, device=input.device)
        ws_bytes = workspace.numel() * workspace.element_size()
        grad_input = grad_factor = None
        with torch.cuda.device(input.device):
            if need_input:
                grad_input = torch.empty_like(input)
                _lib.check(lib.ksmm_factor_backward_input(
                    grad_output.data_ptr(), factor.data_ptr(), grad_input.data_ptr(), batch, a, b, c, d, dt,
                    int(bs_last), float(scale), workspace.data_ptr(), ws_bytes, _stream_ptr(input)))
            if need_weight:
                grad_factor = torch.empty_like(factor)
                _lib.check(lib.ksmm_factor_backward_weight(
                    grad_output.data_ptr(), input.data_ptr(), grad_factor.data_ptr(), batch, a, b, c, d, dt,
                    int(bs_last), float(scale), workspace.data_ptr(), ws_bytes, _stream_ptr(input)))
        return grad_input, grad_factor

    @staticmethod
    def chain_forward(input, factors, patterns, bs_last, scales=None, fuse=True, workspace=None,
                      bias=None, act=None, static_scratch=False, out=None):
        """All factors of a KSLinear in one call (factor-chain launcher).  ``bias``/``act`` are
        applied by the last factor's kernel.  ``static_scratch=True`` uses the library's fixed
        32 MiB scratch array instead of a workspace tensor (no device allocation besides the
        output, which ``out`` can supply)."""
        lib = _lib.load()
        _check_input(input, "input")
        n = len(factors)
        assert n == len(patterns) and 1 <= n <= _lib.MAX_FACTORS
        bs_last = bool(bs_last)
        descs = (_lib.KsmmFactorDesc * n)()
        any_fp8 = False
        for i, (f, p) in enumerate(zip(factors, patterns)):
            _check_input(f, "factor")
            a, b, c, d = p
            assert f.dim() == 2 and f.size(0) == a * c * d and f.size(1) == b
            descs[i].w = f.data_ptr()
            descs[i].a, descs[i].b, descs[i].c, descs[i].d = a, b, c, d
            descs[i].w_dtype = dtype_code(f.dtype)
            descs[i].scale = 1.0 if scales is None else float(scales[i])
            any_fp8 |= f.dtype == torch.float8_e4m3fn
        a0, _, c0, d0 = patterns[0]
        al, bl, _, dl = patterns[-1]
        assert input.dim() == 2 and input.size(0 if bs_last else 1) == a0 * c0 * d0
        batch = input.size(1 if bs_last else 0)
        out_dtype = torch.float16 if any_fp8 else input.dtype
        out_size = al * bl * dl
        shape = (out_size, batch) if bs_last else (batch, out_size)
        if out is None:
            out = torch.empty(shape, dtype=out_dtype, device=input.device)
        else:
            assert out.shape == shape and out.dtype == out_dtype and out.is_contiguous()
        ep, _keep = _epilogue(bias, act, out_size, out_dtype, input.device)
        ep_ref = ctypes.byref(ep) if ep is not None else None
        if static_scratch:
            with torch.cuda.device(input.device):
                rc = lib.ksmm_chain_forward_static(descs, n, input.data_ptr(), out.data_ptr(), batch,
                                                   dtype_code(input.dtype), dtype_code(out_dtype), int(bs_last),
                                                   int(bool(fuse)), ep_ref, _stream_ptr(input))
            _lib.check(rc)
            return out
        need = lib.ksmm_chain_workspace_layout(descs, n, batch, dtype_code(input.dtype),
                                               dtype_code(out_dtype), int(bs_last))
        if need < 0:
            _lib.check(int(need))
        if need > 0 and (workspace is None or workspace.numel() * workspace.element_size() < need):
            workspace = torch.empty(need, dtype=torch.uint8, device=input.device)
        ws_ptr = workspace.data_ptr() if need > 0 else None
        ws_bytes = workspace.numel() * workspace.element_size() if need > 0 else 0
        with torch.cuda.device(input.device):
            rc = lib.ksmm_chain_forward_ep(descs, n, input.data_ptr(), out.data_ptr(), ws_ptr, ws_bytes,
                                           batch, dtype_code(input.dtype), dtype_code(out_dtype),
                                           int(bs_last), int(bool(fuse)), ep_ref, _stream_ptr(input))
        _lib.check(rc)
        return out


class KSFactorFunction(torch.autograd.Function):
    """One factor with a backward pass, for training through ``KSLinear(algo='kernel')``."""

    @staticmethod
    def forward(ctx, input, factor, bs_last, pattern):
        ctx.save_for_backward(input, factor)
        ctx.bs_last, ctx.pattern = bs_last, pattern
        return Kernel.forward(input, factor, bs_last, *pattern)

    @staticmethod
    def backward(ctx, grad_output):
        input, factor = ctx.saved_tensors
        gi, gf = Kernel.backward(grad_output.contiguous(), input, factor, ctx.bs_last, *ctx.pattern,
                                 need_input=ctx.needs_input_grad[0], need_weight=ctx.needs_input_grad[1])
        return gi, gf, None, None


def query_tile(batch, pattern, x_dtype, w_dtype=None, bs_last=True, algo=_lib.ALGO_AUTO, variant=-1):
    """What the tile table picks for one factor (host only; no GPU needed).  With the automatic
    choice, variant -1 consults the measured table first and -3 only the heuristics."""
    lib = _lib.load()
    w_dtype = x_dtype if w_dtype is None else w_dtype
    y_dtype = torch.float16 if w_dtype == torch.float8_e4m3fn else x_dtype
    t = _lib.KsmmTile()
    a, b, c, d = pattern
    _lib.check(lib.ksmm_query_tile_variant(batch, a, b, c, d, dtype_code(x_dtype), dtype_code(w_dtype),
                                           dtype_code(y_dtype), int(bool(bs_last)), int(algo), int(variant),
                                           ctypes.byref(t)))
    return t.as_dict()


def tuned_table(full=False):
    """Rows (a, b, c, d, combo, bs_last, algo, variant) of the measured table compiled into the
    library (combo 0 = fp32, 1 = fp16, 2 = e4m3 -> fp16); ``variant`` is what the row's stable
    instance id resolves to in this build.  ``full=True`` returns the id and the parameter too:
    (a, b, c, d, combo, bs_last, algo, id, param, variant)."""
    lib = _lib.load()
    rows = []
    buf = (ctypes.c_int * 10)()
    for i in range(lib.ksmm_tuned_count()):
        _lib.check(lib.ksmm_tuned_row(i, ctypes.byref(buf)))
        r = tuple(buf)
        rows.append(r if full else r[:7] + (r[9],))
    return rows


_COMBO_DTYPES = {0: (_lib.KSMM_F32,) * 3, 1: (_lib.KSMM_F16,) * 3,
                 2: (_lib.KSMM_FP8_E4M3, _lib.KSMM_FP8_E4M3, _lib.KSMM_F16),
                 3: (_lib.KSMM_F16, _lib.KSMM_FP8_E4M3, _lib.KSMM_F16)}


def variant_id(algo, variant, combo, bs_last):
    """(instance id, parameter) of a forced (family, variant) for an element-type combination."""
    lib = _lib.load()
    iid, par = ctypes.c_uint32(), ctypes.c_int()
    xd, wd, yd = _COMBO_DTYPES[combo]
    _lib.check(lib.ksmm_variant_id(int(algo), int(variant), xd, wd, yd, int(bool(bs_last)), ctypes.byref(iid),
                                   ctypes.byref(par)))
    return iid.value, par.value


def variant_from_id(algo, iid, param, combo, bs_last):
    lib = _lib.load()
    v = ctypes.c_int()
    xd, wd, yd = _COMBO_DTYPES[combo]
    _lib.check(lib.ksmm_variant_from_id(int(algo), int(iid), int(param), xd, wd, yd, int(bool(bs_last)),
                                        ctypes.byref(v)))
    return v.value
