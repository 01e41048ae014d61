"""Operator front end on torch tensors, over the C ABI.

Mirrors the call surface of the reference's Python layer: ``gemm``,
``conv2d`` and ``attention`` of ``PyContext`` (src/interface/python.rs:124-462)
and ``tracea.ops.conv2d`` (tracea-python/python/tracea/ops.py:39-70), including
its epilogue string grammar ("bias+relu", src/interface/python.rs:41-87).
torch supplies device memory and the current stream; all arithmetic happens in
``libtracea.so``.
"""
import ctypes as C

import torch

from . import capi

_DTYPES = {torch.float32: capi.F32, torch.float16: capi.F16, torch.bfloat16: capi.BF16,
           torch.int32: capi.I32, torch.int8: capi.I8}


_VIEW_CACHE = {}


def _view(t, shape=None, stride=None):
    """TraceaTensorView of a tensor.  Building the ctypes structure costs 2-3 us, four or five
    times per call, more than the library's own dispatch: views are kept by (address, extents,
    strides, type, device), which a loop over the same tensors hits every time.  A view holds no
    reference to the tensor, so a stale entry is only a few hundred bytes."""
    if shape is None:
        shape = t.shape
    if stride is None:
        stride = t.stride()
    key = (t.data_ptr(), shape, stride, t.dtype, t.get_device())
    v = _VIEW_CACHE.get(key)
    if v is None:
        dtype = _DTYPES.get(t.dtype)
        if dtype is None:
            raise TypeError("unsupported dtype %s" % t.dtype)
        if len(_VIEW_CACHE) >= 1024:
            _VIEW_CACHE.clear()
        # get_device(): the device index of a GPU tensor, -1 for a host tensor (which the library rejects)
        v = _VIEW_CACHE[key] = capi.View(key[0], shape, stride, dtype, key[4])
    return v


def _stream(t):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream) if t.is_cuda else None


_EPILOGUE_STRINGS = {
    "": capi.EPI_IDENTITY, "none": capi.EPI_IDENTITY, "identity": capi.EPI_IDENTITY,
    "bias": capi.EPI_BIAS_ADD, "relu": capi.EPI_RELU, "gelu": capi.EPI_GELU, "silu": capi.EPI_SILU,
    "bias+relu": capi.EPI_BIAS_RELU, "bias+silu": capi.EPI_BIAS_SILU,
    "residual": capi.EPI_RESIDUAL, "residual+relu": capi.EPI_RESIDUAL_RELU,
}


def parse_epilogue(spec):
    """"bias+relu" style string or a TraceaEpilogueKind integer -> kind."""
    if isinstance(spec, int):
        return spec
    key = (spec or "").strip().lower().replace(" ", "")
    if key not in _EPILOGUE_STRINGS:
        raise ValueError("unknown epilogue %r" % spec)
    return _EPILOGUE_STRINGS[key]


def gemm(a, b, out=None, bias=None, residual=None, epilogue="none", out_dtype=None):
    """out[M,N] = epilogue(a[M,K] @ b[K,N]).  b may be any strided 2-D view; a
    column-major B is ``storage_nk.t()``."""
    m, k = a.shape
    k2, n = b.shape
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype or a.dtype, device=a.device)
    va, vb, vc = _view(a), _view(b), _view(out)
    vbias = _view(bias) if bias is not None else None
    vres = _view(residual) if residual is not None else None
    params = capi.GemmParams(parse_epilogue(epilogue), _stream(a))
    st = capi.lib().tracea_gemm(va.c, vb.c, C.byref(vbias.c) if vbias else None,
                                C.byref(vres.c) if vres else None, C.byref(vc.c), params)
    capi.check("tracea_gemm", st)
    return out


def gemm_noalloc(a, b, out, bias=None, residual=None, epilogue="none"):
    """tracea_gemm_noalloc: as :func:`gemm` with the split-K workspace taken from the library's
    static device array.  ``out`` is required (this wrapper allocates no device memory either);
    calls that may overlap on one GPU share the workspace and must be ordered by the caller."""
    va, vb, vc = _view(a), _view(b), _view(out)
    vbias = _view(bias) if bias is not None else None
    vres = _view(residual) if residual is not None else None
    params = capi.GemmParams(parse_epilogue(epilogue), _stream(a))
    st = capi.lib().tracea_gemm_noalloc(va.c, vb.c, C.byref(vbias.c) if vbias else None,
                                        C.byref(vres.c) if vres else None, C.byref(vc.c), params)
    capi.check("tracea_gemm_noalloc", st)
    return out


def low_rank_mlp(x, a, b, out=None, bias=None, residual=None, epilogue="none", out_dtype=None):
    """out[M,N] = epilogue((x[M,K] @ a[K,R]) @ b[R,N]); the rank-R product is rounded to the
    operands' type in between (the reference's LowRankMlp operator)."""
    m, _ = x.shape
    _, n = b.shape
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype or x.dtype, device=x.device)
    vx, va, vb, vc = _view(x), _view(a), _view(b), _view(out)
    vbias = _view(bias) if bias is not None else None
    vres = _view(residual) if residual is not None else None
    params = capi.GemmParams(parse_epilogue(epilogue), _stream(x))
    st = capi.lib().tracea_low_rank_mlp(vx.c, va.c, vb.c, C.byref(vbias.c) if vbias else None,
                                        C.byref(vres.c) if vres else None, C.byref(vc.c), params)
    capi.check("tracea_low_rank_mlp", st)
    return out


def apply_epilogue(x, ops, out=None, out_dtype=None):
    """out = chain(x) in one pass over a channels-last tensor, e.g. standalone BatchNorm
    [(OP_BATCHNORM, gamma, beta, mean, var, eps)], ReLU [(OP_RELU,)], Add [(OP_RESIDUAL_ADD, other)]."""
    if out is None:
        out = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    arr, _keep = _ops_array(ops)
    vx, vo = _view(x), _view(out)
    st = capi.lib().tracea_apply_epilogue(vx.c, C.byref(vo.c), arr, len(ops), _stream(x))
    capi.check("tracea_apply_epilogue", st)
    return out


def batchnorm(x, gamma, beta, mean, var, eps=1e-5, out=None):
    """Inference BatchNorm over the last (channel) axis."""
    return apply_epilogue(x, [(capi.OP_BATCHNORM, gamma, beta, mean, var, eps)], out=out)


def softmax(x, out=None, out_dtype=None):
    """Softmax over the last axis."""
    if out is None:
        out = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    vx, vo = _view(x), _view(out)
    capi.check("tracea_softmax", capi.lib().tracea_softmax(vx.c, C.byref(vo.c), _stream(x)))
    return out


def global_avg_pool(x, out=None, out_dtype=None):
    """x [N,H,W,C] -> [N,C]."""
    if out is None:
        out = torch.empty((x.shape[0], x.shape[3]), dtype=out_dtype or x.dtype, device=x.device)
    vx, vo = _view(x), _view(out)
    capi.check("tracea_global_avg_pool", capi.lib().tracea_global_avg_pool(vx.c, C.byref(vo.c), _stream(x)))
    return out


def linear(a, w, bias=None, epilogue=None, out=None, out_dtype=None):
    """c[b] = epilogue(a[b] @ w[b]); a [B,M,K], w [B,K,N] or [K,N]."""
    if out is None:
        out = torch.empty((a.shape[0], a.shape[1], w.shape[-1]), dtype=out_dtype or a.dtype, device=a.device)
    if epilogue is None:
        epilogue = "bias" if bias is not None else "none"
    va, vw, vc = _view(a), _view(w), _view(out)
    vbias = _view(bias) if bias is not None else None
    params = capi.GemmParams(parse_epilogue(epilogue), _stream(a))
    st = capi.lib().tracea_linear(va.c, vw.c, C.byref(vbias.c) if vbias else None, C.byref(vc.c), params)
    capi.check("tracea_linear", st)
    return out


def _ops_array(ops):
    """[(kind, tensors..., [eps])] -> (EpilogueOp array, keep-alive list)."""
    arr = (capi.EpilogueOp * max(1, len(ops)))()
    keep = []
    for i, op in enumerate(ops):
        kind = op[0]
        tensors = [t for t in op[1:] if isinstance(t, torch.Tensor)]
        scalars = [t for t in op[1:] if not isinstance(t, torch.Tensor)]
        if kind in (capi.OP_BATCHNORM, capi.OP_SCALE_SHIFT):
            # the kernels read these per-channel vectors as fp32 (the library refuses anything else);
            # all of them are checked here, the library only sees the first one's type
            for t in tensors:
                if t.dtype != torch.float32:
                    raise ValueError("BatchNorm / scale-shift parameters must be float32 tensors, got %s "
                                     "(convert once with .float())" % (t.dtype,))
        arr[i].kind = kind
        arr[i].dtype = _DTYPES[tensors[0].dtype] if tensors else capi.F32
        for slot, t in zip(("p0", "p1", "p2", "p3"), tensors):
            setattr(arr[i], slot, t.data_ptr())
            keep.append(t)
        arr[i].epsilon = float(scalars[0]) if scalars else 0.0
        arr[i].ld = 0
        if kind == capi.OP_RESIDUAL_ADD and tensors:
            arr[i].ld = tensors[0].stride(-2) if tensors[0].dim() >= 2 else 0
    return arr, keep


def gemm_ex(a, b, ops, out=None, out_dtype=None):
    """GEMM with an explicit operator chain, e.g. [(OP_BIAS_ADD, bias), (OP_RELU,)]."""
    m, _ = a.shape
    _, n = b.shape
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype or a.dtype, device=a.device)
    va, vb, vc = _view(a), _view(b), _view(out)
    arr, _keep = _ops_array(ops)
    params = capi.GemmParams(capi.EPI_IDENTITY, _stream(a))
    st = capi.lib().tracea_gemm_ex(va.c, vb.c, C.byref(vc.c), params, arr, len(ops))
    capi.check("tracea_gemm_ex", st)
    return out


def conv_out_shape(x_shape, w_shape, stride, padding, dilation):
    n, h, w, _ = x_shape
    k, r, s, _ = w_shape
    ho = (h + 2 * padding[0] - dilation[0] * (r - 1) - 1) // stride[0] + 1
    wo = (w + 2 * padding[1] - dilation[1] * (s - 1) - 1) // stride[1] + 1
    return (n, ho, wo, k)


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def _weight_view(w, layout):
    """Filter view with dims [K,R,S,C] whatever the storage order."""
    if layout == "krsc":
        return _view(w)
    if layout == "rsck":
        r, s, c, k = w.shape
        sr, ss, sc, sk = w.stride()
        return _view(w, shape=(k, r, s, c), stride=(sk, sr, ss, sc))
    raise ValueError("weight layout must be 'krsc' or 'rsck'")


def conv2d(x, w, bias=None, residual=None, stride=1, padding=0, dilation=1, epilogue="none",
           out=None, weight_layout="krsc", out_dtype=None):
    """x [N,H,W,C] (NHWC); w [K,R,S,C] ('krsc') or [R,S,C,K] ('rsck'); out [N,Ho,Wo,K]."""
    stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
    vw = _weight_view(w, weight_layout)
    if out is None:
        wshape = tuple(vw.c.shape[i] for i in range(4))
        out = torch.empty(conv_out_shape(x.shape, wshape, stride, padding, dilation),
                          dtype=out_dtype or x.dtype, device=x.device)
    vx, vo = _view(x), _view(out)
    vbias = _view(bias) if bias is not None else None
    vres = _view(residual) if residual is not None else None
    params = capi.Conv2dParams(stride[0], stride[1], padding[0], padding[1], dilation[0],
                               dilation[1], 1, parse_epilogue(epilogue), _stream(x))
    st = capi.lib().tracea_conv2d(vx.c, vw.c, C.byref(vbias.c) if vbias else None,
                                  C.byref(vres.c) if vres else None, C.byref(vo.c), params)
    capi.check("tracea_conv2d", st)
    return out


def conv2d_ex(x, w, ops, stride=1, padding=0, dilation=1, out=None, weight_layout="krsc",
              out_dtype=None):
    """Convolution with an explicit operator chain (BatchNorm, scale/shift, ...)."""
    stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
    vw = _weight_view(w, weight_layout)
    if out is None:
        wshape = tuple(vw.c.shape[i] for i in range(4))
        out = torch.empty(conv_out_shape(x.shape, wshape, stride, padding, dilation),
                          dtype=out_dtype or x.dtype, device=x.device)
    vx, vo = _view(x), _view(out)
    arr, _keep = _ops_array(ops)
    params = capi.Conv2dParams(stride[0], stride[1], padding[0], padding[1], dilation[0],
                               dilation[1], 1, capi.EPI_IDENTITY, _stream(x))
    st = capi.lib().tracea_conv2d_ex(vx.c, vw.c, C.byref(vo.c), params, arr, len(ops))
    capi.check("tracea_conv2d_ex", st)
    return out


def conv_transpose_out_shape(x_shape, w_shape, stride, padding, output_padding):
    n, h, w, _ = x_shape
    k, r, s, _ = w_shape
    ho = (h - 1) * stride[0] - 2 * padding[0] + r + output_padding[0]
    wo = (w - 1) * stride[1] - 2 * padding[1] + s + output_padding[1]
    return (n, ho, wo, k)


def _transposed_weight_view(w, layout):
    """Filter view with dims [K,R,S,C] (K output channels) whatever the storage order."""
    order = {"crsk": (3, 1, 2, 0),   # the reference kernel's [C*R*S, K] rows
             "ckrs": (1, 2, 3, 0),   # torch.nn.ConvTranspose2d.weight
             "krsc": (0, 1, 2, 3),
             "rskc": (2, 0, 1, 3)}.get(layout)  # what the half-precision GEMM stage reads in place
    if order is None:
        raise ValueError("weight layout must be 'crsk', 'ckrs', 'krsc' or 'rskc'")
    return _view(w, shape=tuple(w.shape[i] for i in order), stride=tuple(w.stride()[i] for i in order))


def _conv_transpose_setup(x, w, stride, padding, output_padding, out, weight_layout, out_dtype):
    stride, padding, output_padding = _pair(stride), _pair(padding), _pair(output_padding)
    vw = _transposed_weight_view(w, weight_layout)
    wshape = tuple(vw.c.shape[i] for i in range(4))
    if out is None:
        out = torch.empty(conv_transpose_out_shape(x.shape, wshape, stride, padding, output_padding),
                          dtype=out_dtype or x.dtype, device=x.device)
    return vw, out, stride, padding, output_padding


def conv_transpose2d(x, w, bias=None, residual=None, stride=1, padding=0, output_padding=0, epilogue="none",
                     out=None, weight_layout="crsk", out_dtype=None):
    """x [N,H,W,C] (NHWC); w [C,R,S,K] ('crsk'), [C,K,R,S] ('ckrs'), [K,R,S,C] ('krsc') or [R,S,K,C]
    ('rskc'); out [N,Ho,Wo,K]
    with Ho = (H-1)*stride - 2*padding + R + output_padding."""
    vw, out, stride, padding, output_padding = _conv_transpose_setup(x, w, stride, padding, output_padding, out,
                                                                     weight_layout, out_dtype)
    vx, vo = _view(x), _view(out)
    vbias = _view(bias) if bias is not None else None
    vres = _view(residual) if residual is not None else None
    params = capi.ConvTranspose2dParams(stride[0], stride[1], padding[0], padding[1], output_padding[0],
                                        output_padding[1], 1, 1, 1, parse_epilogue(epilogue), _stream(x))
    st = capi.lib().tracea_conv_transpose2d(vx.c, vw.c, C.byref(vbias.c) if vbias else None,
                                            C.byref(vres.c) if vres else None, C.byref(vo.c), params)
    capi.check("tracea_conv_transpose2d", st)
    return out


def conv_transpose2d_ex(x, w, ops, stride=1, padding=0, output_padding=0, out=None, weight_layout="crsk",
                        out_dtype=None):
    """Transposed convolution with an explicit operator chain."""
    vw, out, stride, padding, output_padding = _conv_transpose_setup(x, w, stride, padding, output_padding, out,
                                                                     weight_layout, out_dtype)
    vx, vo = _view(x), _view(out)
    arr, _keep = _ops_array(ops)
    params = capi.ConvTranspose2dParams(stride[0], stride[1], padding[0], padding[1], output_padding[0],
                                        output_padding[1], 1, 1, 1, capi.EPI_IDENTITY, _stream(x))
    st = capi.lib().tracea_conv_transpose2d_ex(vx.c, vw.c, C.byref(vo.c), params, arr, len(ops))
    capi.check("tracea_conv_transpose2d_ex", st)
    return out


def attention(q, k, v, causal=False, scale=0.0, out=None):
    """q,k,v [B,H,S,D] -> softmax(scale q k^T) v; scale 0 means 1/sqrt(D)."""
    if out is None:
        out = torch.empty_like(q)
    vq, vk, vv, vo = _view(q), _view(k), _view(v), _view(out)
    params = capi.AttentionParams(1 if causal else 0, 0, float(scale), _stream(q))
    st = capi.lib().tracea_attention(vq.c, vk.c, vv.c, C.byref(vo.c), params)
    capi.check("tracea_attention", st)
    return out
