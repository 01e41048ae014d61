"""ctypes front end of the CPU checker in ``tracea_oracle.c``.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  The product library never
loads it.  Every routine takes and returns numpy arrays; half-precision inputs
are passed as float32 arrays that already hold the rounded values.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

EPI_NONE, EPI_BIAS_ADD, EPI_RELU, EPI_GELU, EPI_SILU = 0, 1, 2, 3, 4
EPI_RESIDUAL_ADD, EPI_BIAS_ADD_SILU, EPI_BATCHNORM, EPI_SCALE_SHIFT = 5, 6, 7, 8


def build(force=False):
    """Compile ``liboracle.so`` next to its source (gcc, a second or two)."""
    src = os.path.join(_HERE, "tracea_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "liboracle.so"])
    return _LIB_PATH


class _EpilogueOp(C.Structure):
    _fields_ = [("kind", C.c_int32), ("epsilon", C.c_float),
                ("p0", C.c_void_p), ("p1", C.c_void_p), ("p2", C.c_void_p), ("p3", C.c_void_p)]


class ConvParams(C.Structure):
    """80-byte ConvParams block (reference: src/emitter/cuda/conv.rs:134-142)."""
    _fields_ = [(n, C.c_int32) for n in
                ("batch", "h_in", "w_in", "c_in", "k_out", "h_out", "w_out", "r_sz", "s_sz",
                 "stride", "pad", "dilation")] + \
               [(n, C.c_uint32) for n in
                ("hw_m", "hw_s", "w_m", "w_s", "sic_m", "sic_s", "c_m", "c_s")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_divmod_check.restype = C.c_int64
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def default_threads():
    return max(1, min(os.cpu_count() or 1, 64))


def gemm_cpu_packed(a, b, c, mc=128, nc=128, kc=256, mr=6, k_unroll=4, prefetch_distance=128,
                    nthreads=None):
    """c += a @ b in place (fp32, row-major), hero tiling by default
    (reference: src/optimizer/heroscope.rs:18-23, src/optimizer/policy.rs:484-505)."""
    assert a.dtype == np.float32 and b.dtype == np.float32 and c.dtype == np.float32
    assert a.flags.c_contiguous and b.flags.c_contiguous and c.flags.c_contiguous
    m, k = a.shape
    k2, n = b.shape
    assert k == k2 and c.shape == (m, n)
    rc = lib().oracle_gemm_cpu_packed(m, n, k, mc, nc, kc, mr, k_unroll, prefetch_distance,
                                      _ptr(a), _ptr(b), _ptr(c),
                                      nthreads or default_threads())
    if rc != 0:
        raise ValueError("oracle_gemm_cpu_packed: bad argument")
    return c


def gemm_f64(a, b, nthreads=None):
    """float64 a @ b for float32 a [M,K] and b [K,N]; any element strides."""
    assert a.dtype == np.float32 and b.dtype == np.float32
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    out = np.empty((m, n), dtype=np.float64)
    sa = [s // 4 for s in a.strides]
    sb = [s // 4 for s in b.strides]
    rc = lib().oracle_gemm_f64(m, n, k, _ptr(a), C.c_int64(sa[0]), C.c_int64(sa[1]),
                               _ptr(b), C.c_int64(sb[0]), C.c_int64(sb[1]), _ptr(out),
                               nthreads or default_threads())
    if rc != 0:
        raise ValueError("oracle_gemm_f64: bad argument")
    return out


def epilogue_apply(x, ops):
    """Apply an epilogue chain in order to a copy of x ([rows, cols] fp32).

    ops: list of tuples (kind, *arrays[, epsilon]) --
      (EPI_BIAS_ADD, bias) (EPI_RELU,) (EPI_GELU,) (EPI_SILU,) (EPI_RESIDUAL_ADD, res)
      (EPI_BIAS_ADD_SILU, bias) (EPI_BATCHNORM, gamma, beta, mean, var, eps)
      (EPI_SCALE_SHIFT, scale, shift)
    """
    x = _f32(x).copy()
    rows = int(np.prod(x.shape[:-1]))
    cols = x.shape[-1]
    arr = (_EpilogueOp * max(1, len(ops)))()
    keep = []
    for i, op in enumerate(ops):
        kind = op[0]
        arr[i].kind = kind
        arrays = [_f32(t) for t in op[1:] if isinstance(t, np.ndarray)]
        keep.extend(arrays)
        if kind == EPI_BATCHNORM:
            arr[i].epsilon = float(op[5])
        for slot, t in zip(("p0", "p1", "p2", "p3"), arrays):
            setattr(arr[i], slot, t.ctypes.data)
    rc = lib().oracle_epilogue_apply(_ptr(x), C.c_int64(rows), C.c_int64(cols), arr, len(ops))
    if rc != 0:
        raise ValueError("oracle_epilogue_apply: unknown op")
    return x


def magic_u32(n):
    m, p = C.c_uint32(), C.c_uint32()
    lib().oracle_magic_u32(C.c_uint32(n), C.byref(m), C.byref(p))
    return m.value, p.value


def fast_divmod(n, m, s, d):
    q, r = C.c_int32(), C.c_int32()
    lib().oracle_fast_divmod(C.c_int32(n), C.c_uint32(m), C.c_int32(s), C.c_int32(d),
                             C.byref(q), C.byref(r))
    return q.value, r.value


def divmod_check(d, n_max):
    """First n < n_max where fast_divmod disagrees with (/, %), or -1."""
    return int(lib().oracle_divmod_check(C.c_uint32(d), C.c_uint32(n_max)))


def conv_params(n, h, w, c, k, r, s, stride, pad, dilation=1):
    p = ConvParams()
    rc = lib().oracle_conv_params_pack(n, h, w, c, k, r, s, stride, pad, dilation, C.byref(p))
    if rc != 0:
        raise ValueError("oracle_conv_params_pack: bad argument")
    return p


def conv_coords(p):
    m = p.batch * p.h_out * p.w_out
    kk = p.r_sz * p.s_sz * p.c_in
    rows = np.empty((m, 3), dtype=np.int32)
    base = np.empty((m,), dtype=np.int64)
    cols = np.empty((kk, 3), dtype=np.int32)
    lib().oracle_conv_coords(C.byref(p), _ptr(rows), _ptr(base), _ptr(cols))
    return rows, base, cols


def conv2d_nhwc(x, w, stride=1, pad=0, dilation=1, nthreads=None):
    """x [N,H,W,C], w [R,S,C,K] -> [N,Ho,Wo,K] float32."""
    x, w = _f32(x), _f32(w)
    n, h, wd, c = x.shape
    r, s, c2, k = w.shape
    assert c == c2
    ho = (h + 2 * pad - dilation * (r - 1) - 1) // stride + 1
    wo = (wd + 2 * pad - dilation * (s - 1) - 1) // stride + 1
    y = np.empty((n, ho, wo, k), dtype=np.float32)
    rc = lib().oracle_conv2d_nhwc(_ptr(x), _ptr(w), _ptr(y), n, h, wd, c, k, r, s, stride, pad,
                                  dilation, nthreads or default_threads())
    if rc != 0:
        raise ValueError("oracle_conv2d_nhwc: bad argument")
    return y


def conv_transpose_out_shape(h, w, r, s, stride, pad, output_padding):
    """(H_out, W_out) of the reference (src/emitter/conv_transpose.rs:36-37)."""
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    oh, ow = _pair(output_padding)
    return (h - 1) * sh - 2 * ph + r + oh, (w - 1) * sw - 2 * pw + s + ow


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def conv_transpose2d_nhwc(x, w, stride=1, pad=0, output_padding=0, nthreads=None):
    """x [N,H,W,C], w [C,R,S,K] (the reference kernel's [C*R*S, K] rows) -> [N,Ho,Wo,K] float32."""
    x, w = _f32(x), _f32(w)
    n, h, wd, c = x.shape
    c2, r, s, k = w.shape
    assert c == c2
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    oh, ow = _pair(output_padding)
    ho, wo = conv_transpose_out_shape(h, wd, r, s, stride, pad, output_padding)
    if ho <= 0 or wo <= 0:
        raise ValueError("oracle_conv_transpose2d_nhwc: empty output")
    y = np.empty((n, ho, wo, k), dtype=np.float32)
    rc = lib().oracle_conv_transpose2d_nhwc(_ptr(x), _ptr(w), _ptr(y), n, h, wd, c, k, r, s, sh, sw,
                                            ph, pw, oh, ow, nthreads or default_threads())
    if rc != 0:
        raise ValueError("oracle_conv_transpose2d_nhwc: bad argument")
    return y


def attention(q, k, v, scale, causal, rows=None, nthreads=None):
    """One (batch, head) slice: q,k,v [S,D] -> out [len(rows), D] float32."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    s, d = q.shape
    if rows is None:
        rows = np.arange(s, dtype=np.int32)
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    out = np.empty((len(rows), d), dtype=np.float32)
    rc = lib().oracle_attention(_ptr(q), _ptr(k), _ptr(v), _ptr(out), s, d, C.c_float(scale),
                                int(bool(causal)), _ptr(rows), len(rows),
                                nthreads or default_threads())
    if rc != 0:
        raise ValueError("oracle_attention: bad argument")
    return out


def attention_bhsd(q, k, v, scale, causal, nthreads=None):
    """q,k,v [B,H,S,D] -> [B,H,S,D] float32 (full check for small sizes)."""
    b, h, s, d = q.shape
    out = np.empty((b, h, s, d), dtype=np.float32)
    for bi in range(b):
        for hi in range(h):
            out[bi, hi] = attention(q[bi, hi], k[bi, hi], v[bi, hi], scale, causal,
                                    nthreads=nthreads)
    return out
