"""The reference's Python package surface, served by ``libtracea.so``.

``from tracea_amd import tracea_compat as tracea`` gives what
``import tracea`` gives with the reference (tracea-python/python/tracea/__init__.py:12-56):
``tracea.ops``, ``tracea.Context`` (the PyContext methods of
src/interface/python.rs:89-547 that belong to the dense-contraction path),
``tracea.patch_conv2d`` and ``tracea.TraceaConv2d``.  Tensors are torch tensors
on the GPU; nothing is copied except where a layout has to change (NCHW module
weights are repacked once per weight version).
"""
import math

import torch

from .. import capi
from .. import ops as _ops

__version__ = "0.1.0"
__all__ = ["ops", "Context", "__version__", "patch_conv2d", "TraceaConv2d", "parse_epilogue"]


def parse_epilogue(spec, bias=None, residual=None):
    """"bias+relu" -> operator chain, the grammar of src/interface/python.rs:41-87:
    '+'-separated, case-insensitive names out of identity / relu / gelu / silu / bias /
    residual, applied left to right; 'bias' or 'residual' without the tensor and any
    other name raise ValueError."""
    chain = []
    if spec is None:
        return chain
    for part in spec.split("+"):
        name = part.strip().lower()
        if name == "identity":
            continue
        if name == "relu":
            chain.append((capi.OP_RELU,))
        elif name == "gelu":
            chain.append((capi.OP_GELU,))
        elif name == "silu":
            chain.append((capi.OP_SILU,))
        elif name == "bias":
            if bias is None:
                raise ValueError("Epilogue contains 'bias' but no bias argument provided")
            chain.append((capi.OP_BIAS_ADD, bias))
        elif name == "residual":
            if residual is None:
                raise ValueError("Epilogue contains 'residual' but no reference provided")
            chain.append((capi.OP_RESIDUAL_ADD, residual))
        else:
            raise ValueError("Unknown epilogue op: %s" % part)
    if len(chain) > capi.MAX_EPILOGUE_OPS:
        raise ValueError("at most %d epilogue operators are supported" % capi.MAX_EPILOGUE_OPS)
    return chain


def _check_shape(name, t, shape):
    if tuple(t.shape) != tuple(shape):
        raise ValueError("%s has shape %s, the arguments say %s" % (name, tuple(t.shape), tuple(shape)))


class Context:
    """``tracea.Context`` (src/interface/python.rs:24, 89-97).  ``arch`` is accepted and ignored,
    as in the reference.  Every method writes its pre-allocated output tensor and returns the
    index of the kernel variant that ran (the reference returns its kernel id)."""

    def __init__(self, arch=None):
        capi.init()

    def synchronize(self):
        torch.cuda.synchronize()

    def gemm(self, a, b, c, m, n, k, m_tile=None, n_tile=None, k_tile=None, epilogue=None, bias=None,
             residual=None, variant=None):
        """c [m,n] = epilogue(a [m,k] . b [k,n]) (python.rs:280-366).  The tile and variant hints
        select among kernels the reference generates at run time; here the precompiled variant
        comes from the tuning cache or the selector."""
        _check_shape("a", a, (m, k)); _check_shape("b", b, (k, n)); _check_shape("c", c, (m, n))
        _ops.gemm_ex(a, b, parse_epilogue(epilogue, bias, residual), out=c)
        return _variant_index("gemm")

    def conv2d(self, x, w, o, n, c, h, w_in, k, r, s, stride=1, pad=0, dilation=1, epilogue=None, bias=None,
               residual=None):
        """x [n,h,w_in,c] NHWC, w [k,r,s,c], o [n,ho,wo,k] (python.rs:367-462)."""
        _check_shape("x", x, (n, h, w_in, c)); _check_shape("w", w, (k, r, s, c))
        _ops.conv2d_ex(x, w, parse_epilogue(epilogue, bias, residual), stride=stride, padding=pad,
                       dilation=dilation, out=o)
        return _variant_index("conv2d")

    def conv_transpose2d(self, x, w, o, n, c, h, w_in, k, r, s, stride=1, pad=0, output_padding=0, dilation=1,
                         epilogue=None, bias=None, residual=None):
        """x [n,h,w_in,c] NHWC, w with dims [k,r,s,c] as the reference reads them and the storage
        order of its strides, o [n,ho,wo,k] (python.rs:465-546)."""
        _check_shape("x", x, (n, h, w_in, c)); _check_shape("w", w, (k, r, s, c))
        if dilation != 1:
            raise ValueError("conv_transpose2d: dilation must be 1")
        _ops.conv_transpose2d_ex(x, w, parse_epilogue(epilogue, bias, residual), stride=stride, padding=pad,
                                 output_padding=output_padding, out=o, weight_layout="krsc")
        # the kernel that ran: a convolution variant when the call went out by output phase, else the
        # GEMM of the partial-product form (an index into the one variant table both operators share)
        by_phase = _variant_index("conv2d")
        return by_phase if by_phase >= 0 else _variant_index("gemm")

    def attention(self, q, k, v, o, b_in, h_in, s_in, d_in, dh_in, causal=False, scale_sqrt=True, m_tile=None,
                  n_tile=None, stages=None, warps=None, softmax_mode=None, variant=None):
        """o = softmax(scale q k^T) v on [b,h,s,dh] tensors (python.rs:124-278); scale is
        1/sqrt(dh) when scale_sqrt, else 1.  The softmax granularity modes all compute the same
        function; the kernel here rescales per key tile."""
        for name, t in (("q", q), ("k", k), ("v", v), ("o", o)):
            _check_shape(name, t, (b_in, h_in, s_in, dh_in))
        _ops.attention(q, k, v, causal=causal, scale=(1.0 / math.sqrt(dh_in)) if scale_sqrt else 1.0, out=o)
        return _variant_index("attention")


def _variant_index(op):
    name = capi.last_variant(op)
    names = capi.variants(op)
    return names.index(name) if name in names else -1


from . import ops  # noqa: E402  (needs Context)


class TraceaConv2d(torch.nn.Conv2d):
    """Drop-in replacement for torch.nn.Conv2d (tracea-python/python/tracea/__init__.py:29-56):
    NCHW in, NCHW out.  groups != 1, dilation != (1,1), a padding mode other than "zeros" fall back
    to PyTorch as in the reference; so does what the convolution kernels here do not take: tensors
    off the GPU, dtypes other than f16 / bf16, string padding.  (Input channels that are not a multiple of 8,
    an RGB first layer, run from copies padded to 8 inside the library.)"""

    def _tracea_supported(self, x):
        return (self.groups == 1 and self.dilation == (1, 1) and self.padding_mode == "zeros"
                and not isinstance(self.padding, str) and x.is_cuda and x.dim() == 4
                and x.dtype in (torch.float16, torch.bfloat16) and self.weight.dtype == x.dtype)

    def _tracea_weight(self):
        # [K,C,R,S] -> [K,R,S,C], once per weight version
        key = (self.weight.data_ptr(), self.weight._version, self.weight.dtype)
        cached = getattr(self, "_tracea_w", None)
        if cached is None or cached[0] != key:
            cached = (key, self.weight.detach().permute(0, 2, 3, 1).contiguous())
            self._tracea_w = cached
        return cached[1]

    def _needs_grad(self, x):
        # the kernels here are forward only and their result carries no grad_fn: a training step
        # must go through PyTorch, or it would silently get no gradients
        return torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad
                                            or (self.bias is not None and self.bias.requires_grad))

    def forward(self, x):
        if not self._tracea_supported(x) or self._needs_grad(x):
            return super().forward(x)
        x_nhwc = x.permute(0, 2, 3, 1).contiguous()  # free for a channels_last tensor
        bias = self.bias.detach() if self.bias is not None else None
        y = _ops.conv2d(x_nhwc, self._tracea_weight(), bias=bias, stride=self.stride, padding=self.padding,
                        epilogue="bias" if bias is not None else "none")
        return y.permute(0, 3, 1, 2)  # NCHW view of channels_last storage


_TORCH_CONV2D = torch.nn.Conv2d


def patch_conv2d():
    """Monkey patch torch.nn.Conv2d to use this backend (reference __init__.py:18-26).
    Modules built afterwards are TraceaConv2d; unsupported configurations fall back to PyTorch."""
    torch.nn.Conv2d = TraceaConv2d


def unpatch_conv2d():
    """Undo patch_conv2d (no counterpart in the reference; for tests and notebooks)."""
    torch.nn.Conv2d = _TORCH_CONV2D
