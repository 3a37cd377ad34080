"""Norms over the width of the residual stream."""

import ctypes

from ..ops import kernels, native
from .base import Norm, TensorSpec, register_norm


class LayerNorm(Norm):
    """``(x - mean) / sqrt(var + eps) * weight + bias`` with biased variance.

    ``nn.LayerNorm(n_embd, eps=layer_norm_epsilon)`` in
    mlx_lm/models/gpt2.py:92-96,123.  Reads the float32 residual stream,
    computes in float32, writes the compute dtype.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, width, eps, bias=True, weight_name="weight", bias_name="bias", prefix=""):
        super().__init__(prefix)
        self.width, self.eps, self.has_bias = width, float(eps), bias
        self.weight_name, self.bias_name = self._name(weight_name), self._name(bias_name)
        self.weight = self.bias = None

    def tensors(self):
        t = {self.weight_name: TensorSpec((self.width,), "vector")}
        if self.has_bias:
            t[self.bias_name] = TensorSpec((self.width,), "vector")
        return t

    def load(self, tensors):
        self.weight = tensors[self.weight_name]
        self.bias = tensors[self.bias_name] if self.has_bias else None

    settles_pending = True  # adds a sum that is pending on ``x`` before (or while) it norms the rows
    reads_ahead = True  # ``forward`` takes ``ahead``, the weights that its result meets first

    def make_native(self):
        return native.made(native.lib().eng_make_layernorm(self.width, self.eps, native.ptr(self.weight),
                                                           native.ptr(self.bias)), "layernorm")

    def forward(self, ctx, x, rows=None, n_rows=None, lazy=False, ahead=None):
        """``ahead``: the weights of the product that reads the result first, if its caller knows
        them: a kernel here that leaves most of the GPU idle reads them into the caches meanwhile.
        (The native twin does the work: a pending sum is added, fused with the norm where the
        kernel takes it; with ``lazy`` the norm may be left to the consumer's first product.)"""
        out = native.EngValue()
        xm = native.mat(x)
        with ctx.enter():
            rc = native.lib().eng_norm_forward(
                self.native(), ctypes.byref(ctx.c), ctypes.byref(xm), native.ptr(rows), int(n_rows or 0),
                int(bool(lazy)), ctypes.byref(ahead.c) if ahead is not None and hasattr(ahead, "c") else None,
                ctypes.byref(out))
        native.check(rc, "layernorm")
        if out.lazy:
            return kernels.NormedInput(ctx.scratch, x, self.weight, self.bias, self.eps, ctx.dtype)
        return ctx.tensor(out.m)


class RMSNorm(Norm):
    """``x / sqrt(mean(x^2) + eps) * weight``: no mean is taken off, eps sits inside the root.
    With ``offset`` the scale is ``offset + weight`` (a tensor that holds the scale's difference from one: ``offset = 1``).

    Reads the float32 residual stream, computes in float32, writes the compute dtype (``rows``:
    only those rows, for the rows whose logits are wanted).  An arrangement that norms after
    its sums (``post_norm``) takes ``weight`` and ``eps`` from here and fuses the norm into its
    own kernel.  No counterpart in mlx_lm/models/gpt2.py, whose norms are LayerNorms.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, width, eps, weight_name="weight", offset=0.0, prefix=""):
        super().__init__(prefix)
        if eps < 0:
            raise ValueError(f"eps must not be negative, got {eps}")
        self.width, self.eps, self.offset = width, float(eps), float(offset)
        self.weight_name = self._name(weight_name)
        self.weight = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.width,), "vector")}

    def load(self, tensors):
        # ``offset``: the scale is ``offset + tensor`` (float32)
        self.weight = tensors[self.weight_name] + self.offset if self.offset else tensors[self.weight_name]

    def make_native(self):
        L = native.part_library("rmsnorm", {"make_rmsnorm": [ctypes.c_int, ctypes.c_float, ctypes.c_void_p]})
        return native.made(L.make_rmsnorm(native.host(), self.width, self.eps, native.ptr(self.weight)), "rmsnorm")

    def forward(self, ctx, x, rows=None, n_rows=None, lazy=False):
        out = native.EngValue()
        xm = native.mat(x)
        with ctx.enter():
            rc = native.lib().eng_norm_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(xm), native.ptr(rows),
                                               int(n_rows or 0), 0, None, ctypes.byref(out))
        native.check(rc, "rmsnorm")
        return ctx.tensor(out.m)


register_norm("layernorm", LayerNorm)
register_norm("rmsnorm", RMSNorm)
