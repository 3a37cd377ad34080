"""Feed-forward parts."""

import ctypes

import torch

from ..ops import kernels, native
from .base import FeedForward, TensorSpec, register_feed_forward, value_of

_TANH_GELU = ("gelu_new", "gelu_pytorch_tanh", "gelu_tanh", "gelu_approx")


class GeluMLP(FeedForward):
    """``residual += c_proj(gelu_tanh(c_fc(x)))``, dense, with biases.

    mlx_lm/models/gpt2.py:71-80; the activation and the bias add are fused
    into the first product, the residual add into the second.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    accepts_lazy_input = True  # the first product can norm its input itself

    def __init__(self, width, inner, activation="gelu_new", prefix=""):
        super().__init__(prefix)
        if activation not in _TANH_GELU:
            raise ValueError(
                f"activation '{activation}' is not implemented (only the tanh GELU: {_TANH_GELU})"
            )
        if width % 8:
            raise ValueError(f"the feed-forward's width must be a multiple of 8, got {width}")
        if inner <= 0:
            raise ValueError(f"the feed-forward's inner size must be positive, got {inner}")
        self.width, self.inner = width, inner
        # The products want a multiple of 8 along K.  Inner features beyond ``inner`` get zero
        # weights and a zero bias: gelu(0) = 0 meets zero columns, so the sum is unchanged.
        self.inner_padded = (inner + 7) // 8 * 8
        self.fc_w = self.fc_b = self.proj_w = self.proj_b = None

    def tensors(self):
        n = self._name
        return {
            n("c_fc.weight"): TensorSpec((self.inner, self.width), "matrix"),
            n("c_fc.bias"): TensorSpec((self.inner,), "vector"),
            n("c_proj.weight"): TensorSpec((self.width, self.inner), "matrix"),
            n("c_proj.bias"): TensorSpec((self.width,), "vector"),
        }

    def load(self, tensors):
        n = self._name
        self.fc_w, self.fc_b = tensors[n("c_fc.weight")], tensors[n("c_fc.bias")]
        self.proj_w, self.proj_b = tensors[n("c_proj.weight")], tensors[n("c_proj.bias")]
        pad = self.inner_padded - self.inner
        if pad:
            self.fc_w = torch.cat([self.fc_w, self.fc_w.new_zeros(pad, self.width)]).contiguous()
            self.fc_b = torch.cat([self.fc_b, self.fc_b.new_zeros(pad)]).contiguous()
            self.proj_w = torch.cat([self.proj_w, self.proj_w.new_zeros(self.width, pad)], dim=1).contiguous()
        self.fc_w, self.proj_w = kernels.for_decode(self.fc_w), kernels.for_decode(self.proj_w)
        self.first_weight = self.fc_w  # what the first product reads

    def make_native(self):
        fc_w, proj_w = kernels.weight_struct(self.fc_w), kernels.weight_struct(self.proj_w)
        return native.made(native.lib().eng_make_gelu_mlp(
            self.width, self.inner_padded, ctypes.byref(fc_w), native.ptr(self.fc_b), ctypes.byref(proj_w),
            native.ptr(self.proj_b)), "gelu_mlp")

    def forward(self, ctx, x, residual):
        v, r = value_of(x), native.mat(residual)
        with ctx.enter():
            rc = native.lib().eng_ffn_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(v), ctypes.byref(r))
        native.check(rc, "gelu_mlp")


class Relu2MLP(FeedForward):
    """``down(relu(up(x))^2)``, dense, no biases.

    The activation is fused into the first product.  The second adds into ``residual``, or, in an
    arrangement that wants the output by itself (``post_norm``), writes it there.  No counterpart
    in mlx_lm/models/gpt2.py, whose MLP is the tanh GELU's.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, width, inner, up_name="up", down_name="down", prefix=""):
        super().__init__(prefix)
        if width % 8:
            raise ValueError(f"the feed-forward's width must be a multiple of 8, got {width}")
        if inner <= 0:
            raise ValueError(f"the feed-forward's inner size must be positive, got {inner}")
        self.width, self.inner = width, inner
        self.inner_padded = (inner + 7) // 8 * 8  # zero weights beyond ``inner``: relu(0)^2 = 0 meets zero columns
        self.up_name, self.down_name = self._name(up_name), self._name(down_name)
        self.up_w = self.down_w = None

    def tensors(self):
        return {self.up_name: TensorSpec((self.inner, self.width), "matrix"),
                self.down_name: TensorSpec((self.width, self.inner), "matrix")}

    def load(self, tensors):
        up, down = tensors[self.up_name], tensors[self.down_name]
        pad = self.inner_padded - self.inner
        if pad:
            up = torch.cat([up, up.new_zeros(pad, self.width)]).contiguous()
            down = torch.cat([down, down.new_zeros(self.width, pad)], dim=1).contiguous()
        self.up_w, self.down_w = kernels.for_decode(up), kernels.for_decode(down)
        self.first_weight = self.up_w

    def make_native(self):
        W = ctypes.POINTER(native.EngWeight)
        L = native.part_library("relu2_mlp", {"make_relu2_mlp": [ctypes.c_int, ctypes.c_int, W, W]})
        up_w, down_w = kernels.weight_struct(self.up_w), kernels.weight_struct(self.down_w)
        return native.made(L.make_relu2_mlp(native.host(), self.width, self.inner_padded, ctypes.byref(up_w),
                                            ctypes.byref(down_w)), "relu2_mlp")

    def forward(self, ctx, x, residual):
        v, r = value_of(x), native.mat(residual)
        with ctx.enter():
            rc = native.lib().eng_ffn_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(v), ctypes.byref(r))
        native.check(rc, "relu2_mlp")


class GatedMLP(FeedForward):
    """``down(act(gate(x)) * up(x))``, dense, no biases; ``activation``: ``silu`` or ``gelu_tanh``.

    One product gives ``[gate | up]``; the activation and the product of the two halves are one
    kernel (``silu_mul``, which the experts' shared expert uses too); the second product adds into
    ``residual``.  No counterpart in mlx_lm/models/gpt2.py, whose MLP (:71-80) has no gate.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    takes_normed_input = True  # ``x`` may be a ``kernels.NormedInput``: the first product norms the rows itself

    def __init__(self, width, inner, gate_name="gate", up_name="up", down_name="down", activation="silu", prefix=""):
        super().__init__(prefix)
        if activation not in kernels.GATE_ACTIVATIONS:
            raise ValueError(f"gate activation {activation!r} is not implemented (known: {sorted(kernels.GATE_ACTIVATIONS)})")
        self.activation = activation
        if width % 8:
            raise ValueError(f"the feed-forward's width must be a multiple of 8, got {width}")
        if inner <= 0:
            raise ValueError(f"the feed-forward's inner size must be positive, got {inner}")
        self.width, self.inner = width, inner
        self.inner_padded = (inner + 7) // 8 * 8  # zero weights beyond ``inner``: silu(0) * 0 = 0 meets zero columns
        self.gate_name, self.up_name, self.down_name = self._name(gate_name), self._name(up_name), self._name(down_name)
        self.gate_up_w = self.down_w = None

    def tensors(self):
        return {self.gate_name: TensorSpec((self.inner, self.width), "matrix"),
                self.up_name: TensorSpec((self.inner, self.width), "matrix"),
                self.down_name: TensorSpec((self.width, self.inner), "matrix")}

    def load(self, tensors):
        gate, up, down = tensors[self.gate_name], tensors[self.up_name], tensors[self.down_name]
        pad = self.inner_padded - self.inner
        if pad:
            zeros = gate.new_zeros(pad, self.width)
            gate, up = torch.cat([gate, zeros]), torch.cat([up, zeros])
            down = torch.cat([down, down.new_zeros(self.width, pad)], dim=1)
        self.gate_up_w = kernels.for_decode(torch.cat([gate, up]).contiguous())
        self.down_w = kernels.for_decode(down.contiguous())
        self.first_weight = self.gate_up_w

    def forward(self, ctx, x, residual):
        T, F = x.shape[0], self.inner_padded
        mark = ctx.scratch_mark()
        gate_up = ctx.scratch((T, 2 * F), ctx.dtype)
        kernels.linear(gate_up, x, self.gate_up_w, splits=kernels.splits_alone(T))
        act = ctx.scratch((T, F), ctx.dtype)
        kernels.silu_mul(act, gate_up, self.activation)
        kernels.linear(residual, act, self.down_w, accumulate=True, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


register_feed_forward("gelu_mlp", GeluMLP)
register_feed_forward("gated_mlp", GatedMLP)
register_feed_forward("relu2_mlp", Relu2MLP)
