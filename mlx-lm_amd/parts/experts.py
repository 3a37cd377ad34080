"""A feed-forward of many small gated experts of which every token uses a few."""

import torch

from ..ops import kernels
from .base import FeedForward, TensorSpec, register_feed_forward


class GatedExperts(FeedForward):
    """``sum over a token's chosen experts of s_e * expert_e(x)  (+ shared(x))`` with

    * ``expert(x) = Wdown (silu(Wgate x) * (Wup x))``, no biases; ``n_experts`` of them with tensors
      ``e<i>.gate``, ``e<i>.up`` (``[inner, width]``) and ``e<i>.down`` (``[width, inner]``);
    * ``s = softmax(Wrouter x)`` over all ``n_experts + n_identity`` router outputs (32-bit sums
      of the products of the compute dtype's operands); the ``top`` largest of ``s + correction``
      are chosen (``correction``: a tensor, or none), and weigh in with ``s`` itself; with
      ``renormalize`` divided by the chosen ones' sum (+ 1e-20); times ``weight_scale``;
    * the last ``n_identity`` router outputs stand for experts that give their input back;
    * ``shared_inner > 0``: one more expert of that inner size (``shared.gate`` ...) that every
      token uses with weight one.

    The choice runs on the device (csrc/experts.hip), so a step launches kernels only.  For few
    tokens the chosen experts' weights are read straight from the stacked tensors, a wave a
    feature, by kernels that touch nothing else; for many tokens the picks are sorted by expert on
    the device and go to the matrix cores in tiles of up to 64 picks of one expert.  The shared
    expert goes through the framework's products.  No counterpart in
    mlx_lm/models/gpt2.py, whose feed-forward (:71-84) is dense.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    can_overwrite = True
    MERGED_UP_TO = 16  # up to this many tokens the router's and the shared expert's first products are one
    TILES_FROM = 64  # from this many tokens in a step the picks are sorted and go to the matrix cores in tiles

    def __init__(self, width, n_experts, inner, top, n_identity=0, shared_inner=0, correction=True, renormalize=False,
                 weight_scale=1.0, prefix=""):
        super().__init__(prefix)
        self.renormalize, self.weight_scale = bool(renormalize), float(weight_scale)
        if n_experts < 0 or n_identity < 0 or n_experts + n_identity <= 0:
            raise ValueError(f"{n_experts} experts and {n_identity} identity experts")
        if not 0 < top <= n_experts + n_identity:
            raise ValueError(f"{top} of {n_experts + n_identity} experts a token")
        if width % 8:
            raise ValueError(f"the feed-forward's width must be a multiple of 8, got {width}")
        if n_experts and inner <= 0:
            raise ValueError(f"the experts' inner size must be positive, got {inner}")
        self.width, self.n_experts, self.inner, self.top = width, n_experts, inner, top
        self.n_identity, self.shared_inner, self.has_correction = n_identity, int(shared_inner or 0), bool(correction)
        self.n_out = n_experts + n_identity
        self.shared_padded = (self.shared_inner + 7) // 8 * 8  # zero weights beyond: silu(0) * 0 = 0 meets zero columns
        self.overwrite = False

    def tensors(self):
        n, t = self._name, {}
        for e in range(self.n_experts):
            t[n(f"e{e}.gate")] = TensorSpec((self.inner, self.width), "matrix")
            t[n(f"e{e}.up")] = TensorSpec((self.inner, self.width), "matrix")
            t[n(f"e{e}.down")] = TensorSpec((self.width, self.inner), "matrix")
        t[n("router")] = TensorSpec((self.n_out, self.width), "matrix")
        if self.has_correction:
            t[n("correction")] = TensorSpec((self.n_out,), "vector")
        if self.shared_inner:
            t[n("shared.gate")] = TensorSpec((self.shared_inner, self.width), "matrix")
            t[n("shared.up")] = TensorSpec((self.shared_inner, self.width), "matrix")
            t[n("shared.down")] = TensorSpec((self.width, self.shared_inner), "matrix")
        return t

    def load(self, tensors):
        n = self._name
        self.w_gate = self.w_up = self.w_down = None
        if self.n_experts:
            self.w_gate = torch.stack([tensors[n(f"e{e}.gate")] for e in range(self.n_experts)]).contiguous()
            self.w_up = torch.stack([tensors[n(f"e{e}.up")] for e in range(self.n_experts)]).contiguous()
            self.w_down = torch.stack([tensors[n(f"e{e}.down")] for e in range(self.n_experts)]).contiguous()
        self.router_w = kernels.for_decode(tensors[n("router")].contiguous())
        self.first_weight = self.router_w
        self.correction = tensors[n("correction")] if self.has_correction else None
        self.shared_in = self.shared_out = None
        if self.shared_inner:
            g, u, d = tensors[n("shared.gate")], tensors[n("shared.up")], tensors[n("shared.down")]
            pad = self.shared_padded - self.shared_inner
            if pad:
                g = torch.cat([g, g.new_zeros(pad, self.width)])
                u = torch.cat([u, u.new_zeros(pad, self.width)])
                d = torch.cat([d, d.new_zeros(self.width, pad)], 1)
            self.shared_in = kernels.for_decode(torch.cat([g, u]).contiguous())
            self.shared_out = kernels.for_decode(d.contiguous())
            # for steps of few tokens: router, gate and up in one product (float32 rows)
            self.merged_in = kernels.for_decode(torch.cat([tensors[n("router")], g, u]).contiguous())

    def forward(self, ctx, x, residual):
        T = x.shape[0]
        mark = ctx.scratch_mark()
        idx = ctx.scratch((T, self.top), torch.int32)
        weight = ctx.scratch((T, self.top), torch.float32)
        accumulate = not self.overwrite
        if self.shared_inner and T <= self.MERGED_UP_TO:
            # few tokens: what a launch costs counts for more than what it computes
            zu = ctx.scratch((T, self.n_out + 2 * self.shared_padded), torch.float32)
            kernels.linear(zu, x, self.merged_in)
            act = ctx.scratch((T, self.shared_padded), ctx.dtype)
            kernels.route_and_gate(idx, weight, act, zu, self.correction, self.top, self.n_out, self.renormalize, self.weight_scale)
            kernels.linear(residual, act, self.shared_out, accumulate=accumulate)
            accumulate = True
        else:
            z = ctx.scratch((T, self.n_out), torch.float32)
            kernels.linear(z, x, self.router_w, splits=kernels.splits_alone(T))
            kernels.router_choice(idx, weight, z, self.correction, self.top, self.renormalize, self.weight_scale)
        if self.shared_inner and T > self.MERGED_UP_TO:
            gu = ctx.scratch((T, 2 * self.shared_padded), ctx.dtype)
            kernels.linear(gu, x, self.shared_in, splits=kernels.splits_alone(T))
            act = ctx.scratch((T, self.shared_padded), ctx.dtype)
            kernels.silu_mul(act, gu)
            kernels.linear(residual, act, self.shared_out, accumulate=accumulate, splits=kernels.splits_alone(T))
            accumulate = True
        if self.n_experts and T >= self.TILES_FROM and kernels.expert_tiles_takes(self.inner, self.width, x.dtype):
            kernels.expert_tiles(residual, x, self.w_gate, self.w_up, self.w_down, idx, weight, self.top, ctx.scratch,
                                 accumulate=accumulate)
        else:
            act = ctx.scratch((T * self.top, self.inner), ctx.dtype) if self.n_experts else None
            kernels.expert_rows(residual, x, self.w_gate, self.w_up, self.w_down, idx, weight, self.top, act,
                                accumulate=accumulate)
        ctx.scratch_release(mark)


register_feed_forward("gated_experts", GatedExperts)
