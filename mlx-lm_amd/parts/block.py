"""Arrangements of norms, mixer and feed-forward in a layer."""

import ctypes

from ..config.plan import StateNeed
from ..ops import native
from .base import Block, TensorSpec, register_block


class PreNormBlock(Block):
    """``h += mixer(norm1(h)); h += ffn(norm2(h))``.

    mlx_lm/models/gpt2.py:98-108.  The two sums happen inside the mixer's and
    the feed-forward's last matrix product, in float32.  Such a product may
    leave its sum into ``h`` pending (``ctx.pending``); the norm that reads
    ``h`` next adds it (``handles_pending``).  A mixer whose kernels leave CUs
    idle may have them read the weights that come after its own (the
    feed-forward's first).  The arrangement itself runs in the native host
    (``PreNormBlock`` in csrc/engine.hip); its parts may be native or Python.
    The feed-forward, with its norm, may be absent.  A mixer that keeps per-request state beside
    its pages (``wants_state`` and ``state_need()``) gets the run's state slot too.
    """

    PARTS = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}
    OPTIONAL = ("ffn_norm", "ffn")
    handles_pending = True

    def __init__(self, mixer_norm, mixer, ffn_norm=None, ffn=None, prefix=""):
        super().__init__(prefix)
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a pre-norm layer has a feed-forward and its norm, or neither")
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.parts())

    def parts(self):
        out = []

        def walk(part):
            if part is None:
                return
            out.append(part)
            for sub in getattr(part, "sub_parts", lambda: ())():
                walk(sub)

        for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn):
            walk(p)
        return tuple(out)

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        if getattr(self.mixer, "wants_state", False) and hasattr(self.mixer, "state_need"):
            return self.mixer.state_need()
        return None

    def make_native(self):
        return native.made(native.lib().eng_make_pre_norm_block(
            self.mixer_norm.native(), self.mixer.native(), self.ffn_norm.native() if self.ffn_norm is not None else None,
            self.ffn.native() if self.ffn is not None else None), "pre-norm block")

    def forward(self, ctx, h, cache, writes_cache=True, state=None):
        hm = native.mat(h)
        with ctx.enter():
            rc = native.lib().eng_block_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(hm), cache.slot,
                                                int(bool(writes_cache)), state.slot if state is not None else -1)
        native.check(rc, "pre-norm block")
        return h


class PostNormBlock(Block):
    """``h = norm1(alpha h + s1 * mixer(shift(h))); h = norm2(alpha h + s2 * ffn(h))``: the norms
    come after the sums, and the sublayers read the stream itself.

    ``layer_scale``: the sublayers' outputs are multiplied per column by the tensors ``ls1`` and
    ``ls2`` before they enter the sums.  ``token_shift``: the mixer reads ``h_t + (h_{t-1} - h_t) *
    shift`` per column (zeros before a request's first token); the row before a portion's first
    is per-request state that the arrangement keeps, one slot for each run of the layer
    (``state_need``).  The feed-forward (with its norm) may be absent.  Both norms are RMS norms
    (``rmsnorm`` parts give weight and eps); sums, scales, shift and norms run in float32 in the
    arrangement's own kernels (csrc/post_norm_block.hip).  No counterpart in
    mlx_lm/models/gpt2.py, whose blocks norm before their sublayers (:98-108).
    """

    PARTS = {"mixer": "mixer", "mixer_norm": "norm", "ffn": "feed_forward", "ffn_norm": "norm"}
    OPTIONAL = ("ffn", "ffn_norm")
    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, mixer, mixer_norm, ffn=None, ffn_norm=None, alpha=1.0, layer_scale=False, token_shift=False,
                 scale_names=("ls1", "ls2"), shift_name="shift", prefix=""):
        super().__init__(prefix)
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a post-norm layer has a feed-forward and its norm, or neither")
        for norm in (mixer_norm, ffn_norm):
            if norm is not None and not (hasattr(norm, "weight") and hasattr(norm, "eps") and not hasattr(norm, "bias")):
                raise ValueError(f"the post-norm arrangement fuses RMS norms, not a {type(norm).__name__}")
        if ffn_norm is not None and (ffn_norm.eps != mixer_norm.eps or ffn_norm.width != mixer_norm.width):
            raise ValueError("the two norms of a post-norm layer share width and eps")
        self.mixer, self.mixer_norm, self.ffn, self.ffn_norm = mixer, mixer_norm, ffn, ffn_norm
        self.width, self.alpha = mixer_norm.width, float(alpha)
        self.layer_scale, self.token_shift = bool(layer_scale), bool(token_shift)
        self.scale_names, self.shift_name = tuple(self._name(n) for n in scale_names), self._name(shift_name)
        self.scale1 = self.scale2 = self.shift = None

    def parts(self):
        # (the arrangement owns tensors itself, so it is one of its own parts)
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self) if p is not None)

    def tensors(self):
        t = {}
        if self.layer_scale:
            t[self.scale_names[0]] = TensorSpec((self.width,), "vector")
            if self.ffn is not None:
                t[self.scale_names[1]] = TensorSpec((self.width,), "vector")
        if self.token_shift:
            t[self.shift_name] = TensorSpec((self.width,), "vector")
        return t

    def load(self, tensors):
        if self.layer_scale:
            self.scale1 = tensors[self.scale_names[0]]
            self.scale2 = tensors[self.scale_names[1]] if self.ffn is not None else None
        if self.token_shift:
            self.shift = tensors[self.shift_name]

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return StateNeed((self.width,), "float32") if self.token_shift else None

    def make_native(self):
        P, F = ctypes.c_void_p, ctypes.c_float
        L = native.part_library("post_norm_block", {"make_post_norm_block": [P, P, ctypes.c_int, F, F, P, P, P, P, P]})
        return native.made(L.make_post_norm_block(
            native.host(), self.mixer.native(), self.ffn.native() if self.ffn is not None else None, self.width,
            self.alpha, self.mixer_norm.eps, native.ptr(self.mixer_norm.weight),
            native.ptr(self.ffn_norm.weight) if self.ffn_norm is not None else None, native.ptr(self.scale1),
            native.ptr(self.scale2), native.ptr(self.shift)), "post-norm block")

    def forward(self, ctx, h, cache, writes_cache=True, state=None):
        """``state``: the ``CacheView`` of the run's state slot (with ``token_shift``)."""
        hm = native.mat(h)
        with ctx.enter():
            rc = native.lib().eng_block_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(hm), cache.slot,
                                                int(bool(writes_cache)), state.slot if state is not None else -1)
        native.check(rc, "post-norm block")
        return h


class SandwichBlock(Block):
    """``h += m * post1(mixer(pre1(h))); h += m * post2(ffn(pre2(h)))``: every sublayer has a norm
    ahead of it and one behind it, and its normed output enters the stream times ``residual_mult``.

    The four norms are LayerNorms with a weight and no bias (``layernorm`` parts give weight and
    eps).  The sublayers write their outputs as float32 rows (a part that can only add gets rows
    of zeros); the norm behind a sublayer, the scaled sum into the float32 stream and the norm
    ahead of the next sublayer are one kernel (csrc/sandwich_block.hip).  The feed-forward, with
    its two norms, may be absent.  A mixer that keeps pages and per-request state at once
    (``wants_state``) gets the run's state slot beside its cache slot.  No counterpart in
    mlx_lm/models/gpt2.py, whose blocks norm ahead of their sublayers only (:98-108).
    """

    PARTS = {"mixer_norm": "norm", "mixer": "mixer", "mixer_post_norm": "norm", "ffn_norm": "norm",
             "ffn": "feed_forward", "ffn_post_norm": "norm"}
    OPTIONAL = ("ffn_norm", "ffn", "ffn_post_norm")

    def __init__(self, mixer_norm, mixer, mixer_post_norm, ffn_norm=None, ffn=None, ffn_post_norm=None,
                 residual_mult=1.0, prefix=""):
        super().__init__(prefix)
        if len({ffn is None, ffn_norm is None, ffn_post_norm is None}) != 1:
            raise ValueError("a layer has a feed-forward and its two norms, or none of the three")
        norms = [n for n in (mixer_norm, mixer_post_norm, ffn_norm, ffn_post_norm) if n is not None]
        for n in norms:
            if not (hasattr(n, "weight") and hasattr(n, "eps")) or getattr(n, "has_bias", True):
                raise ValueError(f"this arrangement fuses LayerNorms without a bias, not a {type(n).__name__}")
            if n.eps != norms[0].eps or n.width != norms[0].width:
                raise ValueError("the norms of a layer share width and eps")
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.ffn_norm, self.ffn, self.ffn_post_norm = ffn_norm, ffn, ffn_post_norm
        self.width, self.eps, self.residual_mult = norms[0].width, norms[0].eps, float(residual_mult)
        for part in (mixer, ffn):
            if part is not None and getattr(part, "can_overwrite", False) and hasattr(part, "overwrite"):
                part.overwrite = True
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.parts())

    def parts(self):
        out = []

        def walk(part):
            if part is None:
                return
            out.append(part)
            for sub in getattr(part, "sub_parts", lambda: ())():
                walk(sub)

        for p in (self.mixer_norm, self.mixer, self.mixer_post_norm, self.ffn_norm, self.ffn, self.ffn_post_norm):
            walk(p)
        return tuple(out)

    def cache_need(self):
        return self.mixer.cache_need()

    def state_need(self):
        return self.mixer.state_need() if hasattr(self.mixer, "state_need") else None

    def forward(self, ctx, h, cache, writes_cache=True, state=None):
        import torch

        from ..ops import kernels

        T = h.shape[0]
        mark = ctx.scratch_mark()
        x = ctx.scratch((T, self.width), ctx.dtype)
        kernels.layernorm(x, h, self.mixer_norm.weight, None, self.eps)
        y = ctx.scratch((T, self.width), torch.float32)
        if not getattr(self.mixer, "overwrite", False):
            y.zero_()
        if getattr(self.mixer, "wants_state", False):
            self.mixer.forward(ctx, x, y, cache, writes_cache, state=state)
        else:
            self.mixer.forward(ctx, x, y, cache, writes_cache)
        if self.ffn is None:
            kernels.add_normed(h, y, self.mixer_post_norm.weight, self.residual_mult, self.eps)
        else:
            kernels.add_normed(h, y, self.mixer_post_norm.weight, self.residual_mult, self.eps, self.ffn_norm.weight, x)
            if not getattr(self.ffn, "overwrite", False):
                y.zero_()
            self.ffn.forward(ctx, x, y)
            kernels.add_normed(h, y, self.ffn_post_norm.weight, self.residual_mult, self.eps)
        ctx.scratch_release(mark)
        return h


class SharedNormBlock(Block):
    """``y = h + mixer(u + conv(u)) + ffn(u)`` with ``u = norm(h)``: one norm, which both sublayers
    read, and their outputs enter the stream together.  Two options around it:

    * ``input_taps``: what the mixer reads passes a causal convolution over time on each channel
      first and is added to itself, ``u_t + sum_j w[:, j] u_(t - taps + 1 + j)`` (tensor
      ``input_conv_name``, ``[width, taps]``, no bias, zeros before a request's start); the
      feed-forward reads ``u`` as it is.  The last ``taps - 1`` normed rows are the request's state.
    * ``depth``: the stream that leaves the layer is a weighted sum over depth, ``h <- sum_(j <=
      depth + 1) a[j] Y_j`` with ``Y_0`` the stream as the first layer found it, ``Y_(i+1)`` the
      ``y`` of the layer with ``depth = i``, and ``a`` the tensor ``depth_name`` (``depth + 2``
      values).  The layers of a step share the ``Y`` through ``ctx.shared`` (``depth_total``
      layers: the one with ``depth = 0`` takes the memory, the sublayers add straight into ``Y``).

    The norm is an RMS norm (an ``rmsnorm`` part gives weight and eps).  Norm, convolution, the
    sums and the weighted sum are 32-bit (csrc/parallel_block.hip).  The
    run's state slot holds the convolution's inputs and, behind them, what a mixer that keeps
    state beside its pages (``wants_state``) asks for.  No counterpart in mlx_lm/models/gpt2.py,
    whose blocks have a norm for each sublayer and run them in turn (:98-108).
    """

    PARTS = {"norm": "norm", "mixer": "mixer", "ffn": "feed_forward"}
    OPTIONAL = ("ffn",)

    def __init__(self, norm, mixer, ffn=None, input_taps=0, input_conv_name="canon1", depth=None, depth_total=0,
                 depth_name="dwa", prefix=""):
        from .convolution import ShortConvolution

        super().__init__(prefix)
        if not (hasattr(norm, "weight") and hasattr(norm, "eps")) or hasattr(norm, "bias"):
            raise ValueError(f"this arrangement fuses an RMS norm, not a {type(norm).__name__}")
        self.norm, self.mixer, self.ffn = norm, mixer, ffn
        self.width, self.eps = norm.width, norm.eps
        if self.width % 8:
            raise ValueError(f"width {self.width} must be a multiple of 8")
        # (the part holds the weights and knows the state's layout; the kernels are this arrangement's own)
        self.input_conv = ShortConvolution((self.width,), int(input_taps), (input_conv_name,), prefix=prefix) if input_taps else None
        if depth is not None and not 0 <= depth < depth_total:
            raise ValueError(f"depth {depth} of {depth_total} layers")
        self.depth, self.depth_total, self.depth_name = depth, int(depth_total), self._name(depth_name)
        self.depth_w = None
        self.conv_floats = self.input_conv.state_floats if self.input_conv is not None else 0
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.parts() if p is not self)

    def parts(self):
        out = []

        def walk(part):
            if part is None:
                return
            out.append(part)
            for sub in getattr(part, "sub_parts", lambda: ())():
                walk(sub)

        for p in (self.norm, self.input_conv, self.mixer, self.ffn):
            walk(p)
        return tuple(out) + (self,)  # (the arrangement owns a tensor itself, so it is one of its own parts)

    def tensors(self):
        return {self.depth_name: TensorSpec((self.depth + 2,), "vector")} if self.depth is not None else {}

    def load(self, tensors):
        if self.depth is not None:
            self.depth_w = tensors[self.depth_name].contiguous()

    def cache_need(self):
        return self.mixer.cache_need()

    def _mixer_state_need(self):
        if getattr(self.mixer, "wants_state", False) and hasattr(self.mixer, "state_need"):
            return self.mixer.state_need()
        return None

    def state_need(self):
        need, floats = self._mixer_state_need(), self.conv_floats
        if need is not None:
            if need.dtype != "float32" or len(need.shape) != 1:
                raise ValueError("a mixer's state beside its pages is a row of float32")
            floats += need.shape[0]
        return StateNeed((floats,), "float32") if floats else None

    def forward(self, ctx, h, cache, writes_cache=True, state=None):
        import torch

        from ..engine.context import CacheView
        from ..ops import kernels

        T, W = h.shape
        kept = target = None
        if self.depth is not None:
            if self.depth == 0:
                # every layer's result of this step, the stream as it came first: kept to the step's end
                ctx.shared["depth_results"] = ctx.scratch((self.depth_total + 1, T, W), torch.float32)
            kept = ctx.shared["depth_results"]
            target = kept[self.depth + 1]
        mark = ctx.scratch_mark()
        u = ctx.scratch((T, W), ctx.dtype)
        um, u32, canon, conv = u, None, None, self.input_conv
        if conv is not None:
            um = ctx.scratch((T, W), ctx.dtype)
            rows = state.state if conv.state_floats else conv.no_state
            canon = kernels.InputConvolution(conv.weight, rows, 0, ctx.token_req, ctx.array("sequences.starts"), ctx.slot_ids, um)
        # a step in which every request brings one token: norm, convolution and the state's move are one kernel
        single = canon is not None and ctx.array("sequences.longest") == 1 and W <= kernels.CANON_FUSED_MAX_WIDTH
        if canon is not None and not single:
            u32 = ctx.scratch((T, W), torch.float32)
        # the norm; the stream itself goes where the sublayers add to it (and, first of all, to Y_0)
        kernels.norm_fanout(u, h, self.norm.weight, self.eps, out32=u32, copy_a=target,
                            copy_b=kept[0] if self.depth == 0 else None, canon=canon if single else None)
        if canon is not None and not single:
            kernels.canon_rows(u32, canon)
            if conv.state_floats:
                kernels.conv_state_update(u32, 0, conv.taps, W, rows, 0, ctx.array("sequences.starts"), ctx.array("sequences.lens"),
                                          ctx.slot_ids, ctx.n_requests)
        into = target if target is not None else h
        if self._mixer_state_need() is not None:
            self.mixer.forward(ctx, um, into, cache, writes_cache,
                               state=CacheView(state.slot, state=state.state, offset=self.conv_floats))
        else:
            self.mixer.forward(ctx, um, into, cache, writes_cache)
        if self.ffn is not None:
            self.ffn.forward(ctx, u, into)
        ctx.scratch_release(mark)
        if kept is not None:
            kernels.depth_average(h, kept, self.depth_w, self.depth + 2)
        return h


register_block("pre_norm", PreNormBlock)
register_block("shared_norm", SharedNormBlock)
register_block("sandwich", SandwichBlock)
register_block("post_norm", PostNormBlock)
