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


register_block("pre_norm", PreNormBlock)
register_block("sandwich", SandwichBlock)
register_block("post_norm", PostNormBlock)
