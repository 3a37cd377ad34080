"""Softmax attention whose scores are shaped on their way to the softmax: capped, or biased by distance."""

import math

import torch

from ..config.plan import CacheNeed
from ..ops import kernels
from .attention import CausalSelfAttention
from .base import Mixer, TensorSpec, register_mixer
from .linear_state import _matrix


def distance_bucket(n, rows, far):
    """The row of a distance table of ``rows`` rows for the distance ``n >= 0``: distances below
    half the table have a row of their own; from there on rows are spaced evenly in ``ln n`` so
    that ``far`` would reach the table's end, and everything beyond shares the last row."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


class ScoredAttention(Mixer):
    """Causal softmax attention over the paged cache with grouped key heads (query head ``h`` reads
    key head ``h // (n_heads / n_kv_heads)``), separate ``q``, ``k``, ``v``, ``o`` matrices without
    biases, keys of ``key_dim`` and values of ``value_dim`` columns a head, and no rotation.  A score
    is ``(q . k) * scale`` and then, each where asked for:

    * ``softcap``: ``softcap * tanh(score / softcap)``;
    * ``bias_rows`` (with ``bias_far``): a learned term ``rel[bucket(i - j), h]`` from the tensor
      ``rel`` ``[bias_rows, n_heads]`` is added (``distance_bucket``), after the scaling.

    ``whole_norm``: queries and keys are RMS-normed over their whole projection (all heads at once,
    before the split into heads) with plain weights ``q.norm`` and ``k.norm`` of that size.
    ``gate``: the concatenated heads are multiplied by ``sigmoid(Wg x)`` (tensor ``g``) ahead of
    the output projection.

    One product gives ``[q | k | v | g]`` as float32 rows; the norms are 32-bit and run as ``head_prepare``
    lays the heads into the next head size that the fast attention kernels take (zeros beyond a
    head's own columns), keys and values straight into their pages.  The table of the distance
    term is made once, a float for every (head, distance) up to ``bias_far`` (beyond it the last
    row holds), and the attention kernels look it up as they make a score; cap, term and gate
    ride in those kernels (``kernels.ScoreTerms``).  Scores and softmax are 32-bit.  No counterpart
    in mlx_lm/models/gpt2.py, whose attention (:44-68) has none of these.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    takes_normed_input = True  # ``x`` may be a ``kernels.NormedInput``: the first product norms the rows itself
    can_overwrite = True  # writes its output instead of adding it where ``overwrite`` is set
    step_arrays_key = CausalSelfAttention.step_arrays_key
    step_array_names = CausalSelfAttention.step_array_names
    step_arrays = staticmethod(CausalSelfAttention.step_arrays)
    length_class = staticmethod(CausalSelfAttention.length_class)

    def __init__(self, width, n_heads, key_dim, value_dim=None, n_kv_heads=None, scale=None, softcap=0.0, gate=False,
                 whole_norm=False, eps=1e-6, bias_rows=0, bias_far=0.0, max_positions=0, window=0, prefix=""):
        super().__init__(prefix)
        n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        value_dim = key_dim if value_dim is None else value_dim
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads cannot be grouped over {n_kv_heads} key heads")
        if key_dim <= 0 or value_dim <= 0 or max(key_dim, value_dim) > 256:
            raise ValueError(f"heads of {key_dim} key and {value_dim} value columns (1 to 256)")
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        if softcap < 0 or window < 0:
            raise ValueError(f"softcap {softcap} and window {window} must not be negative")
        if bias_rows and (bias_rows < 2 or bias_far <= bias_rows // 2 or max_positions <= 0):
            raise ValueError(f"a distance table of {bias_rows} rows reaching {bias_far} over {max_positions} positions")
        self.width, self.n_heads, self.n_kv_heads = width, n_heads, n_kv_heads
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.head_dim = kernels.attention_head_dim(max(key_dim, value_dim))
        self.scale = float(scale) if scale is not None else key_dim**-0.5
        self.softcap, self.has_gate, self.whole_norm, self.eps = float(softcap), bool(gate), bool(whole_norm), float(eps)
        self.bias_rows, self.bias_far, self.max_positions = int(bias_rows), float(bias_far), int(max_positions)
        self.window = int(window)
        self.q_cols, self.k_cols, self.v_cols = n_heads * key_dim, n_kv_heads * key_dim, n_kv_heads * value_dim
        self.g_cols = n_heads * value_dim if self.has_gate else 0
        self.distance_bias = None
        self.overwrite = False
        self.projection_given = False  # a pair of parallel mixers makes both mixers' projections in one product

    def cache_need(self):
        return CacheNeed(self.n_kv_heads, self.head_dim, self.window)

    def tensors(self):
        n = self._name
        t = {n("q"): TensorSpec((self.q_cols, self.width), "matrix"), n("k"): TensorSpec((self.k_cols, self.width), "matrix"),
             n("v"): TensorSpec((self.v_cols, self.width), "matrix"),
             n("o"): TensorSpec((self.width, self.n_heads * self.value_dim), "matrix")}
        if self.has_gate:
            t[n("g")] = TensorSpec((self.g_cols, self.width), "matrix")
        if self.whole_norm:
            t[n("q.norm")], t[n("k.norm")] = TensorSpec((self.q_cols,), "vector"), TensorSpec((self.k_cols,), "vector")
        if self.bias_rows:
            t[n("rel")] = TensorSpec((self.bias_rows, self.n_heads), "vector")
        return t

    def input_names(self):
        """The tensors whose rows, in this order, are the projection that ``forward`` starts with."""
        return [self._name(x) for x in ("q", "k", "v") + (("g",) if self.has_gate else ())]

    def load(self, tensors):
        n, H, hd, dv = self._name, self.n_heads, self.head_dim, self.value_dim
        if not self.projection_given:
            self.in_w = _matrix(torch.cat([tensors[x] for x in self.input_names()]))
            self.first_weight = self.in_w
        # the output projection meets heads of ``head_dim`` columns: zero columns beyond a head's values
        o = tensors[n("o")].view(self.width, H, dv)
        self.out_w = _matrix(torch.cat([o, o.new_zeros(self.width, H, hd - dv)], 2).reshape(self.width, H * hd))
        self.q_norm = tensors[n("q.norm")] if self.whole_norm else None
        self.k_norm = tensors[n("k.norm")] if self.whole_norm else None
        if self.bias_rows:
            rel = tensors[n("rel")].float().cpu()
            # a float for every (head, distance); from ``bias_far`` on the bucket is the last row's
            n_dist = max(1, min(self.max_positions, int(math.ceil(self.bias_far)) + 1))
            rows = torch.tensor([distance_bucket(d, self.bias_rows, self.bias_far) for d in range(n_dist)])
            self.distance_bias = rel[rows].t().contiguous().to(tensors[n("rel")].device)

    def forward(self, ctx, x, residual, cache, writes_cache=True, rows=None):
        """``rows``: the projection's float32 rows, where the caller has made them already."""
        T, H, G, hd, d, dv = x.shape[0], self.n_heads, self.n_kv_heads, self.head_dim, self.key_dim, self.value_dim
        mark = ctx.scratch_mark()
        qc, kc, vc = self.q_cols, self.k_cols, self.v_cols
        u = rows
        if u is None:
            u = ctx.scratch((T, qc + kc + vc + self.g_cols), torch.float32)
            kernels.linear(u, x, self.in_w, splits=kernels.splits_alone(T))
        q = ctx.scratch((T, H * hd), ctx.dtype)
        place = dict(dst_stride=hd, dst_fill=hd)
        q_norm = dict(norm_whole=qc, norm_weight=self.q_norm, eps=self.eps) if self.whole_norm else {}
        k_norm = dict(norm_whole=kc, norm_weight=self.k_norm, eps=self.eps) if self.whole_norm else {}
        calls = [(q, u, 0, H, d, dict(place, **q_norm))]
        if writes_cache:
            pages = [kernels.PagesOut(cache.kv, values, cache.block_table, ctx.token_req, ctx.positions) for values in (False, True)]
            calls.append((pages[0], u, qc, G, d, dict(place, **k_norm)))
            calls.append((pages[1], u, qc + kc, G, dv, place))
        gate = None
        if self.has_gate:
            gate = ctx.scratch((T, H * hd), ctx.dtype)
            calls.append((gate, u, qc + kc + vc, H, dv, place))
        kernels.head_prepare_many(*calls)  # (queries, gate, and keys and values straight to their pages: one launch)
        terms = None
        if gate is not None or self.softcap or self.distance_bias is not None:
            terms = kernels.ScoreTerms(gate=gate, softcap=self.softcap, distance_bias=self.distance_bias)
        att = ctx.scratch((T, H * hd), ctx.dtype)
        kernels.attend(ctx, att, q, cache, H, G, hd, self.scale, self.window, terms=terms)
        kernels.linear(residual, att, self.out_w, accumulate=not self.overwrite, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


register_mixer("scored_attention", ScoredAttention)
