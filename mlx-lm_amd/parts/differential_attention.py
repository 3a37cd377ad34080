"""Differential attention: two softmax maps over the same values, one taken off the other."""

import torch

from ..config.plan import CacheNeed
from ..ops import kernels
from .attention import CausalSelfAttention
from .base import Mixer, TensorSpec, register_mixer
from .convolution import ShortConvolution
from .linear_state import _matrix, _padded_columns, _rows_for
from .rotary import rotary_table


class DifferentialAttention(Mixer):
    """Every query head has two maps, each a causal softmax attention of its own with queries and
    keys of ``key_dim`` columns, over the same values of ``value_dim``:

        ``o = a1 - lambda a2``,  ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff``

    then ``o`` is divided by its root mean square over the head (no weight) and multiplied by
    ``1 - diff``; ``Wo`` on the concatenated heads.  ``q``, ``k``, ``v`` come from three matrices
    with biases, ``q`` laid out ``[head][map][key_dim]`` and ``k`` ``[key head][map][key_dim]``;
    query head ``h`` reads key head ``h // (n_heads / n_kv_heads)``.  Between projection and
    scores: an optional short causal convolution on every channel (``taps``; its last inputs are
    per-request state, ``ShortConvolution``), an RMS norm of every map of every head with a weight
    shared by all (``q.norm``, ``k.norm``), and a rotation of the first ``rot_dims`` columns of
    every map, pairs ``(2i, 2i + 1)``, optionally with frequencies interpolated by wavelength
    (``rot_scaling``, ``parts/rotary.py``).

    On the GPU the two maps are two heads of the framework's paged attention: ``2 n_heads`` query
    heads over ``2 n_kv_heads`` key heads of ``head_dim = max(key_dim, value_dim)`` rounded up to
    a size that the fast attention kernels take (``kernels.attention_head_dim``), ordered ``[key head][map][query head of the group]`` so that the kernels' grouping
    of query heads over key heads pairs map with map; a key head's values are written beside both
    of its maps' keys.  One product gives ``[q | k | v]`` as float32 rows; convolution, norm and
    rotation are 32-bit (csrc/head_prepare.hip) and write the compute dtype; the attention kernels
    are the built-in part's (``kernels.attend``); ``diff_combine`` joins the maps.  No counterpart
    in mlx_lm/models/gpt2.py, whose attention (:44-68) has one map.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    takes_normed_input = True  # ``x`` may be a ``kernels.NormedInput``: the first product norms the rows itself
    step_arrays_key = CausalSelfAttention.step_arrays_key
    step_array_names = CausalSelfAttention.step_array_names
    step_arrays = staticmethod(CausalSelfAttention.step_arrays)
    length_class = staticmethod(CausalSelfAttention.length_class)

    def __init__(self, width, n_heads, key_dim, value_dim, scale, diff, eps, n_kv_heads=None, taps=0, rot_dims=0,
                 rot_base=10000.0, rot_scaling=None, prefix=""):
        super().__init__(prefix)
        n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads cannot be grouped over {n_kv_heads} key heads")
        if key_dim <= 0 or value_dim <= 0 or max(key_dim, value_dim) > 256:
            raise ValueError(f"keys of {key_dim} and values of {value_dim} columns a head (at most 256)")
        self.head_dim = kernels.attention_head_dim(max(key_dim, value_dim))
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        if rot_dims % 2 or not 0 <= rot_dims <= key_dim:
            raise ValueError(f"{rot_dims} turning columns of {key_dim}: an even number within a map")
        self.width, self.n_heads, self.n_kv_heads = width, n_heads, n_kv_heads
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.diff, self.eps = float(scale), float(diff), float(eps)
        self.rot_dims, self.rot_base, self.rot_scaling = int(rot_dims), float(rot_base), rot_scaling
        self.q_cols, self.k_cols, self.v_cols = 2 * n_heads * key_dim, 2 * n_kv_heads * key_dim, n_kv_heads * value_dim
        self.taps = int(taps or 0)
        self.conv = None
        if self.taps >= 1:
            self.conv = ShortConvolution((self.q_cols, self.k_cols, self.v_cols), self.taps, ("q.conv", "k.conv", "v.conv"),
                                         prefix=prefix)
        self.wants_state = self.conv is not None and self.conv.state_floats > 0

    def sub_parts(self):
        return (self.conv,) if self.conv is not None else ()

    def cache_need(self):
        return CacheNeed(2 * self.n_kv_heads, self.head_dim, 0)

    def state_need(self):
        return self.conv.state_need() if self.conv is not None else None

    def tensors(self):
        n, d = self._name, self.key_dim
        t = {n("q"): TensorSpec((self.q_cols, self.width), "matrix"), n("q.b"): TensorSpec((self.q_cols,), "vector"),
             n("k"): TensorSpec((self.k_cols, self.width), "matrix"), n("k.b"): TensorSpec((self.k_cols,), "vector"),
             n("v"): TensorSpec((self.v_cols, self.width), "matrix"), n("v.b"): TensorSpec((self.v_cols,), "vector"),
             n("q.norm"): TensorSpec((d,), "vector"), n("k.norm"): TensorSpec((d,), "vector"),
             n("o"): TensorSpec((self.width, self.n_heads * self.value_dim), "matrix")}
        for name in ("lq1", "lk1", "lq2", "lk2"):
            t[n(name)] = TensorSpec((d,), "vector")
        return t

    def load(self, tensors):
        n = self._name
        dev = tensors[n("q")].device
        self.in_w = _matrix(torch.cat([tensors[n(x)] for x in ("q", "k", "v")]))
        self.in_b = torch.cat([tensors[n(x + ".b")] for x in ("q", "k", "v")]).contiguous()
        self.out_w = _matrix(_padded_columns(tensors[n("o")]))
        self.first_weight = self.in_w
        self.q_norm, self.k_norm = tensors[n("q.norm")], tensors[n("k.norm")]
        lam = [(tensors[n("lq" + i)].double() * tensors[n("lk" + i)].double()).sum().exp().item() for i in "12"]
        self.lam = float(torch.tensor(lam[0] - lam[1] + self.diff, dtype=torch.float32))
        self.inv_freq, self.rot_mult = None, 1.0
        if self.rot_dims:
            self.inv_freq, self.rot_mult = rotary_table(self.rot_dims, self.rot_base, self.rot_scaling, dev)
        # where a head of the checkpoint's order goes among the attention kernels' heads
        H, G = self.n_heads, self.n_kv_heads
        r = H // G
        place = lambda h, m: (h // r) * 2 * r + m * r + h % r  # noqa: E731
        ints = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)  # noqa: E731
        self.q_place = ints([place(h, m) for h in range(H) for m in range(2)])
        self.v_place = ints([2 * g for g in range(G)] + [2 * g + 1 for g in range(G)])
        self.first, self.second = ints([place(h, 0) for h in range(H)]), ints([place(h, 1) for h in range(H)])

    def forward(self, ctx, x, residual, cache, writes_cache=True, state=None):
        T, H2, G2, hd, d = x.shape[0], 2 * self.n_heads, 2 * self.n_kv_heads, self.head_dim, self.key_dim
        mark = ctx.scratch_mark()
        u = ctx.scratch((T, self.q_cols + self.k_cols + self.v_cols), torch.float32)
        kernels.linear(u, x, self.in_w, bias=self.in_b, splits=kernels.splits_alone(T))
        conv = self.conv.ahead(ctx, state.state if state is not None else None) if self.conv is not None else None
        rot = dict(rot_dims=self.rot_dims, inv_freq=self.inv_freq, rot_mult=self.rot_mult, positions=ctx.positions, conv=conv)
        q = ctx.scratch((T, H2 * hd), ctx.dtype)
        calls = [(q, u, 0, H2, d, dict(dst_stride=hd, dst_fill=hd, norm_dim=d, norm_weight=self.q_norm, eps=self.eps,
                                       dst_head=self.q_place, **rot))]
        if writes_cache:
            # keys and values go straight to their pages
            pages = [kernels.PagesOut(cache.kv, values, cache.block_table, ctx.token_req, ctx.positions) for values in (False, True)]
            calls.append((pages[0], u, self.q_cols, G2, d, dict(dst_stride=hd, dst_fill=hd, norm_dim=d, norm_weight=self.k_norm,
                                                                eps=self.eps, **rot)))
            calls.append((pages[1], u, self.q_cols + self.k_cols, self.n_kv_heads, self.value_dim,
                          dict(dst_stride=hd, dst_fill=hd, dst_head=self.v_place, copies=2, conv=conv)))
        kernels.head_prepare_many(*calls)  # (convolution, norm, rotation, queries and the cache's keys and values: one launch)
        if self.conv is not None:
            self.conv.keep_inputs(ctx, u, state.state if state is not None else None)
        att = ctx.scratch((T, H2 * hd), ctx.dtype)
        kernels.attend(ctx, att, q, cache, H2, G2, hd, self.scale)
        width = self.n_heads * self.value_dim
        out, whole = _rows_for(ctx, T, width, -(-width // 8) * 8)
        kernels.diff_combine(out, att, hd, self.first, self.second, self.lam, 1.0 - self.diff, self.eps, self.value_dim)
        kernels.linear(residual, out if whole is None else whole, self.out_w, accumulate=True, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


register_mixer("differential_attention", DifferentialAttention)
