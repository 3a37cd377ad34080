"""Attention whose keys and values are read out of one small latent vector per token."""

import torch

from ..config.plan import CacheNeed
from ..ops import kernels
from .attention import CausalSelfAttention
from .base import Mixer, TensorSpec, register_mixer
from .linear_state import _matrix, _padded_columns
from .rotary import rotary_table


class LatentAttention(Mixer):
    """Queries through a latent: ``cq = N(Wdq x; dq.norm)``, ``q = Wuq cq``, head by head ``[key_dim
    plain | rot_dim rotated]``.  ``Wdkv x`` gives ``kv_rank + rot_dim`` columns: the first
    ``kv_rank``, RMS-normed, are the latent ``c``; the rest, rotated, one key part shared by all
    heads.  Head ``h`` has keys ``[Wuk_h c | rotated part]`` and values ``Wuv_h c``; causal softmax
    of ``(q . k) * scale``; the head's output times ``sigmoid((Wg x)_h)``; ``Wo`` on the heads.
    Rotation: pairs ``(2i, 2i + 1)`` of the ``rot_dim`` columns by ``position * base^(-2i / rot_dim)``.
    A layer with ``own_latent=False`` has no ``Wdkv``: it reads the cache slot that another such
    layer writes (the plan points its run there), with its own ``Wuk`` and ``Wuv``.

    What a page holds is the token's ``[c | rotated part]`` once, as the key and the value of a
    single key head: since ``q_h . (Wuk_h c) = (Wuk_h^T q_h) . c`` and ``Wo_h (Wuv_h sum_j p_j c_j)``
    is linear in the summed latents, ``Wuk`` is folded into the query projection (``Wuk_h^T Wuq_h``,
    ``kv_rank`` rows a head beside the ``rot_dim`` rotated ones) and ``Wuv`` into the output
    projection (``Wo_h Wuv_h``) when the weights are loaded, in float64.  The attention is then the
    framework's paged attention with ``n_heads`` query heads over one key head of ``kv_rank +
    rot_dim`` columns (rounded up to a size that the fast attention kernels take; at most 256), whose output's first ``kv_rank`` columns a head
    are the summed latents.  One product gives ``[Wdq x | Wg x | Wdkv x]`` as float32 rows; norms and
    rotation are 32-bit (csrc/head_prepare.hip).  No counterpart in mlx_lm/models/gpt2.py.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    takes_normed_input = True  # ``x`` may be a ``kernels.NormedInput``: the first product norms the rows itself
    step_arrays_key = CausalSelfAttention.step_arrays_key
    step_array_names = CausalSelfAttention.step_array_names
    step_arrays = staticmethod(CausalSelfAttention.step_arrays)
    length_class = staticmethod(CausalSelfAttention.length_class)

    def __init__(self, width, n_heads, key_dim, rot_dim, value_dim, q_rank, kv_rank, scale, eps, rot_base=10000.0,
                 rot_scaling=None, own_latent=True, prefix=""):
        super().__init__(prefix)
        if min(n_heads, key_dim, value_dim, q_rank, kv_rank) <= 0 or rot_dim < 0 or rot_dim % 2:
            raise ValueError(f"{n_heads} heads of {key_dim} + {rot_dim} key and {value_dim} value columns, ranks {q_rank} and {kv_rank}")
        if kv_rank + rot_dim > 256:
            raise ValueError(f"a latent of {kv_rank} + {rot_dim} columns (at most 256 together)")
        self.head_dim = kernels.attention_head_dim(kv_rank + rot_dim)
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        self.width, self.n_heads, self.key_dim, self.rot_dim, self.value_dim = width, n_heads, key_dim, rot_dim, value_dim
        self.q_rank, self.kv_rank, self.scale, self.eps = q_rank, kv_rank, float(scale), float(eps)
        self.rot_base, self.rot_scaling, self.own_latent = float(rot_base), rot_scaling, bool(own_latent)
        self.latent_cols = kv_rank + rot_dim

    def cache_need(self):
        return CacheNeed(1, self.head_dim, 0)

    def tensors(self):
        n, H = self._name, self.n_heads
        t = {n("dq"): TensorSpec((self.q_rank, self.width), "matrix"), n("dq.norm"): TensorSpec((self.q_rank,), "vector"),
             n("uq"): TensorSpec((H * (self.key_dim + self.rot_dim), self.q_rank), "matrix"),
             n("uk"): TensorSpec((H * self.key_dim, self.kv_rank), "matrix"),
             n("uv"): TensorSpec((H * self.value_dim, self.kv_rank), "matrix"),
             n("g"): TensorSpec((H, self.width), "matrix"),
             n("o"): TensorSpec((self.width, H * self.value_dim), "matrix")}
        if self.own_latent:
            t[n("dkv")] = TensorSpec((self.latent_cols, self.width), "matrix")
            t[n("dkv.norm")] = TensorSpec((self.kv_rank,), "vector")
        return t

    def load(self, tensors):
        n, H, d, dr, dv, r, hd = self._name, self.n_heads, self.key_dim, self.rot_dim, self.value_dim, self.kv_rank, self.head_dim
        dq = tensors[n("dq")]
        dev, dtype = dq.device, dq.dtype
        first = [dq, tensors[n("g")]] + ([tensors[n("dkv")]] if self.own_latent else [])
        self.in_w = _matrix(torch.cat(first))
        self.first_weight = self.in_w
        self.q_norm = tensors[n("dq.norm")]
        self.c_norm = tensors[n("dkv.norm")] if self.own_latent else None
        uq = tensors[n("uq")].double().view(H, d + dr, self.q_rank)
        uk = tensors[n("uk")].double().view(H, d, r)
        uv = tensors[n("uv")].double().view(H, dv, r)
        o = tensors[n("o")].double().view(self.width, H, dv)
        # queries straight against the latent: kv_rank rows a head from Wuk_h^T Wuq_h, then the rotated rows
        q_rows = torch.cat([torch.einsum("hdr,hdq->hrq", uk, uq[:, :d]), uq[:, d:]], 1).reshape(H * (r + dr), self.q_rank)
        self.q_w = _matrix(_padded_columns(q_rows.to(dtype)))
        out = torch.zeros(self.width, H, hd, dtype=torch.float64, device=dev)
        out[:, :, :r] = torch.einsum("whv,hvr->whr", o, uv)
        self.out_w = _matrix(out.reshape(self.width, H * hd).to(dtype))
        self.inv_freq, self.rot_mult = None, 1.0
        if dr:
            self.inv_freq, self.rot_mult = rotary_table(dr, self.rot_base, self.rot_scaling, dev)

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        T, H, r, dr, hd, Q = x.shape[0], self.n_heads, self.kv_rank, self.rot_dim, self.head_dim, self.q_rank
        mark = ctx.scratch_mark()
        u = ctx.scratch((T, Q + H + (self.latent_cols if self.own_latent else 0)), torch.float32)
        kernels.linear(u, x, self.in_w, splits=kernels.splits_alone(T))
        Qp = -(-Q // 8) * 8
        cq = ctx.scratch((T, Qp), ctx.dtype)
        if Qp == Q:
            kernels.rmsnorm(cq, u, self.q_norm, self.eps)  # (a block a row; the rows' first Q columns)
        else:
            kernels.head_prepare(cq, u, 0, 1, Q, dst_stride=Qp, dst_fill=Qp, norm_dim=Q, norm_weight=self.q_norm, eps=self.eps)
        qf = ctx.scratch((T, H * (r + dr)), torch.float32)
        kernels.linear(qf, cq, self.q_w, splits=kernels.splits_alone(T))
        rot = dict(rot_off=r, rot_dims=dr, inv_freq=self.inv_freq, rot_mult=self.rot_mult, positions=ctx.positions)
        q = ctx.scratch((T, H * hd), ctx.dtype)
        calls = [(q, qf, 0, H, r + dr, dict(dst_stride=hd, dst_fill=hd, **rot))]
        if writes_cache:
            if not self.own_latent:
                raise RuntimeError("a latent-attention layer without a down-projection reads another layer's cache slot")
            # the latent goes straight to its pages, as the one key head's key and as its value
            for values in (False, True):
                pages = kernels.PagesOut(cache.kv, values, cache.block_table, ctx.token_req, ctx.positions)
                calls.append((pages, u, Q + H, 1, r + dr, dict(dst_stride=hd, dst_fill=hd, norm_dim=r, norm_weight=self.c_norm,
                                                               eps=self.eps, **rot)))
        kernels.head_prepare_many(*calls)  # (queries and the latent in one launch)
        att = ctx.scratch((T, H * hd), ctx.dtype)
        kernels.attend(ctx, att, q, cache, H, 1, hd, self.scale)
        kernels.head_gate(att, hd, H, u[:, Q:Q + H])
        kernels.linear(residual, att, self.out_w, accumulate=True, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


register_mixer("latent_attention", LatentAttention)
