"""Mixers whose memory of a sequence is a decaying matrix per head, kept per request between steps."""

import torch

from ..config.plan import StateNeed
from ..ops import kernels
from .base import Mixer, TensorSpec, register_mixer


class _SequenceArrays:
    """The step arrays that a scan over each request's own tokens needs: where a request's tokens
    start in the flat batch and how many they are (its state row is ``ctx.slot_ids``)."""

    step_arrays_key = "sequences"
    step_array_names = ("starts", "lens", "longest", "span_req", "span_start", "span_first", "n_spans")
    CHUNKS_FROM = 8  # from this many tokens of one request in a step, the kernel that takes chunks
    SPAN = 64  # tokens of a span; from two spans of one request on, spans run side by side

    @staticmethod
    def step_arrays(batch):
        span = _SequenceArrays.SPAN
        span_req, span_start, span_first = [], [], []
        for r, n in enumerate(batch.q_lens):
            span_first.append(len(span_req))
            for lo in range(0, n, span):
                span_req.append(r)
                span_start.append(lo)
        return {"starts": list(batch.q_starts), "lens": list(batch.q_lens), "longest": max(batch.q_lens, default=0),
                "span_req": span_req, "span_start": span_start, "span_first": span_first, "n_spans": len(span_req)}

    def _chunked(self, ctx):
        return ctx.array("sequences.longest") >= self.CHUNKS_FROM

    def _spans(self, ctx):
        if ctx.array("sequences.longest") < 2 * self.SPAN:
            return None
        return (self.SPAN, ctx.array("sequences.n_spans"), ctx.array("sequences.span_req"), ctx.array("sequences.span_start"),
                ctx.array("sequences.span_first"), ctx.scratch)


def _matrix(w):
    return kernels.for_decode(w.contiguous())


def _padded_columns(w, multiple=8):
    """``w`` ``[N, K]`` with zero columns up to the next multiple of ``multiple`` (what a product's
    inner size has to be); the rows that meet them carry zeros in those columns."""
    pad = -w.shape[1] % multiple
    return torch.cat([w, w.new_zeros(w.shape[0], pad)], 1) if pad else w


def _rows_for(ctx, n_rows, width, padded):
    """Rows of ``width`` columns for a product whose inner size is ``padded``: a view of zeroed wider
    rows where the two differ."""
    if padded == width:
        return ctx.scratch((n_rows, width), ctx.dtype), None
    whole = ctx.scratch((n_rows, padded), ctx.dtype)
    whole.zero_()
    return whole[:, :width], whole


class Retention(_SequenceArrays, Mixer):
    """Linear attention with a fixed decay per head and neither softmax nor denominator:

        ``S_t = decay_h S_(t-1) + k_t v_t^T``,   ``o_t = S_t^T q_t``

    with ``q = Wq x``, ``k = Wk x`` (``n_heads x key_dim``), ``v = Wv x`` (``n_heads x value_dim``).
    Queries and keys turn with the position on their first ``rot_dims`` columns (column ``i`` with
    column ``i + rot_dims / 2`` by ``position * rot_base^(-2i / rot_dims)``); keys are then
    multiplied by ``key_dim^(-1/2)`` (``key_scale``).  Each head's ``o`` is divided by its root
    mean square (``eps``), the heads are multiplied by ``silu(Wg x)`` and projected by ``Wo``.
    ``S`` (``key_dim x value_dim`` a head, float32, zero at a request's start) is the request's
    state.  One product gives ``[q | k | v | g]`` as float32 rows; angles, the recurrence, the
    norm and the gate are 32-bit (csrc/linear_state.hip).  No counterpart in
    mlx_lm/models/gpt2.py.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    can_overwrite = True  # writes its output instead of adding it where ``overwrite`` is set

    def __init__(self, width, n_heads, key_dim, value_dim, decay, eps, rot_dims=0, rot_base=10000.0, key_scale=None,
                 names=("q", "k", "v", "g", "o"), prefix=""):
        super().__init__(prefix)
        if n_heads <= 0 or key_dim <= 0 or not 0 < value_dim <= 256:
            raise ValueError(f"{n_heads} heads of keys {key_dim} and values {value_dim} (values at most 256)")
        if len(decay) != n_heads:
            raise ValueError(f"{len(decay)} decays for {n_heads} heads")
        if rot_dims % 2 or not 0 <= rot_dims <= key_dim:
            raise ValueError(f"{rot_dims} turning columns of {key_dim}: an even number within the head")
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        self.width, self.n_heads, self.key_dim, self.value_dim = width, n_heads, key_dim, value_dim
        self.decay_values, self.eps = [float(d) for d in decay], float(eps)
        self.rot_dims, self.rot_base = int(rot_dims), float(rot_base)
        self.key_scale = float(key_scale) if key_scale is not None else key_dim**-0.5
        self.qk_width, self.v_width = n_heads * key_dim, n_heads * value_dim
        self.names = dict(zip(("q", "k", "v", "g", "o"), (self._name(n) for n in names)))
        self.overwrite = False
        self.in_w = self.out_w = self.decay = self.inv_freq = None

    def cache_need(self):
        return StateNeed((self.n_heads * self.key_dim * self.value_dim,), "float32")

    def tensors(self):
        n = self.names
        return {n["q"]: TensorSpec((self.qk_width, self.width), "matrix"),
                n["k"]: TensorSpec((self.qk_width, self.width), "matrix"),
                n["v"]: TensorSpec((self.v_width, self.width), "matrix"),
                n["g"]: TensorSpec((self.v_width, self.width), "matrix"),
                n["o"]: TensorSpec((self.width, self.v_width), "matrix")}

    def load(self, tensors):
        n = self.names
        dev = tensors[n["q"]].device
        self.in_w = _matrix(torch.cat([tensors[n[x]] for x in ("q", "k", "v", "g")]))
        self.out_w = _matrix(_padded_columns(tensors[n["o"]]))
        self.first_weight = self.in_w
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=dev)
        half = self.rot_dims // 2
        if half:
            i = torch.arange(half, dtype=torch.float64)
            self.inv_freq = torch.pow(torch.tensor(self.rot_base, dtype=torch.float64), -2.0 * i / self.rot_dims).float().to(dev)

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        T = x.shape[0]
        mark = ctx.scratch_mark()
        u = ctx.scratch((T, 2 * self.qk_width + 2 * self.v_width), torch.float32)
        kernels.linear(u, x, self.in_w, splits=kernels.splits_alone(T))
        a, b = self.qk_width, 2 * self.qk_width
        out, whole = _rows_for(ctx, T, self.v_width, -(-self.v_width // 8) * 8)
        kernels.state_scan(out, u[:, :a], u[:, a:b], u[:, b:b + self.v_width], cache.state, 0,
                           ctx.array("sequences.starts"), ctx.array("sequences.lens"), ctx.slot_ids, ctx.n_requests,
                           self.n_heads, self.n_heads, self.key_dim, self.value_dim, decay=self.decay,
                           k_mult=self.key_scale, rot_dims=self.rot_dims, inv_freq=self.inv_freq,
                           positions=ctx.positions, unit_rms=True, eps=self.eps, gate=u[:, b + self.v_width:],
                           chunked=self._chunked(ctx), spans=self._spans(ctx))
        kernels.linear(residual, out if whole is None else whole, self.out_w, accumulate=not self.overwrite, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


class GatedLinearAttention(_SequenceArrays, Mixer):
    """Linear attention whose state decays by a gate of its own for every key channel:

        ``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``,   ``o_t = S_t^T q_t``

    with ``q = Wq x * key_dim^(-1/2)``, ``k = Wk x`` (``n_heads x key_dim``), ``v = Wv x`` (``n_heads x
    value_dim``) and ``alpha = sigmoid(z)^(1 / tau)``, ``z = Wa2 (Wa1 x) + b`` through a narrow
    middle, laid out like the keys.  Each head's ``o`` is RMS-normed over ``value_dim`` with one
    weight for all heads, the heads are multiplied by ``silu(Wg x)`` and projected by ``Wo``.
    ``S`` (``key_dim x value_dim`` a head, float32, zero at a request's start) is the request's
    state.  One product gives ``[q | k | v | g | z]`` as float32 rows (``Wa2 Wa1`` is multiplied
    out when the weights are loaded: one product and no launches for the middle, for ``key_dim *
    n_heads`` more rows of weights); the
    logarithm of the decay (``log sigmoid(z) / tau``), the recurrence, the norm and the gate are
    32-bit (csrc/linear_state.hip; the factor of the queries rides on the keys, which gives the
    same outputs).  No counterpart in mlx_lm/models/gpt2.py.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    takes_normed_input = True  # ``x`` may be a ``kernels.NormedInput``: the first product norms the rows itself

    def __init__(self, width, n_heads, key_dim, value_dim, tau, eps, decay_rank, prefix=""):
        super().__init__(prefix)
        if n_heads <= 0 or key_dim <= 0 or not 0 < value_dim <= 256 or decay_rank <= 0:
            raise ValueError(f"{n_heads} heads of keys {key_dim} and values {value_dim} (values at most 256), a middle of {decay_rank}")
        if tau <= 0:
            raise ValueError(f"tau must be positive, got {tau}")
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        self.width, self.n_heads, self.key_dim, self.value_dim = width, n_heads, key_dim, value_dim
        self.tau, self.eps, self.decay_rank = float(tau), float(eps), int(decay_rank)
        self.qk_width, self.v_width = n_heads * key_dim, n_heads * value_dim

    def cache_need(self):
        return StateNeed((self.n_heads * self.key_dim * self.value_dim,), "float32")

    def tensors(self):
        n = self._name
        return {n("q"): TensorSpec((self.qk_width, self.width), "matrix"),
                n("k"): TensorSpec((self.qk_width, self.width), "matrix"),
                n("v"): TensorSpec((self.v_width, self.width), "matrix"),
                n("g"): TensorSpec((self.v_width, self.width), "matrix"),
                n("o"): TensorSpec((self.width, self.v_width), "matrix"),
                n("norm"): TensorSpec((self.value_dim,), "vector"),
                n("a1"): TensorSpec((self.decay_rank, self.width), "matrix"),
                n("a2"): TensorSpec((self.qk_width, self.decay_rank), "matrix"),
                n("a2.b"): TensorSpec((self.qk_width,), "vector")}

    def load(self, tensors):
        n = self._name
        a1, a2 = tensors[n("a1")], tensors[n("a2")]
        # the decay's two products through the narrow middle are one matrix times x: it rides in the
        # projection beside q, k, v and g (made in float64, rounded once), its bias with it
        decay_w = (a2.double() @ a1.double()).to(a1.dtype)
        self.in_w = _matrix(torch.cat([tensors[n(x)] for x in ("q", "k", "v", "g")] + [decay_w]))
        self.in_b = torch.cat([tensors[n("a2.b")].new_zeros(2 * self.qk_width + 2 * self.v_width), tensors[n("a2.b")]]).contiguous()
        self.first_weight = self.in_w
        self.out_w = _matrix(_padded_columns(tensors[n("o")]))
        self.norm_w = tensors[n("norm")]

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        T = x.shape[0]
        mark = ctx.scratch_mark()
        u = ctx.scratch((T, 3 * self.qk_width + 2 * self.v_width), torch.float32)
        kernels.linear(u, x, self.in_w, bias=self.in_b, splits=kernels.splits_alone(T))
        a, b = self.qk_width, 2 * self.qk_width
        z = u[:, b + 2 * self.v_width:]
        out, whole = _rows_for(ctx, T, self.v_width, -(-self.v_width // 8) * 8)
        kernels.state_scan(out, u[:, :a], u[:, a:b], u[:, b:b + self.v_width], cache.state, 0,
                           ctx.array("sequences.starts"), ctx.array("sequences.lens"), ctx.slot_ids, ctx.n_requests,
                           self.n_heads, self.n_heads, self.key_dim, self.value_dim, channel_decay=z,
                           channel_logit_mult=1.0 / self.tau, k_mult=self.key_dim**-0.5, unit_rms=True, eps=self.eps,
                           norm_weight=self.norm_w, gate=u[:, b + self.v_width:], chunked=self._chunked(ctx),
                           spans=self._spans(ctx))
        kernels.linear(residual, out if whole is None else whole, self.out_w, accumulate=True, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


class StateSpace(_SequenceArrays, Mixer):
    """The selective state space with a scalar decay a head:

        ``S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T``,   ``y_t = S_t^T C_t + D_h x_t``

    ``Win x`` is laid out ``[z: inner | x: inner | B: groups * state | C: groups * state | dt: heads]``
    with ``inner = n_heads * value_dim``; ``x``, ``B`` and ``C`` pass a causal convolution per
    channel (``taps`` taps, the last for the current token, zeros before a request's start, a
    bias) and a silu; ``dt = softplus(dt + dt_bias)``; head ``h`` reads group ``h // (n_heads /
    groups)``.  ``y * silu(z)`` is RMS-normed in ``norm_groups`` equal parts, multiplied by a
    weight and projected by ``Wo``.  A request's state is its last ``taps - 1`` convolution inputs
    and ``S`` (``state x value_dim`` a head), float32, zero at its start.  The projection writes
    float32 rows; everything up to the normed output is 32-bit (csrc/linear_state.hip).  No
    counterpart in mlx_lm/models/gpt2.py.
    """

    graph_safe = True
    can_overwrite = True

    def __init__(self, width, n_heads, value_dim, state, groups, taps, norm_groups, eps,
                 names=("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o"), prefix=""):
        super().__init__(prefix)
        if n_heads <= 0 or groups <= 0 or n_heads % groups:
            raise ValueError(f"{n_heads} heads cannot be grouped over {groups} groups")
        if not 0 < value_dim <= 256 or state <= 0 or taps < 1:
            raise ValueError(f"values of {value_dim} (at most 256), a state of {state}, {taps} taps")
        inner = n_heads * value_dim
        if norm_groups <= 0 or inner % norm_groups:
            raise ValueError(f"{inner} inner columns cannot be normed in {norm_groups} equal parts")
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        self.width, self.n_heads, self.value_dim, self.state, self.groups = width, n_heads, value_dim, state, groups
        self.taps, self.norm_groups, self.eps, self.inner = int(taps), int(norm_groups), float(eps), inner
        self.channels = inner + 2 * groups * state
        self.in_width = 2 * inner + 2 * groups * state + n_heads
        keys = ("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o")
        self.names = dict(zip(keys, (self._name(n) for n in names)))
        self.conv_floats = (self.taps - 1) * self.channels
        self.overwrite = False

    def cache_need(self):
        return StateNeed((self.conv_floats + self.n_heads * self.state * self.value_dim,), "float32")

    def tensors(self):
        n = self.names
        return {n["in"]: TensorSpec((self.in_width, self.width), "matrix"),
                n["conv"]: TensorSpec((self.channels, self.taps), "vector"),
                n["conv.b"]: TensorSpec((self.channels,), "vector"),
                n["dt_bias"]: TensorSpec((self.n_heads,), "vector"),
                n["A_log"]: TensorSpec((self.n_heads,), "vector"),
                n["D"]: TensorSpec((self.n_heads,), "vector"),
                n["norm"]: TensorSpec((self.inner,), "vector"),
                n["o"]: TensorSpec((self.width, self.inner), "matrix")}

    def load(self, tensors):
        n = self.names
        self.in_w, self.out_w = _matrix(tensors[n["in"]]), _matrix(_padded_columns(tensors[n["o"]]))
        self.first_weight = self.in_w
        self.conv_w, self.conv_b = tensors[n["conv"]].contiguous(), tensors[n["conv.b"]]
        self.dt_bias, self.a_log, self.skip = tensors[n["dt_bias"]], tensors[n["A_log"]], tensors[n["D"]]
        self.norm_w = tensors[n["norm"]]

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        T, H, GN = x.shape[0], self.n_heads, self.groups * self.state
        mark = ctx.scratch_mark()
        u = ctx.scratch((T, self.in_width), torch.float32)
        kernels.linear(u, x, self.in_w, splits=kernels.splits_alone(T))
        xbc = ctx.scratch((T, self.channels), torch.float32)
        dt = ctx.scratch((T, H), torch.float32)
        log_a = ctx.scratch((T, H), torch.float32)
        starts, lens = ctx.array("sequences.starts"), ctx.array("sequences.lens")
        single = ctx.array("sequences.longest") == 1  # a decode step: the convolution's kernel keeps the state itself
        kernels.ssm_prepare(xbc, dt, log_a, u, self.inner, self.inner + self.channels, self.conv_w, self.conv_b,
                            self.dt_bias, self.a_log, cache.state, 0, ctx.token_req, starts, ctx.slot_ids,
                            single_tokens=single)
        if not single:
            kernels.conv_state_update(u, self.inner, self.taps, self.channels, cache.state, 0, starts, lens, ctx.slot_ids,
                                      ctx.n_requests)
        y = ctx.scratch((T, self.inner), torch.float32)
        kernels.state_scan(y, xbc[:, self.inner + GN:], xbc[:, self.inner:self.inner + GN], xbc[:, :self.inner],
                           cache.state, self.conv_floats, starts, lens, ctx.slot_ids, ctx.n_requests, H, self.groups,
                           self.state, self.value_dim, log_a=log_a, k_scale=dt, skip=self.skip, chunked=self._chunked(ctx),
                           spans=self._spans(ctx))
        out, whole = _rows_for(ctx, T, self.inner, -(-self.inner // 8) * 8)
        kernels.gated_group_rmsnorm(out, y, u[:, :self.inner], self.norm_w, self.norm_groups, self.eps)
        kernels.linear(residual, out if whole is None else whole, self.out_w, accumulate=not self.overwrite, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


class LightningAttention(_SequenceArrays, Mixer):
    """Linear attention with a fixed decay per head, activated projections and one norm over all heads:

        ``S_t = decay_h S_(t-1) + k_t v_t^T``,   ``o_t = S_t^T q_t``

    with ``q = silu(Wq x)``, ``k = silu(Wk x)`` (``n_heads x key_dim``), ``v = silu(Wv x)`` (``n_heads x
    value_dim``); nothing else is scaled.  The heads, side by side, pass one RMS norm with the weight
    ``norm`` (``n_heads * value_dim`` values), are multiplied by ``sigmoid(Wg x)`` and projected by
    ``Wo``.  ``S`` (``key_dim x value_dim`` a head, float32, zero at a request's start) is the
    request's state.  One product gives ``[q | k | v | g]`` as float32 rows; the activations, the
    recurrence, the norm and the gate are 32-bit (csrc/state_gates.hip, csrc/linear_state.hip).
    No counterpart in mlx_lm/models/gpt2.py.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    can_overwrite = True  # writes its output instead of adding it where ``overwrite`` is set

    def __init__(self, width, n_heads, key_dim, value_dim, decay, eps, prefix=""):
        super().__init__(prefix)
        if n_heads <= 0 or key_dim <= 0 or not 0 < value_dim <= 256:
            raise ValueError(f"{n_heads} heads of keys {key_dim} and values {value_dim} (values at most 256)")
        if len(decay) != n_heads or any(not 0.0 < float(d) <= 1.0 for d in decay):
            raise ValueError(f"decays {list(decay)}: one in (0, 1] for each of the {n_heads} heads")
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        self.width, self.n_heads, self.key_dim, self.value_dim = width, n_heads, key_dim, value_dim
        self.decay_values, self.eps = [float(d) for d in decay], float(eps)
        self.qk_width, self.v_width = n_heads * key_dim, n_heads * value_dim
        self.overwrite = False
        self.projection_given = False  # a pair of parallel mixers makes both mixers' projections in one product

    def cache_need(self):
        return StateNeed((self.n_heads * self.key_dim * self.value_dim,), "float32")

    def tensors(self):
        n = self._name
        return {n("q"): TensorSpec((self.qk_width, self.width), "matrix"),
                n("k"): TensorSpec((self.qk_width, self.width), "matrix"),
                n("v"): TensorSpec((self.v_width, self.width), "matrix"),
                n("g"): TensorSpec((self.v_width, self.width), "matrix"),
                n("o"): TensorSpec((self.width, self.v_width), "matrix"),
                n("norm"): TensorSpec((self.v_width,), "vector")}

    def input_names(self):
        """The tensors whose rows, in this order, are the projection that ``forward`` starts with."""
        return [self._name(x) for x in ("q", "k", "v", "g")]

    def load(self, tensors):
        n = self._name
        self.out_w = _matrix(_padded_columns(tensors[n("o")]))
        if not self.projection_given:
            self.in_w = _matrix(torch.cat([tensors[x] for x in self.input_names()]))
            self.first_weight = self.in_w
        self.norm_w = tensors[n("norm")]
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=self.norm_w.device)

    def forward(self, ctx, x, residual, cache, writes_cache=True, rows=None):
        """``rows``: the projection's float32 rows, where the caller has made them already."""
        T = x.shape[0]
        mark = ctx.scratch_mark()
        a, b = self.qk_width, 2 * self.qk_width
        u = rows
        if u is None:
            u = ctx.scratch((T, b + 2 * self.v_width), torch.float32)
            kernels.linear(u, x, self.in_w, splits=kernels.splits_alone(T))
        kernels.silu_columns(u, 0, b + self.v_width)
        y = ctx.scratch((T, self.v_width), torch.float32)
        kernels.state_scan(y, u[:, :a], u[:, a:b], u[:, b:b + self.v_width], cache.state, cache.offset,
                           ctx.array("sequences.starts"), ctx.array("sequences.lens"), ctx.slot_ids, ctx.n_requests,
                           self.n_heads, self.n_heads, self.key_dim, self.value_dim, decay=self.decay,
                           chunked=self._chunked(ctx), spans=self._spans(ctx))
        out, whole = _rows_for(ctx, T, self.v_width, -(-self.v_width // 8) * 8)
        kernels.normed_gate(out, y, u[:, b + self.v_width:], self.norm_w, self.eps)
        kernels.linear(residual, out if whole is None else whole, self.out_w, accumulate=not self.overwrite, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


class ForgetGateAttention(_SequenceArrays, Mixer):
    """Linear attention whose key is the complement of its forget gate (HGRN2):

        ``S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T``,   ``o_t = S_t^T q_t``

    with ``q = silu(Wq x)`` (``n_heads x key_dim``), ``v = Wv x`` (``n_heads x value_dim``) and, per
    head and key channel, ``f = l + (1 - l) sigmoid(Wf x + b)`` with the floor ``l`` from the tensor
    ``lower``; the keys come from the gate alone and nothing is scaled.  Each head's ``o`` is RMS-normed over
    ``value_dim`` with the weight ``norm`` (shared by the heads), the heads are concatenated and
    projected by ``Wo``.  ``S`` (``key_dim x value_dim`` a head, float32, zero at a request's start)
    is the request's state.  One product gives ``[q | z | v]`` as float32 rows; ``1 - f`` (made as
    ``(1 - l) sigmoid(-z)``, without cancellation), ``log f``, the recurrence with a decay per key
    channel and the norm are 32-bit (csrc/state_gates.hip, csrc/linear_state.hip).  No counterpart
    in mlx_lm/models/gpt2.py.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, width, n_heads, key_dim, value_dim, eps, prefix=""):
        super().__init__(prefix)
        if n_heads <= 0 or key_dim <= 0 or not 0 < value_dim <= 256:
            raise ValueError(f"{n_heads} heads of keys {key_dim} and values {value_dim} (values at most 256)")
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        self.width, self.n_heads, self.key_dim, self.value_dim, self.eps = width, n_heads, key_dim, value_dim, float(eps)
        self.qk_width, self.v_width = n_heads * key_dim, n_heads * value_dim

    def cache_need(self):
        return StateNeed((self.n_heads * self.key_dim * self.value_dim,), "float32")

    def tensors(self):
        n = self._name
        return {n("q"): TensorSpec((self.qk_width, self.width), "matrix"),
                n("f"): TensorSpec((self.qk_width, self.width), "matrix"),
                n("f.b"): TensorSpec((self.qk_width,), "vector"),
                n("lower"): TensorSpec((self.qk_width,), "vector"),
                n("v"): TensorSpec((self.v_width, self.width), "matrix"),
                n("norm"): TensorSpec((self.value_dim,), "vector"),
                n("o"): TensorSpec((self.width, self.v_width), "matrix")}

    def load(self, tensors):
        n = self._name
        self.in_w = _matrix(torch.cat([tensors[n(x)] for x in ("q", "f", "v")]))
        bias = tensors[n("f.b")]
        self.in_b = torch.cat([bias.new_zeros(self.qk_width), bias, bias.new_zeros(self.v_width)]).contiguous()
        self.first_weight = self.in_w
        self.out_w = _matrix(_padded_columns(tensors[n("o")]))
        self.lower, self.norm_w = tensors[n("lower")].contiguous(), tensors[n("norm")]

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        T = x.shape[0]
        mark = ctx.scratch_mark()
        a, b = self.qk_width, 2 * self.qk_width
        u = ctx.scratch((T, b + self.v_width), torch.float32)
        kernels.linear(u, x, self.in_w, bias=self.in_b, splits=kernels.splits_alone(T))
        keys = ctx.scratch((T, a), torch.float32)
        kernels.forget_gate(u, 0, a, a, self.lower, keys)  # (queries activated, logits to log f, keys = 1 - f)
        out, whole = _rows_for(ctx, T, self.v_width, -(-self.v_width // 8) * 8)
        kernels.state_scan(out, u[:, :a], keys, u[:, b:], cache.state, cache.offset,
                           ctx.array("sequences.starts"), ctx.array("sequences.lens"), ctx.slot_ids, ctx.n_requests,
                           self.n_heads, self.n_heads, self.key_dim, self.value_dim, channel_decay=u[:, a:b],
                           unit_rms=True, eps=self.eps, norm_weight=self.norm_w, chunked=self._chunked(ctx),
                           spans=self._spans(ctx))
        kernels.linear(residual, out if whole is None else whole, self.out_w, accumulate=True, splits=kernels.splits_alone(T))
        ctx.scratch_release(mark)


class ParallelMixers(Mixer):
    """Two mixers side by side that read the same input: ``left_scale * left(x) + right_scale *
    right(x)``.  The left one keeps the run's cache slot, the right one the run's state slot (the
    arrangement passes both on: ``wants_state``).  The two outputs are float32 rows and are summed
    in float32.  Where both mixers start with a projection of ``x`` into float32 rows and name its
    tensors (``input_names``), one product makes both projections and each mixer gets its columns."""

    can_overwrite = True
    wants_state = True

    def __init__(self, left, right, left_scale=1.0, right_scale=1.0, prefix=""):
        from .base import MIXERS, build_part

        super().__init__(prefix)
        self.left = build_part(MIXERS, "mixer", left)
        self.right = build_part(MIXERS, "mixer", right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.overwrite = False
        for m in (self.left, self.right):
            if getattr(m, "can_overwrite", False) and hasattr(m, "overwrite"):
                m.overwrite = True
        self.graph_safe = all(getattr(m, "graph_safe", False) for m in (self.left, self.right))
        # two mixers that start with a projection into float32 rows and say of which tensors
        # (``input_names``) get both from one product
        self.shared_projection = all(hasattr(m, "input_names") and hasattr(m, "projection_given") for m in (self.left, self.right))
        if self.shared_projection:
            self.left.projection_given = self.right.projection_given = True
        self.in_w, self.in_cols = None, None

    def sub_parts(self):
        return (self.left, self.right)

    def load(self, tensors):
        if self.shared_projection:
            parts = [[tensors[n] for n in m.input_names()] for m in (self.left, self.right)]
            self.in_cols = [sum(t.shape[0] for t in ts) for ts in parts]
            self.in_w = _matrix(torch.cat(parts[0] + parts[1]))
            self.first_weight = self.in_w

    def cache_need(self):
        return self.left.cache_need()

    def state_need(self):
        need = self.right.cache_need()
        if need is not None and not isinstance(need, StateNeed):
            raise ValueError("the right one of two parallel mixers keeps per-request state or nothing")
        return need

    # (the two mixers are parts of the model in their own right, ``sub_parts``: the model hands
    # them their tensors and asks them for their step arrays; nothing here owns a tensor)

    def forward(self, ctx, x, residual, cache, writes_cache=True, state=None):
        mark = ctx.scratch_mark()
        outs, rows = [], (None, None)
        if self.shared_projection:
            T, (nl, nr) = x.shape[0], self.in_cols
            u = ctx.scratch((T, nl + nr), torch.float32)
            kernels.linear(u, x, self.in_w, splits=kernels.splits_alone(T))
            rows = (u[:, :nl], u[:, nl:])
        for m, slot, r in ((self.left, cache, rows[0]), (self.right, state, rows[1])):
            y = ctx.scratch(tuple(residual.shape), torch.float32)
            if not getattr(m, "overwrite", False):
                y.zero_()
            if r is not None:
                m.forward(ctx, x, y, slot, writes_cache, rows=r)
            else:
                m.forward(ctx, x, y, slot, writes_cache)
            outs.append(y)
        kernels.scaled_pair_sum(residual, self.left_scale, outs[0], self.right_scale, outs[1], accumulate=not self.overwrite)
        ctx.scratch_release(mark)


register_mixer("retention", Retention)
register_mixer("gated_linear_attention", GatedLinearAttention)
register_mixer("state_space", StateSpace)
register_mixer("lightning_attention", LightningAttention)
register_mixer("forget_gate_attention", ForgetGateAttention)
register_mixer("parallel", ParallelMixers)
