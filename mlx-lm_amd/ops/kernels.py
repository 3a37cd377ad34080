"""Python faces of the HIP kernels: argument checks, pointers, launch.

Each function takes torch tensors that live on the GPU, checks on the host
what the kernel assumes about them (shape, dtype, contiguity) and launches on
torch's current stream.  Nothing here computes on the CPU or through a torch
operator; a missing library raises.  A model's step does not come through
here: the native host (``csrc/engine.hip``) issues its launches itself.  These
faces are for a kernel alone (tests), for parts written in Python, and for
sampling; ``linear`` and ``PendingSum`` call the native host's own product
routine, so there is one place that chooses among the product kernels.
"""

import ctypes
import weakref

import torch

from . import build, native

_c_int = ctypes.c_int
_c_float = ctypes.c_float
_c_size_t = ctypes.c_size_t
_vp = ctypes.c_void_p

DT = {torch.float32: 0, torch.bfloat16: 1}

GEMM_GELU = 1
GEMM_ACCUMULATE = 2
GEMM_OUT_F32 = 4
GEMM_KV = 8

# Up to this many rows a bfloat16 product goes to the decode kernels, which stream the weights
# once and fuse the norm and the cache scatter; more rows go to the tile kernels.
DECODE_MAX_ROWS = 16


# torch's current stream as a raw handle.  torch.cuda.current_stream() builds a Stream object
# through several Python layers (some 4 us a call, once per launch); the binding below is what
# that ends in.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


def raw_stream():
    """The handle of the stream that torch launches on now, as an integer."""
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _stream():
    return _vp(raw_stream())


def n_compute_units():
    """Compute units of the current device (asked of the device once)."""
    return native.lib().eng_compute_units()


_BARE = {}


def bare_context():
    """A native context outside any step: the stream, the split workspace, no scratch memory."""
    dev = torch.cuda.current_device()
    c = _BARE.get(dev)
    if c is None:
        c = _BARE[dev] = native.EngCtx()
        ws = split_workspace(torch.device("cuda", dev))
        c.split_ws, c.split_ws_floats = ws.data_ptr(), ws.numel()
        c.n_compute_units = n_compute_units()
        c.dtype = 1
    c.stream = raw_stream()
    c.force_splits = force_splits
    return c


def _ptr(t):
    return _vp(t.data_ptr()) if t is not None else _vp(0)


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def _fail(msg):
    """``cond or _fail(f"...")``: the message is put together only when the check fails."""
    raise ValueError(msg)


def _dev(t, name, dtype=None):
    t.is_cuda or _fail(f"{name} must be on the GPU")
    t.is_contiguous() or _fail(f"{name} must be contiguous")
    if dtype is not None:
        t.dtype == dtype or _fail(f"{name} must be {dtype}, is {t.dtype}")


def _rows2d(t, name):
    """A 2-D tensor whose rows are contiguous; returns its row stride."""
    t.is_cuda or _fail(f"{name} must be on the GPU")
    (t.dim() == 2 and t.stride(1) == 1) or _fail(f"{name} must be 2-D with contiguous rows")
    return t.stride(0)


# ---------------------------------------------------------------------------


def embed_gather_add(out, table, ids, add_table=None, add_ids=None, scale=1.0):
    """``out[t] = table[ids[t]] * scale (+ add_table[add_ids[t]])`` into float32 ``out``."""
    lib = build.load("embed")
    n, width = out.shape
    _dev(out, "out", torch.float32)
    _dev(table, "table")
    _dev(ids, "ids", torch.int32)
    table.dtype in DT or _fail(f"table dtype {table.dtype} not supported")
    _need(table.shape[1] == width and ids.numel() >= n, "embed_gather_add: shapes disagree")
    if add_table is not None:
        _dev(add_table, "add_table", table.dtype)
        _dev(add_ids, "add_ids", torch.int32)
        _need(add_table.shape[1] == width and add_ids.numel() >= n, "embed_gather_add: shapes disagree")
    rc = lib.embed_scale_add(
        _ptr(out), _ptr(table), _ptr(ids), _ptr(add_table), _ptr(add_ids),
        _c_int(n), _c_int(width), _c_int(DT[table.dtype]), ctypes.c_float(scale), _stream(),
    )
    build.check(lib, rc, "embed_gather_add")
    return out


def feed_tokens(ids, src, index, vocab):
    """``ids[t] = src[index[t]]`` where ``index[t] >= 0``: sampled tokens that are still on the device."""
    lib = build.load("embed")
    for name, t in (("ids", ids), ("src", src), ("index", index)):
        _dev(t, name, torch.int32)
    _need(index.numel() >= ids.numel(), "feed_tokens: an index for every id")
    rc = lib.feed_tokens(_ptr(ids), _ptr(src), _ptr(index), _c_int(ids.numel()), _c_int(vocab), _stream())
    build.check(lib, rc, "feed_tokens")
    return ids


def layernorm(out, x, gamma, beta, eps, rows=None):
    """LayerNorm of float32 rows of ``x`` (all, or those listed in ``rows``) into ``out``."""
    lib = build.load("norm")
    n, width = out.shape
    _dev(out, "out")
    _dev(x, "x", torch.float32)
    out.dtype in DT or _fail(f"out dtype {out.dtype} not supported")
    _need(x.shape[-1] == width, "layernorm: widths disagree")
    if rows is None:
        _need(x.shape[0] >= n, "layernorm: fewer input rows than output rows")
    else:
        _dev(rows, "rows", torch.int32)
        _need(rows.numel() >= n, "layernorm: fewer row indices than output rows")
    for name, v in (("gamma", gamma), ("beta", beta)):
        if v is not None:
            _dev(v, name, torch.float32)
            v.numel() == width or _fail(f"layernorm: {name} has {v.numel()} elements, width is {width}")
    rc = lib.layernorm(
        _ptr(out), _ptr(x), _ptr(rows), _ptr(gamma), _ptr(beta), _c_float(eps),
        _c_int(n), _c_int(width), _c_int(DT[out.dtype]), _stream(),
    )
    build.check(lib, rc, "layernorm")
    return out


class NormedInput:
    """The LayerNorm of float32 rows (``rms``: their root-mean-square norm, no mean taken off and
    no shift), not computed yet.

    ``linear`` takes it as its input and, where its kernel can, norms the rows
    itself while the first weights are on their way; anything else calls
    ``materialize()`` and gets the tensor.
    """

    def __init__(self, alloc, x, gamma, beta, eps, dtype, rms=False):
        self.alloc, self.x, self.gamma, self.beta, self.eps, self.dtype = alloc, x, gamma, beta, eps, dtype
        self.rms = bool(rms)
        self.shape = tuple(x.shape)
        self._out = None

    def materialize(self):
        if self._out is None:
            self._out = self.alloc(self.shape, self.dtype)
            if self.rms:
                rmsnorm(self._out, self.x, self.gamma, self.eps)
            else:
                layernorm(self._out, self.x, self.gamma, self.beta, self.eps)
        return self._out


def normed(x):
    """``x`` as a tensor: a ``NormedInput`` is computed (once), a tensor is itself."""
    return x.materialize() if isinstance(x, NormedInput) else x


def rmsnorm(out, x, weight, eps):
    """``out = x / sqrt(mean(x^2) + eps) * weight`` over float32 rows ``x``; ``out`` float32 or bfloat16."""
    lib = build.load("rmsnorm")
    ldx = _f32_rows(x, "x", out.shape[1])
    _dev(weight, "weight", torch.float32)
    _need(out.is_contiguous() and out.dtype in DT and weight.numel() == out.shape[1] and x.shape[0] >= out.shape[0], "rmsnorm: shapes")
    rc = lib.rmsnorm(_ptr(out), _ptr(x), _c_int(ldx), None, _ptr(weight), _c_float(eps), _c_int(out.shape[0]),
                     _c_int(out.shape[1]), _c_int(DT[out.dtype]), _stream())
    build.check(lib, rc, "rmsnorm")
    return out


class KVScatter:
    """Where the key and value columns of a fused q/k/v projection go: the
    pages of ``kv``, for each token at its request's position."""

    def __init__(self, kv, block_table, token_req, positions, q_width):
        self.kv, self.block_table, self.token_req, self.positions = kv, block_table, token_req, positions
        self.q_width = q_width
        self.kv_width = kv.n_kv_heads * kv.head_dim


class PackedWeight:
    """A bfloat16 weight matrix ``[N, K]`` in the order the decode kernel's lanes read it.

    Tiles of 16 features by 64 k, zero padded; tile ``(b, c)`` holds, for lane
    ``l`` (feature ``l % 16``, k group ``l // 16``), first the 8 values
    ``k = 64 c + 16 (l // 16) + 0..7`` of all lanes, then the 8 values ``+ 8..15``.
    A wave's load is then 1 KB of consecutive bytes.  The kernels that take
    many rows read this order too, so the row-major matrix need not be kept
    (``keep_rows=False`` lets it go: one copy of the weights on the device).
    """

    def __init__(self, w, keep_rows=True):
        _need(w.dtype == torch.bfloat16 and w.dim() == 2, "PackedWeight: a 2-D bfloat16 matrix")
        self.w = w if keep_rows else None
        self.shape, self.dtype, self.device = tuple(w.shape), w.dtype, w.device
        N, K = w.shape
        Np, Kp = (N + 15) // 16 * 16, (K + 63) // 64 * 64
        padded = torch.zeros((Np, Kp), dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
        # (block, feature, k-block, k group, half, 8) -> (block, k-block, half, k group, feature, 8)
        t = padded.view(Np // 16, 16, Kp // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5)
        self.packed = t.contiguous().view(-1)
        # what one block of the decode kernel reads (16 features, all of K) and how many there are
        self.chunk_bytes, self.n_chunks = Kp * 16 * 2, Np // 16
        self.c = native.EngWeight(w.data_ptr() if keep_rows else None, self.packed.data_ptr(), N, K,
                                  w.stride(0) if keep_rows else 0, DT[w.dtype], self.chunk_bytes, self.n_chunks, 0)


class PackedRows:
    """bfloat16 activations ``[M, K]`` in the order in which the product of 17 to 64 rows reads them
    fastest: tiles of 16 rows by 64 columns, each laid out like a tile of ``PackedWeight``.  What
    lies beyond row ``M`` or column ``K`` in the last tiles is never used.

    ``PackedRows.empty(M, K, device)`` makes room for a kernel to write into
    (``sum_partials_norm(..., out=...)``, ``attn_decode``, ``linear(out=...)``);
    ``PackedRows.of(a)`` packs a row-major matrix and ``.rows()`` gives it back (tests)."""

    def __init__(self, data, shape):
        self.data, self.shape = data, tuple(shape)
        self.dtype, self.device = data.dtype, data.device

    @classmethod
    def empty(cls, M, K, device):
        n = (M + 15) // 16 * ((K + 63) // 64) * 1024
        return cls(torch.zeros(n, dtype=torch.bfloat16, device=device), (M, K))

    @classmethod
    def of(cls, a):
        _need(a.dtype == torch.bfloat16 and a.dim() == 2, "PackedRows: a 2-D bfloat16 matrix")
        M, K = a.shape
        Mp, Kp = (M + 15) // 16 * 16, (K + 63) // 64 * 64
        padded = torch.zeros((Mp, Kp), dtype=a.dtype, device=a.device)
        padded[:M, :K] = a
        t = padded.view(Mp // 16, 16, Kp // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5)
        return cls(t.contiguous().view(-1), (M, K))

    def rows(self):
        M, K = self.shape
        Mp, Kp = (M + 15) // 16 * 16, (K + 63) // 64 * 64
        t = self.data.view(Mp // 16, Kp // 64, 2, 4, 16, 8).permute(0, 4, 1, 3, 2, 5)
        return t.reshape(Mp, Kp)[:M, :K].contiguous()

    def data_ptr(self):
        return self.data.data_ptr()


def wants_packed_rows(w, n_rows):
    """Whether the product of ``n_rows`` rows with ``w`` (a ``PackedWeight``) reads its rows fastest
    as ``PackedRows``: the kernel that holds a block's weights in registers takes it."""
    if not isinstance(w, PackedWeight):
        return False
    return bool(native.lib().eng_wants_packed_rows(ctypes.byref(bare_context()), ctypes.byref(w.c), int(n_rows)))


def weight_struct(w):
    """The native description of a weight matrix (a ``PackedWeight`` or a 2-D tensor ``[N, K]``)."""
    if isinstance(w, PackedWeight):
        return w.c
    ld = _rows2d(w, "w")
    w.dtype in DT or _fail(f"weight dtype {w.dtype} not supported")
    return native.EngWeight(w.data_ptr(), None, w.shape[0], w.shape[1], ld, DT[w.dtype], 0, 0, 0)


def read_ahead_pays(w, n_rows, with_norm=False):
    """Whether the rows' next product should have ``w`` read ahead by the kernel before it: a
    ``PackedWeight`` that the decode kernel takes whole, 16 features a block (then block ``j``
    reads chunk ``j``, on die ``j % 8``), for few enough rows that most CUs have none."""
    if not isinstance(w, PackedWeight):
        return False
    return bool(native.lib().eng_read_ahead_pays(ctypes.byref(bare_context()), ctypes.byref(w.c), int(n_rows),
                                                 1 if with_norm else 0))


def for_decode(w, keep_rows=False):
    """``w`` in the packed order where the product kernels can use it (bfloat16 on the GPU),
    instead of the row-major matrix unless ``keep_rows``; anything else is returned as it is."""
    if isinstance(w, torch.Tensor) and w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2:
        return PackedWeight(w, keep_rows=keep_rows)
    return w


_SPLIT_WS = {}
SPLIT_WS_FLOATS = 8 << 20  # 32 MB: sixteen splits of 64 rows by 8192 features

# Tests set this to split K wherever the kernels can, also at sizes where the
# launch would fill the GPU without (tiny models): 0 leaves the choice to the library.
force_splits = 0


def splits_alone(n_rows):
    """``splits`` for a product of ``n_rows`` rows whose partial sums nobody else would add (a part
    written in Python has no norm behind it that takes them): 17 to 64 rows go unsplit, since the
    second kernel that adds the parts costs more there than the split saves (a decode step of 32
    rows, 1,024 wide: 1.92 ms against 2.08); otherwise the library chooses."""
    return 1 if DECODE_MAX_ROWS < n_rows <= 64 else None


def split_workspace(device):
    """Float32 room for the partial sums of projections that split K over blocks.

    One per device, made at first use and kept (before any step is recorded):
    launches on one stream follow each other, and at most one sum is pending.
    """
    device = torch.device(device)
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    ws = _SPLIT_WS.get(key)
    if ws is None:
        ws = torch.empty(SPLIT_WS_FLOATS, dtype=torch.float32, device=device)
        _SPLIT_WS[key] = ws
    return ws


class PendingSum:
    """Partial products that still have to be added into the residual stream.

    A projection that splits K leaves ``n_splits`` partial sums in the
    workspace; with a ``PendingSum`` given, ``linear(accumulate=True)`` may
    stop there.  Whoever reads the stream next either adds them and norms the
    rows in one kernel (``settle_normed``) or just adds them (``settle``).
    ``allowed`` is set by a caller that promises to do so.  The state is a
    struct of the native host's (a step's own lies in its context).
    """

    def __init__(self, c=None, ctx=None):
        self.c = c if c is not None else native.EngPending()
        # the step whose pending sum this is, if any (weakly: the step holds this object)
        self._ctx = weakref.proxy(ctx) if ctx is not None else None

    allowed = property(lambda self: bool(self.c.allowed),
                       lambda self, v: setattr(self.c, "allowed", 1 if v else 0))
    target = property(lambda self: self.c.target)  # the address that the sum goes to, or None
    n_splits = property(lambda self: self.c.n_splits)

    def _native(self):
        if self._ctx is None:
            return bare_context()
        self._ctx.c.stream = raw_stream()
        return self._ctx.c

    def waits_on(self, x):
        c = self.c
        return bool(c.target) and c.target == x.data_ptr() and (c.rows, c.cols) == tuple(x.shape)

    def settle(self):
        """Add what is pending (if anything) into its target."""
        native.check(native.lib().eng_pending_settle(ctypes.byref(self._native()), ctypes.byref(self.c)))

    def settle_normed(self, out, gamma, beta, eps, ahead=None):
        """Add what is pending into its target and write the LayerNorm of the new rows to ``out``.

        ``ahead``: the weights of the product that reads ``out`` (see ``sum_partials_norm``);
        ``out`` may be a ``PackedRows`` where that product reads its rows fastest so."""
        packed = isinstance(out, PackedRows)
        if packed:
            m = native.EngMat(out.data_ptr(), out.shape[0], out.shape[1], 0, DT[out.dtype])
        else:
            _need(out.is_contiguous(), "settle_normed: out must be contiguous")
            m = native.mat(out)
        native.check(native.lib().eng_pending_settle_normed(
            ctypes.byref(self._native()), ctypes.byref(self.c), ctypes.byref(m), native.ptr(gamma),
            native.ptr(beta), float(eps), ctypes.byref(ahead.c) if ahead is not None else None, 1 if packed else 0))

    def can_norm(self, x):
        if not self.waits_on(x) or x.stride(1) != 1:
            return False
        m = native.mat(x)
        return bool(native.lib().eng_pending_can_norm(ctypes.byref(self.c), ctypes.byref(m)))


def _scatter_args(sc):
    return (
        _ptr(sc.kv.k if sc else None), _ptr(sc.kv.v if sc else None),
        _c_size_t(sc.kv.page_stride if sc else 0), _ptr(sc.block_table if sc else None),
        _c_int(sc.block_table.shape[1] if sc else 0), _ptr(sc.token_req if sc else None),
        _ptr(sc.positions if sc else None), _c_int(sc.q_width if sc else 0),
        _c_int(sc.kv_width if sc else 0), _c_int(sc.kv.head_dim if sc else 0),
        _c_int(sc.kv.page_size if sc else 0),
    )


def sum_partials(out, ws, n_splits, bias=None, gelu=False, accumulate=False, scatter=None):
    """``out = epilogue(sum of the partial products ws[:n_splits] + bias)``: the
    second step of a projection that split K (``linear`` runs it itself unless
    the sum stays pending)."""
    lib = build.load("gemm_bf16_decode")
    M, N = out.shape
    _dev(out, "out")
    _dev(ws, "ws", torch.float32)
    _need(ws.numel() >= n_splits * M * N, "sum_partials: workspace too small")
    flags = (GEMM_GELU if gelu else 0) | (GEMM_ACCUMULATE if accumulate else 0)
    if out.dtype == torch.float32:
        flags |= 0 if accumulate else GEMM_OUT_F32
    else:
        _need(out.dtype == torch.bfloat16 and not accumulate, "sum_partials: out must be float32 or bfloat16")
    if scatter is not None:
        flags |= GEMM_KV
    rc = lib.sum_partials(_ptr(out), _ptr(ws), _c_int(n_splits), _ptr(bias), _c_int(M), _c_int(N),
                          _c_int(_rows2d(out, "out")), _c_int(flags), *_scatter_args(scatter), _stream())
    build.check(lib, rc, "sum_partials")
    return out


def sum_partials_norm(h, ws, n_splits, bias, gamma, beta, eps, out, ahead=None):
    """``h += bias + sum of the partial products``; ``out = LayerNorm(h)`` (rows of ``h``, all of them).

    ``ahead``: the ``PackedWeight`` of the product that comes next; CUs that have no row read it
    meanwhile, each the chunks that a block on its own die will ask for."""
    lib = build.load("gemm_bf16_decode")
    M, N = h.shape
    _dev(h, "h", torch.float32)
    _dev(ws, "ws", torch.float32)
    packed = isinstance(out, PackedRows)
    if packed:
        _need(out.shape == (M, N), "sum_partials_norm: out's shape")
    else:
        _dev(out, "out")
        _need(out.dtype in DT and tuple(out.shape) == (M, N) and out.is_contiguous(), "sum_partials_norm: out")
    _need(ws.numel() >= n_splits * M * N, "sum_partials_norm: workspace too small")
    for name, v in (("bias", bias), ("gamma", gamma), ("beta", beta)):
        if v is not None:
            _dev(v, name, torch.float32)
            v.numel() == N or _fail(f"sum_partials_norm: {name} has {v.numel()} elements, width is {N}")
    rc = lib.sum_partials_norm(_ptr(h), _c_int(_rows2d(h, "h")), _ptr(ws), _c_int(n_splits), _ptr(bias),
                               _ptr(gamma), _ptr(beta), _c_float(eps), _ptr(out.data if packed else out),
                               _c_int(DT[out.dtype]), _c_int(1 if packed else 0),
                               _c_int(M), _c_int(N), _ptr(ahead.packed if ahead is not None else None),
                               _c_size_t(ahead.chunk_bytes if ahead is not None else 0),
                               _c_int(ahead.n_chunks if ahead is not None else 0), _stream())
    build.check(lib, rc, "sum_partials_norm")
    return out


ACTIVATIONS = {None: 0, "gelu_tanh": 1, "relu2": 2}  # the product kernels' epilogue activations, by code


def linear(out, a, w, bias=None, gelu=False, accumulate=False, variant=0, scatter=None, splits=None,
           pending=None, activation=None):
    """``out = epilogue(a @ w.T + bias)``.

    ``gelu`` asks for the tanh GELU in the epilogue; ``activation`` names any of ``ACTIVATIONS``
    (``"relu2"``: the square of the ReLU) instead.

    ``a`` is ``[M, K]`` (or a ``NormedInput``), ``w`` is ``[N, K]`` (or a
    ``PackedWeight``, whose packed copy the decode kernel reads), both
    float32 or both bfloat16; ``bias`` float32.  ``accumulate`` adds into a
    float32 ``out`` (the residual stream); otherwise ``out`` is float32 or the
    operands' dtype.  With ``scatter`` (a ``KVScatter``) the columns from
    ``scatter.q_width`` on are also written to the key/value pages.  Up to 16
    bfloat16 rows go to the decode kernels, which fuse the norm and the
    scatter; 17 to 48 rows of packed weights to the kernel that holds a
    block's weights in registers; more go to the tile kernels.  Where the launch
    would not fill the GPU, both split K over ``splits`` blocks and add the
    partial sums in a second kernel; with ``accumulate`` and a ``pending``
    that allows it, that second step is left to the next reader of ``out``.
    The choices are the native host's (``linear`` in csrc/engine.hip), which
    a model's step uses too.
    """
    L = native.lib()
    ctx = pending._native() if pending is not None else bare_context()
    call = native.EngLinear()
    call.w = weight_struct(w)
    N, K = call.w.N, call.w.K
    if isinstance(a, NormedInput):
        M = a.shape[0]
        fused = variant == 0 and L.eng_linear_norms_itself(ctypes.byref(ctx), M, N, K, DT[a.dtype], splits or 0)
        if not fused:
            a = a.materialize()
    if isinstance(a, NormedInput):
        _dev(a.x, "x", torch.float32)
        call.a.lazy, call.a.ldx = 2 if a.rms else 1, a.x.stride(0)
        call.a.m = native.EngMat(None, a.shape[0], a.shape[1], a.shape[1], DT[a.dtype])
        call.a.x, call.a.gamma, call.a.beta, call.a.eps = a.x.data_ptr(), native.ptr(a.gamma), native.ptr(a.beta), a.eps
    elif isinstance(a, PackedRows):
        call.a.m = native.EngMat(a.data_ptr(), a.shape[0], a.shape[1], 0, DT[a.dtype])
        call.a.packed = 1
    else:
        call.a.m = native.mat(a)
    if isinstance(out, PackedRows):
        call.out = native.EngMat(out.data_ptr(), out.shape[0], out.shape[1], 0, DT[out.dtype])
        call.out_packed = 1
    else:
        call.out = native.mat(out)
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        _need(bias.numel() == N, "linear: bias length")
        call.bias = bias.data_ptr()
    sc = None
    if scatter is not None:
        kv = scatter.kv
        _attn_common(out, kv, scatter.block_table, scatter.token_req, scatter.positions)
        sc = native.EngScatter(kv.k.data_ptr(), kv.v.data_ptr(), kv.page_stride, kv.n_kv_heads, kv.head_dim,
                               kv.page_size, DT[kv.k.dtype], scatter.block_table.data_ptr(),
                               scatter.token_req.data_ptr(), scatter.positions.data_ptr(),
                               scatter.block_table.shape[1], scatter.q_width, scatter.kv_width, 0)
        call.scatter = ctypes.pointer(sc)
    if activation not in ACTIVATIONS:
        _fail(f"linear: unknown activation {activation!r} (known: {sorted(k for k in ACTIVATIONS if k)})")
    code = ACTIVATIONS[activation] or int(bool(gelu))
    call.gelu, call.accumulate, call.variant, call.splits = code, int(accumulate), int(variant), int(splits or 0)
    rc = L.eng_linear(ctypes.byref(ctx), ctypes.byref(call), ctypes.byref(pending.c) if pending is not None else None)
    native.check(rc, "linear")
    return out


# ---------------------------------------------------------------------------


class PagedKV:
    """Keys and values of one cache slot: two views ``[n_pages, Hkv, page, hd]``."""

    __slots__ = ("k", "v", "page_stride", "n_kv_heads", "head_dim", "page_size")

    def __init__(self, k, v):
        _need(k.shape == v.shape and k.dim() == 4, "PagedKV: k and v must be [pages, heads, page, dim]")
        _need(k.dtype == v.dtype and k.dtype in DT, "PagedKV: dtype")
        for t in (k, v):
            _need(t.is_cuda and t.stride(3) == 1 and t.stride(2) == t.shape[3]
                  and t.stride(1) == t.shape[2] * t.shape[3], "PagedKV: a page must be contiguous")
        _need(k.stride(0) == v.stride(0), "PagedKV: k and v page strides differ")
        self.k, self.v = k, v
        self.page_stride = k.stride(0)
        _, self.n_kv_heads, self.page_size, self.head_dim = k.shape


def _attn_common(qkv_like, kv, block_table, token_req, positions):
    _dev(block_table, "block_table", torch.int32)
    _dev(token_req, "token_req", torch.int32)
    _dev(positions, "positions", torch.int32)
    _need(block_table.dim() == 2, "block_table must be [requests, max_blocks]")
    _need(qkv_like.dtype == kv.k.dtype, "queries and cache must share a dtype")


def kv_write(k_src, v_src, kv, block_table, token_req, positions):
    """Scatter rows of ``k_src``/``v_src`` ``[T, Hkv*hd]`` into their pages."""
    lib = build.load("attention")
    ld = _rows2d(k_src, "k_src")
    _need(_rows2d(v_src, "v_src") == ld, "kv_write: k and v row strides differ")
    n = k_src.shape[0]
    _need(k_src.shape == v_src.shape and k_src.shape[1] == kv.n_kv_heads * kv.head_dim,
          "kv_write: source width must be n_kv_heads*head_dim")
    _attn_common(k_src, kv, block_table, token_req, positions)
    _need(token_req.numel() >= n and positions.numel() >= n, "kv_write: per-token arrays too short")
    rc = lib.kv_write(
        _ptr(k_src), _ptr(v_src), _c_int(ld), _ptr(kv.k), _ptr(kv.v), _c_size_t(kv.page_stride),
        _ptr(block_table), _c_int(block_table.shape[1]), _ptr(token_req), _ptr(positions),
        _c_int(n), _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size),
        _c_int(DT[k_src.dtype]), _stream(),
    )
    build.check(lib, rc, "kv_write")


class AttnTerms(ctypes.Structure):
    """Mirror of ``AttnTerms`` in csrc/attention_tiles.h."""

    _fields_ = [("head_scale", _vp), ("slopes", _vp), ("gate", _vp), ("ldg", _c_int), ("keep_first", _c_int),
                ("softcap", _c_float), ("dist_bias", _vp), ("n_dist", _c_int)]


class ScoreTerms:
    """Optional terms that the four attention kernels take beside the plain causal scores:
    ``head_scale`` (float32 ``[n_heads]``, instead of ``scale``), ``slopes`` (float32 ``[n_heads]``:
    ``slope * (query position - key position)`` is taken off a score), ``gate`` (``[tokens,
    n_heads * head_dim]`` of the queries' dtype: the output is multiplied by its sigmoid),
    ``keep_first`` (with a window, the first so many keys stay visible), ``softcap`` (a scaled
    score ``s`` becomes ``softcap * tanh(s / softcap)``) and ``distance_bias`` (float32 ``[n_heads,
    n]``: entry ``min(distance, n - 1)`` of the head's row is added to a score).  A score takes
    them in this order: scale, cap, slope, table."""

    def __init__(self, head_scale=None, slopes=None, gate=None, keep_first=0, softcap=0.0, distance_bias=None):
        self.head_scale, self.slopes, self.gate, self.keep_first = head_scale, slopes, gate, int(keep_first)
        self.softcap, self.distance_bias = float(softcap), distance_bias

    def struct(self, q, n_heads):
        """The terms as the kernels' ``_terms`` entry points and the native host take them."""
        a = self.args(q, n_heads)
        t = AttnTerms()
        t.head_scale, t.slopes, t.gate = _ptr(self.head_scale), _ptr(self.slopes), _ptr(self.gate)
        t.ldg, t.keep_first, t.softcap = a[3].value, self.keep_first, self.softcap
        _need(self.softcap >= 0.0, "softcap must not be negative")
        if self.distance_bias is not None:
            _dev(self.distance_bias, "distance_bias", torch.float32)
            _need(self.distance_bias.dim() == 2 and self.distance_bias.shape[0] == n_heads and self.distance_bias.is_contiguous(),
                  "distance_bias: a contiguous row a head")
            t.dist_bias, t.n_dist = _ptr(self.distance_bias), self.distance_bias.shape[1]
        return t

    def args(self, q, n_heads):
        for name in ("head_scale", "slopes"):
            t = getattr(self, name)
            if t is not None:
                _dev(t, name, torch.float32)
                _need(t.numel() == n_heads, f"{name}: one value a head")
        ldg = 0
        if self.gate is not None:
            ldg = _rows2d(self.gate, "gate")
            _need(self.gate.dtype == q.dtype and self.gate.shape == q.shape, "gate: the queries' shape and dtype")
        return [_ptr(self.head_scale), _ptr(self.slopes), _ptr(self.gate), _c_int(ldg), _c_int(self.keep_first)]


def _terms(terms, q, n_heads):
    """The terms as the one argument that the kernels' ``_terms`` entry points take."""
    return [ctypes.byref((terms or ScoreTerms()).struct(q, n_heads))]


def attn_tile(out, q, kv, block_table, token_req, positions, tiles, n_tiles, n_heads, scale, window=0, terms=None):
    """Attention for tiles of up to 16 consecutive queries of one request each.

    ``tiles`` is int32 ``[n_tiles, 2]``: first flat row and number of rows.  ``terms``: ``ScoreTerms``.
    """
    lib = build.load("attention")
    ldq, ldo = _rows2d(q, "q"), _rows2d(out, "out")
    _need(q.shape[1] == n_heads * kv.head_dim, "attn_tile: q width must be n_heads*head_dim")
    _need(out.shape[1] == n_heads * kv.head_dim and out.dtype == q.dtype, "attn_tile: out shape/dtype")
    _attn_common(q, kv, block_table, token_req, positions)
    _dev(tiles, "tiles", torch.int32)
    _need(tiles.numel() >= 2 * n_tiles, "attn_tile: tile list too short")
    rc = lib.attn_tile_terms(
        _ptr(out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(tiles), _c_int(n_tiles), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), _c_int(DT[q.dtype]), *_terms(terms, q, n_heads), _stream(),
    )
    build.check(lib, rc, "attn_tile")
    return out


ATTN_ROW_MAX_HEAD_DIM = 144  # beyond this the per-wave key tiles do not fit in LDS


def attn_row(out, q, kv, block_table, token_req, positions, rows, n_rows, n_heads, scale,
             window=0, n_splits=1, part_o=None, part_ml=None, terms=None):
    """Attention for single query rows, keys split ``n_splits`` ways."""
    lib = build.load("attention")
    ldq, ldo = _rows2d(q, "q"), _rows2d(out, "out")
    _need(q.shape[1] == n_heads * kv.head_dim, "attn_row: q width must be n_heads*head_dim")
    _need(out.shape[1] == n_heads * kv.head_dim and out.dtype == q.dtype, "attn_row: out shape/dtype")
    _need(kv.head_dim <= ATTN_ROW_MAX_HEAD_DIM,
          f"attn_row: head_dim {kv.head_dim} above {ATTN_ROW_MAX_HEAD_DIM}; use attn_tile")
    _attn_common(q, kv, block_table, token_req, positions)
    _dev(rows, "rows", torch.int32)
    _need(rows.numel() >= n_rows, "attn_row: row list too short")
    if n_splits > 1:
        _dev(part_o, "part_o", torch.float32)
        _dev(part_ml, "part_ml", torch.float32)
        _need(part_o.numel() >= n_rows * n_heads * n_splits * kv.head_dim, "attn_row: part_o too small")
        _need(part_ml.numel() >= n_rows * n_heads * n_splits * 2, "attn_row: part_ml too small")
    rc = lib.attn_row_terms(
        _ptr(out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(rows), _c_int(n_rows), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), _c_int(n_splits), _ptr(part_o), _ptr(part_ml), _c_int(DT[q.dtype]),
        *_terms(terms, q, n_heads), _stream(),
    )
    build.check(lib, rc, "attn_row")
    return out


_TILE_SIZES = None


def attn_tile_sizes():
    """``(queries a tile of attn_tile, queries a tile of attn_prefill)``: what the kernels are
    compiled with (``csrc/attention_tiles.h``, the one place these sizes are written), asked of
    the native host, which includes the same header."""
    global _TILE_SIZES
    if _TILE_SIZES is None:
        a, b = ctypes.c_int(), ctypes.c_int()
        native.lib().eng_attn_tile_sizes(ctypes.byref(a), ctypes.byref(b))
        _TILE_SIZES = (a.value, b.value)
    return _TILE_SIZES


def rows_split_from():
    """The context length from which a decode step may split a row's keys over blocks (the native
    host's policy; recorded decode steps are kept apart by it)."""
    return int(native.lib().eng_rows_split_from())


def attn_prefill_takes(q_dtype, kv):
    """Whether the matrix-core prefill kernel takes this cache geometry."""
    return q_dtype == torch.bfloat16 and kv.head_dim in (32, 64, 128, 256)


def attn_prefill(out, q, kv, block_table, token_req, positions, tiles, n_tiles, n_heads, scale, window=0, terms=None):
    """``attn_tile`` on the matrix cores: bfloat16, head_dim 32/64/128/256, tiles of up to 128 queries."""
    lib = build.load("attention_prefill")
    ldq, ldo = _rows2d(q, "q"), _rows2d(out, "out")
    _need(q.dtype == torch.bfloat16, "attn_prefill: bfloat16 only")
    _need(q.shape[1] == n_heads * kv.head_dim, "attn_prefill: q width must be n_heads*head_dim")
    _need(out.shape[1] == n_heads * kv.head_dim and out.dtype == q.dtype, "attn_prefill: out shape/dtype")
    _attn_common(q, kv, block_table, token_req, positions)
    _dev(tiles, "tiles", torch.int32)
    _need(tiles.numel() >= 2 * n_tiles, "attn_prefill: tile list too short")
    rc = lib.attn_prefill_terms(
        _ptr(out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(tiles), _c_int(n_tiles), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), *_terms(terms, q, n_heads), _stream(),
    )
    build.check(lib, rc, "attn_prefill")
    return out


def attn_decode_takes(q_dtype, kv):
    """Whether the register-streaming decode kernel takes this cache geometry."""
    if q_dtype not in (torch.bfloat16, torch.float32):
        return False
    key_bytes = kv.head_dim * q_dtype.itemsize
    return key_bytes in (64, 128, 256, 512) and kv.page_size % (1024 // key_bytes) == 0


def attn_decode(out, q, kv, block_table, token_req, positions, rows, n_rows, n_heads, scale,
                window=0, n_splits=1, part_o=None, part_ml=None, n_waves=4, ahead=None, ahead_chunks=0,
                rows_are_requests=False, key_tile=32, join_in_kernel=0, terms=None):
    """``attn_row`` for keys of 64 to 512 bytes (bfloat16 with head_dim 32, 64, 128 or 256, float32
    with 16, 32, 64 or 128): keys stream into registers.

    ``ahead``: a ``PackedWeight`` whose first ``ahead_chunks`` chunks the CUs without a row read
    meanwhile, each the chunks that a block on its own die will ask for (``sum_partials_norm``).
    ``rows_are_requests``: item ``i`` of ``rows`` is row ``i`` of request ``i`` (the caller says so).
    ``key_tile``: 32 or 64 keys a wave at a time.  ``join_in_kernel``: 0, a second kernel joins
    the ``n_splits`` parts of a (row, head); 1, the block that finishes it last does; 2, the same,
    and a short row takes fewer than ``n_splits`` by its own length."""
    lib = build.load("attention_decode")
    packed_out = isinstance(out, PackedRows)  # (the order that the product after attention reads fastest)
    ldq, ldo = _rows2d(q, "q"), 0 if packed_out else _rows2d(out, "out")
    _need(q.dtype in (torch.bfloat16, torch.float32), "attn_decode: bfloat16 or float32")
    _need(q.shape[1] == n_heads * kv.head_dim, "attn_decode: q width must be n_heads*head_dim")
    _need(out.shape[1] == n_heads * kv.head_dim and out.dtype == q.dtype, "attn_decode: out shape/dtype")
    if packed_out:
        _need(out.shape[0] >= q.shape[0], "attn_decode: out has fewer rows than q")
    _attn_common(q, kv, block_table, token_req, positions)
    _dev(rows, "rows", torch.int32)
    _need(rows.numel() >= n_rows, "attn_decode: row list too short")
    if n_splits > 1:
        _dev(part_o, "part_o", torch.float32)
        _dev(part_ml, "part_ml", torch.float32)
        _need(part_o.numel() >= n_rows * n_heads * n_splits * kv.head_dim, "attn_decode: part_o too small")
        _need(part_ml.numel() >= n_rows * n_heads * n_splits * 2, "attn_decode: part_ml too small")
    if rows_are_requests:
        _need(n_rows <= block_table.shape[0], "attn_decode: more rows than requests")
    rc = lib.attn_decode_rows_terms(
        _ptr(out.data if packed_out else out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(rows), _c_int(n_rows), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), _c_int(n_splits), _ptr(part_o), _ptr(part_ml), _c_int(n_waves),
        _ptr(ahead.packed if ahead is not None else None),
        _c_size_t(ahead.chunk_bytes if ahead is not None else 0),
        _c_int(min(ahead_chunks, ahead.n_chunks) if ahead is not None else 0),
        _c_int(1 if rows_are_requests else 0), _c_int(DT[q.dtype]), _c_int(key_tile),
        _c_int(int(join_in_kernel)), *_terms(terms, q, n_heads), _stream(),
    )
    build.check(lib, rc, "attn_decode")
    return out


def attn_decode_group(out, q, kv, block_table, token_req, positions, rows, n_rows, n_heads, scale, window=0, n_splits=1,
                      part_o=None, part_ml=None, rows_are_requests=False):
    """``attn_row`` for bfloat16 caches with head_dim 64, 128 or 256 where many query heads share a key
    head: a block takes sixteen query heads of a key head at once, on the matrix cores, so a key is
    read once for all of them.  ``n_splits`` parts of a row's keys, joined by a second kernel."""
    lib = build.load("attention_decode")
    ldq, ldo = _rows2d(q, "q"), _rows2d(out, "out")
    _need(q.dtype == torch.bfloat16 and out.dtype == q.dtype, "attn_decode_group: bfloat16 only")
    _need(q.shape[1] == n_heads * kv.head_dim and out.shape[1] == q.shape[1], "attn_decode_group: rows of n_heads*head_dim")
    _attn_common(q, kv, block_table, token_req, positions)
    _dev(rows, "rows", torch.int32)
    _need(rows.numel() >= n_rows, "attn_decode_group: row list too short")
    if n_splits > 1:
        _dev(part_o, "part_o", torch.float32)
        _dev(part_ml, "part_ml", torch.float32)
        _need(part_o.numel() >= n_rows * n_heads * n_splits * kv.head_dim, "attn_decode_group: part_o too small")
        _need(part_ml.numel() >= n_rows * n_heads * n_splits * 2, "attn_decode_group: part_ml too small")
    if rows_are_requests:
        _need(n_rows <= block_table.shape[0], "attn_decode_group: more rows than requests")
    rc = lib.attn_decode_group(
        _ptr(out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v), _c_size_t(kv.page_stride), _ptr(block_table),
        _c_int(block_table.shape[1]), _ptr(token_req), _ptr(positions), _ptr(rows), _c_int(n_rows), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window), _c_float(scale), _c_int(n_splits),
        _ptr(part_o), _ptr(part_ml), _c_int(1 if rows_are_requests else 0), _stream())
    build.check(lib, rc, "attn_decode_group")
    return out


# ---------------------------------------------------------------------------


def sample_rows(tokens, token_logprob, logits, temp, top_p, min_p, min_keep, top_k, xtc_prob,
                xtc_thr, seed, counter, xtc_special=None, logprobs=None):
    """Sample one token from each row of float32 ``logits``; see csrc/sampling.hip."""
    lib = build.load("sampling")
    ld = _rows2d(logits, "logits")
    n, vocab = logits.shape
    _need(logits.dtype == torch.float32, "sample_rows: logits must be float32")
    _dev(tokens, "tokens", torch.int32)
    _dev(token_logprob, "token_logprob", torch.float32)
    for name, t, dt in (("temp", temp, torch.float32), ("top_p", top_p, torch.float32),
                        ("min_p", min_p, torch.float32), ("min_keep", min_keep, torch.int32),
                        ("top_k", top_k, torch.int32), ("xtc_prob", xtc_prob, torch.float32),
                        ("xtc_thr", xtc_thr, torch.float32), ("seed", seed, torch.int64),
                        ("counter", counter, torch.int32)):
        _dev(t, name, dt)
        t.numel() >= n or _fail(f"sample_rows: {name} shorter than the rows")
    _need(tokens.numel() >= n and token_logprob.numel() >= n, "sample_rows: outputs too short")
    n_special = 0
    if xtc_special is not None and xtc_special.numel() > 0:
        _dev(xtc_special, "xtc_special", torch.int32)
        n_special = xtc_special.numel()
    ld_lp = 0
    if logprobs is not None:
        ld_lp = _rows2d(logprobs, "logprobs")
        _need(logprobs.dtype == torch.float32 and logprobs.shape[0] >= n and logprobs.shape[1] >= vocab,
              "sample_rows: logprobs shape/dtype")
    rc = lib.sample_rows(
        _ptr(tokens), _ptr(token_logprob), _ptr(logprobs), _c_int(ld_lp), _ptr(logits), _c_int(ld),
        _c_int(n), _c_int(vocab), _ptr(temp), _ptr(top_p), _ptr(min_p), _ptr(min_keep), _ptr(top_k),
        _ptr(xtc_prob), _ptr(xtc_thr), _ptr(seed), _ptr(counter),
        _ptr(xtc_special if n_special else None), _c_int(n_special), _stream(),
    )
    build.check(lib, rc, "sample_rows")


def apply_logit_bias(logits, offsets, idx, val):
    lib = build.load("sampling")
    ld = _rows2d(logits, "logits")
    _need(logits.dtype == torch.float32, "apply_logit_bias: logits must be float32")
    _dev(offsets, "offsets", torch.int32)
    _dev(idx, "idx", torch.int32)
    _dev(val, "val", torch.float32)
    _need(offsets.numel() == logits.shape[0] + 1, "apply_logit_bias: offsets length")
    rc = lib.apply_logit_bias(_ptr(logits), _c_int(ld), _c_int(logits.shape[0]), _ptr(offsets),
                              _ptr(idx), _ptr(val), _stream())
    build.check(lib, rc, "apply_logit_bias")


def apply_penalties(logits, offsets, hist, rep, rep_ctx, pres, pres_ctx, freq, freq_ctx):
    lib = build.load("sampling")
    ld = _rows2d(logits, "logits")
    n = logits.shape[0]
    _need(logits.dtype == torch.float32, "apply_penalties: logits must be float32")
    _dev(offsets, "offsets", torch.int32)
    _dev(hist, "hist", torch.int32)
    _need(offsets.numel() == n + 1, "apply_penalties: offsets length")
    for name, t, dt in (("rep", rep, torch.float32), ("pres", pres, torch.float32),
                        ("freq", freq, torch.float32), ("rep_ctx", rep_ctx, torch.int32),
                        ("pres_ctx", pres_ctx, torch.int32), ("freq_ctx", freq_ctx, torch.int32)):
        _dev(t, name, dt)
        t.numel() >= n or _fail(f"apply_penalties: {name} shorter than the rows")
    rc = lib.apply_penalties(_ptr(logits), _c_int(ld), _c_int(n), _ptr(offsets), _ptr(hist),
                             _ptr(rep), _ptr(rep_ctx), _ptr(pres), _ptr(pres_ctx), _ptr(freq),
                             _ptr(freq_ctx), _c_int(logits.shape[1]), _stream())
    build.check(lib, rc, "apply_penalties")


# ---------------------------------------------------------------------------
# layers normed on both sides of their sublayers; heads normed one by one


def add_normed(h, y, w_post, mult, eps, w_next=None, out=None):
    """``h += mult * LN(y; w_post)`` on float32 rows, and ``out = LN(h; w_next)`` of the new rows
    where ``w_next`` is given (csrc/sandwich_block.hip)."""
    lib = build.load("sandwich_block")
    ldh, ldy = _rows2d(h, "h"), _rows2d(y, "y")
    _need(h.dtype == torch.float32 and y.dtype == torch.float32 and h.shape == y.shape, "add_normed: float32 rows of one shape")
    n, width = h.shape
    _dev(w_post, "w_post", torch.float32)
    _need(w_post.numel() == width, "add_normed: w_post length")
    if w_next is not None:
        _dev(w_next, "w_next", torch.float32)
        _dev(out, "out")
        _need(w_next.numel() == width and tuple(out.shape) == (n, width) and out.dtype in DT, "add_normed: w_next / out")
    rc = lib.add_normed(_ptr(h), _c_int(ldh), _ptr(y), _c_int(ldy), _ptr(w_post), _c_float(mult), _c_float(eps),
                        _ptr(w_next), _ptr(out if w_next is not None else None), _c_int(n), _c_int(width),
                        _c_int(DT[out.dtype] if w_next is not None else 0), _stream())
    build.check(lib, rc, "add_normed")
    return h


def scaled_pair_sum(y, a, ya, b, yb, accumulate=False):
    """``y = a * ya + b * yb`` (``+= `` with ``accumulate``) on float32 rows of one shape."""
    lib = build.load("sandwich_block")
    for name, t in (("y", y), ("ya", ya), ("yb", yb)):
        _dev(t, name, torch.float32)
        _need(t.shape == y.shape, "scaled_pair_sum: shapes differ")
    rc = lib.scaled_pair_sum(_ptr(y), _c_float(a), _ptr(ya), _c_float(b), _ptr(yb), ctypes.c_long(y.numel()),
                             _c_int(int(bool(accumulate))), _stream())
    build.check(lib, rc, "scaled_pair_sum")
    return y


def head_rmsnorm(x, n_heads, head_stride, dim, weight, eps):
    """RMS norm of the first ``dim`` columns of each of ``n_heads`` heads, ``head_stride`` columns
    apart, of every row of ``x``, in place (csrc/head_norm.hip)."""
    lib = build.load("head_norm")
    ld = _rows2d(x, "x")
    _need(x.dtype in DT, "head_rmsnorm: float32 or bfloat16")
    _need(0 < dim <= head_stride and (n_heads - 1) * head_stride + dim <= x.shape[1], "head_rmsnorm: heads do not fit the rows")
    if weight is not None:
        _dev(weight, "weight", torch.float32)
        _need(weight.numel() == dim, "head_rmsnorm: weight length")
    rc = lib.head_rmsnorm(_ptr(x), _c_int(ld), _c_int(x.shape[0]), _c_int(n_heads), _c_int(head_stride), _c_int(dim),
                          _ptr(weight), _c_float(eps), _c_int(DT[x.dtype]), _stream())
    build.check(lib, rc, "head_rmsnorm")
    return x


# ---------------------------------------------------------------------------
# mixers with a decaying matrix state per head (csrc/linear_state.hip)


class ScanArgs(ctypes.Structure):
    """Mirror of ``ScanArgs`` in csrc/linear_state.hip."""

    _fields_ = [("q", _vp), ("k", _vp), ("v", _vp), ("ldq", _c_int), ("ldk", _c_int), ("ldv", _c_int),
                ("log_a", _vp), ("decay", _vp), ("k_scale", _vp), ("k_mult", _c_float), ("skip", _vp),
                ("rot_dims", _c_int), ("inv_freq", _vp), ("positions", _vp), ("unit_rms", _c_int), ("eps", _c_float),
                ("gate", _vp), ("ldg", _c_int), ("out", _vp), ("ldo", _c_int), ("out_dtype", _c_int),
                ("state", _vp), ("state_stride", _c_size_t), ("state_offset", _c_size_t), ("seq_start", _vp),
                ("seq_len", _vp), ("slot_ids", _vp), ("n_requests", _c_int), ("H", _c_int), ("Hk", _c_int),
                ("N", _c_int), ("P", _c_int), ("n_tokens_hint", _c_int), ("chan_a", _vp), ("ldca", _c_int),
                ("chan_logit", _c_int), ("chan_mult", _c_float), ("norm_w", _vp)]


def _f32_rows(t, name, min_cols):
    ld = _rows2d(t, name)
    _need(t.dtype == torch.float32, f"{name} must be float32")
    _need(t.shape[1] >= min_cols, f"{name}: rows of {t.shape[1]} columns, {min_cols} needed")
    return ld


def state_scan(out, q, k, v, state, state_offset, seq_start, seq_len, slot_ids, n_requests, n_heads, n_key_heads,
               key_dim, value_dim, log_a=None, decay=None, k_scale=None, k_mult=1.0, skip=None, rot_dims=0,
               inv_freq=None, positions=None, unit_rms=False, eps=0.0, gate=None, chunked=False, spans=None,
               channel_decay=None, channel_logit_mult=None, norm_weight=None):
    """``S = a S + k v^T; o = S^T q`` token by token for every (request, head), from and into the
    requests' rows of ``state`` (float32 ``[slots, floats a request]``, head ``h``'s matrix
    ``[key_dim, value_dim]`` at ``state_offset + h * key_dim * value_dim``).  ``q``, ``k``
    (``[tokens, >= n_key_heads * key_dim]``), ``v`` (``[tokens, >= n_heads * value_dim]``) and
    ``gate`` are float32 rows (column views of a projection's output are fine; with ``chunked`` and
    ``rot_dims`` the rows of ``q`` and ``k`` are turned in place, so they are work memory); ``out`` is
    ``[tokens, n_heads * value_dim]`` in float32 or bfloat16.  ``chunked``: the kernel that takes
    up to 64 tokens of a request at a time (for steps in which a request brings many); otherwise
    token by token.  ``spans``: ``(tokens a span, number of spans, span_req, span_start,
    span_first, alloc)`` cuts long portions into spans that run side by side (int32 device arrays:
    the request and the first token of every span, counted from the request's first token of
    this step, and every request's first span; ``alloc(shape, dtype)`` gives the work memory).
    ``channel_decay`` (float32 ``[tokens, >= n_heads * key_dim]``): a decay for every key channel
    instead of one a head, given as its logarithm, or, with ``channel_logit_mult = m``, as a logit
    ``z`` with ``log a = m * log sigmoid(z)``.  ``norm_weight`` (float32 ``[value_dim]``): with
    ``unit_rms``, the normed output times this weight, the same for every head.
    See csrc/linear_state.hip for the options."""
    lib = build.load("linear_state")
    a = ScanArgs()
    T = out.shape[0]
    a.ldq, a.ldk = _f32_rows(q, "q", n_key_heads * key_dim), _f32_rows(k, "k", n_key_heads * key_dim)
    a.ldv = _f32_rows(v, "v", n_heads * value_dim)
    _need(q.shape[0] >= T and k.shape[0] >= T and v.shape[0] >= T, "state_scan: fewer operand rows than output rows")
    a.q, a.k, a.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    for name, t in (("log_a", log_a), ("k_scale", k_scale)):
        if t is not None:
            _dev(t, name, torch.float32)
            _need(t.numel() >= T * n_heads, f"state_scan: {name} is [tokens, heads]")
            setattr(a, name, t.data_ptr())
    for name, t in (("decay", decay), ("skip", skip)):
        if t is not None:
            _dev(t, name, torch.float32)
            _need(t.numel() == n_heads, f"state_scan: {name} has one value a head")
            setattr(a, name, t.data_ptr())
    _need(log_a is not None or decay is not None or channel_decay is not None,
          "state_scan: a decay per token, per head or per key channel is needed")
    if channel_decay is not None:
        _need(n_key_heads == n_heads, "state_scan: decays per key channel need a key head for every head")
        a.ldca, a.chan_a = _f32_rows(channel_decay, "channel_decay", n_heads * key_dim), channel_decay.data_ptr()
        _need(channel_decay.shape[0] >= T, "state_scan: fewer decay rows than output rows")
        if channel_logit_mult is not None:
            a.chan_logit, a.chan_mult = 1, float(channel_logit_mult)
    if norm_weight is not None:
        _dev(norm_weight, "norm_weight", torch.float32)
        _need(unit_rms and norm_weight.numel() == value_dim, "state_scan: norm_weight has value_dim values and goes with unit_rms")
        a.norm_w = norm_weight.data_ptr()
    a.k_mult = float(k_mult)
    if rot_dims:
        _dev(inv_freq, "inv_freq", torch.float32)
        _dev(positions, "positions", torch.int32)
        _need(inv_freq.numel() == rot_dims // 2 and positions.numel() >= T, "state_scan: inv_freq / positions")
        a.rot_dims, a.inv_freq, a.positions = int(rot_dims), inv_freq.data_ptr(), positions.data_ptr()
    a.unit_rms, a.eps = int(bool(unit_rms)), float(eps)
    if gate is not None:
        a.ldg, a.gate = _f32_rows(gate, "gate", n_heads * value_dim), gate.data_ptr()
    a.ldo = _rows2d(out, "out")
    _need(out.dtype in DT and out.shape[1] == n_heads * value_dim, "state_scan: out is [tokens, heads * value_dim]")
    a.out, a.out_dtype = out.data_ptr(), DT[out.dtype]
    _dev(state, "state", torch.float32)
    _need(state.dim() == 2 and state_offset + n_heads * key_dim * value_dim <= state.shape[1], "state_scan: the state rows are too short")
    a.state, a.state_stride, a.state_offset = state.data_ptr(), state.stride(0), int(state_offset)
    for name, t in (("seq_start", seq_start), ("seq_len", seq_len), ("slot_ids", slot_ids)):
        _dev(t, name, torch.int32)
        _need(t.numel() >= n_requests, f"state_scan: {name} is shorter than the requests")
        setattr(a, name, t.data_ptr())
    a.n_requests, a.H, a.Hk, a.N, a.P = int(n_requests), int(n_heads), int(n_key_heads), int(key_dim), int(value_dim)
    a.n_tokens_hint = int(T)
    if spans is not None and chunked:
        span, n_spans, span_req, span_start, span_first, alloc = spans
        for name, t, n in (("span_req", span_req, n_spans), ("span_start", span_start, n_spans), ("span_first", span_first, n_requests)):
            _dev(t, name, torch.int32)
            _need(t.numel() >= n, f"state_scan: {name} too short")
        ws_state = alloc((n_spans * n_heads * key_dim * value_dim,), torch.float32)
        ws_decay = alloc((n_spans * n_heads * (key_dim if channel_decay is not None else 1),), torch.float32)
        rc = lib.state_scan(ctypes.byref(a), _c_int(2), _c_int(span), _c_int(n_spans), _ptr(span_req), _ptr(span_start),
                            _ptr(span_first), _ptr(ws_state), _ptr(ws_decay), _stream())
    else:
        rc = lib.state_scan(ctypes.byref(a), _c_int(int(bool(chunked))), _c_int(0), _c_int(0), None, None, None, None, None,
                            _stream())
    build.check(lib, rc, "state_scan")
    return out


# ---------------------------------------------------------------------------
# between a projection and the attention that reads its heads, and behind it (csrc/head_prepare.hip)


class PrepareArgs(ctypes.Structure):
    """Mirror of ``PrepareArgs`` in csrc/head_prepare.hip."""

    _fields_ = [("src", _vp), ("lds", _c_int), ("src_col", _c_int), ("src_stride", _c_int), ("n_rows", _c_int),
                ("n_heads", _c_int), ("dim", _c_int), ("norm_dim", _c_int), ("norm_w", _vp), ("eps", _c_float),
                ("rot_off", _c_int), ("rot_dims", _c_int), ("interleaved", _c_int), ("inv_freq", _vp),
                ("rot_mult", _c_float), ("positions", _vp), ("dst", _vp), ("ldd", _c_int), ("dst_stride", _c_int),
                ("dst_fill", _c_int), ("copies", _c_int), ("dst_head", _vp),
                ("conv_w", _vp), ("taps", _c_int), ("conv_channels", _c_int), ("conv_single", _c_int), ("conv_state", _vp),
                ("conv_state_stride", _c_size_t), ("conv_offset", _c_size_t), ("seq_start", _vp), ("slot_ids", _vp),
                ("token_req", _vp), ("block_table", _vp), ("max_blocks", _c_int), ("page_size", _c_int),
                ("page_stride", _c_size_t), ("norm_whole", _c_int)]


class ConvolutionAhead:
    """A causal convolution that ``head_prepare`` runs over its source's columns on their way in:
    ``y[t, c] = sum_j weight[c, j] * u[t - taps + 1 + j, c]`` over each request's own tokens (column
    ``c`` of ``u`` is channel ``c``); the inputs of earlier steps come from the request's row of
    ``state`` (``[taps - 1, channels]`` at ``offset``, the latest last).  With ``single`` (every
    request brings one token) the kernel also moves these up by one; otherwise ``conv_state_update``
    does afterwards."""

    def __init__(self, weight, state, offset, token_req, seq_start, slot_ids, single):
        _dev(weight, "weight", torch.float32)
        _dev(state, "state", torch.float32)
        for name, t in (("token_req", token_req), ("seq_start", seq_start), ("slot_ids", slot_ids)):
            _dev(t, name, torch.int32)
        channels, taps = weight.shape
        _need(weight.is_contiguous() and state.dim() == 2 and offset + (taps - 1) * channels <= state.shape[1],
              "a convolution's weight is [channels, taps] and its state rows hold taps - 1 inputs of every channel")
        self.weight, self.state, self.offset, self.single = weight, state, int(offset), bool(single)
        self.token_req, self.seq_start, self.slot_ids = token_req, seq_start, slot_ids


class PagesOut:
    """The keys' (or values') pages of a cache view as the place ``head_prepare`` writes to: a row goes
    where its request's block table and its position say, as ``kv_write`` has it."""

    def __init__(self, kv, values, block_table, token_req, positions):
        self.pages = kv.v if values else kv.k
        self.kv, self.block_table, self.token_req, self.positions = kv, block_table, token_req, positions
        for name, t in (("block_table", block_table), ("token_req", token_req), ("positions", positions)):
            _dev(t, name, torch.int32)
        self.dtype, self.shape = self.pages.dtype, None


def head_prepare(dst, src, src_col, n_heads, dim, **options):
    """Heads of a float32 projection row on their way to an attention: head ``h`` is ``dim`` columns
    of ``src`` from ``src_col + h * src_stride``; RMS norm over its first ``norm_dim`` columns
    (times ``norm_weight``, shared by the heads); rotation of ``rot_dims`` columns from ``rot_off``
    by ``position * inv_freq[i]`` (pairs ``(2i, 2i + 1)`` with ``interleaved``, else ``(i, i +
    rot_dims / 2)``; cos and sin times ``rot_mult``); written to ``dst`` (float32 or bfloat16) at
    column ``dst_head[c, h] * dst_stride`` for each of ``copies`` copies (``h * dst_stride`` without
    a table), with zeros from ``dim`` up to ``dst_fill`` columns.  ``norm_whole = n``: the norm runs over
    the ``n`` columns from ``src_col`` on, all heads at once, with ``norm_weight`` of ``n`` values, and
    every column of a head is normed.  ``conv`` (a ``ConvolutionAhead``):
    the source's columns pass a causal convolution first.  ``dst`` may be a ``PagesOut``."""
    lib = build.load("head_prepare")
    a = _prepare_args(dst, src, src_col, n_heads, dim, **options)
    rc = lib.head_prepare(ctypes.byref(a), _c_int(DT[dst.dtype]), _stream())
    build.check(lib, rc, "head_prepare")
    return dst


def head_prepare_many(*calls):
    """Several ``head_prepare`` calls in one launch: each of ``calls`` is ``(dst, src, src_col,
    n_heads, dim, options)``; at most four, their ``dst`` (a matrix or a ``PagesOut``) of one dtype."""
    lib = build.load("head_prepare")
    _need(1 <= len(calls) <= 4 and len({c[0].dtype for c in calls}) == 1, "head_prepare_many: one to four calls, outputs of one dtype")
    args = (PrepareArgs * len(calls))(*[_prepare_args(*c[:5], **c[5]) for c in calls])
    rc = lib.head_prepare_many(args, _c_int(len(calls)), _c_int(DT[calls[0][0].dtype]), _stream())
    build.check(lib, rc, "head_prepare_many")


def _prepare_args(dst, src, src_col, n_heads, dim, src_stride=None, dst_stride=None, dst_fill=None, norm_dim=0,
                  norm_weight=None, eps=0.0, rot_off=0, rot_dims=0, inv_freq=None, rot_mult=1.0, interleaved=True,
                  positions=None, dst_head=None, copies=1, conv=None, norm_whole=0):
    a = PrepareArgs()
    src_stride = dim if src_stride is None else src_stride
    n_rows = src.shape[0] if isinstance(dst, PagesOut) else dst.shape[0]
    dst_stride = dim if dst_stride is None else dst_stride
    a.lds = _f32_rows(src, "src", src_col + (n_heads - 1) * src_stride + dim)
    a.src, a.src_col, a.src_stride = src.data_ptr(), int(src_col), int(src_stride)
    a.n_rows, a.n_heads, a.dim = n_rows, int(n_heads), int(dim)
    _need(src.shape[0] >= n_rows, "head_prepare: fewer source rows than rows of dst")
    a.norm_dim, a.eps, a.norm_whole = int(norm_dim), float(eps), int(norm_whole)
    if norm_weight is not None:
        _dev(norm_weight, "norm_weight", torch.float32)
        _need(norm_weight.numel() == (norm_whole or norm_dim), "head_prepare: norm_weight has norm_dim values (norm_whole, for a norm over all heads)")
        a.norm_w = norm_weight.data_ptr()
    if rot_dims:
        _dev(inv_freq, "inv_freq", torch.float32)
        _dev(positions, "positions", torch.int32)
        _need(inv_freq.numel() == rot_dims // 2 and positions.numel() >= n_rows, "head_prepare: inv_freq / positions")
        a.rot_off, a.rot_dims, a.interleaved = int(rot_off), int(rot_dims), int(bool(interleaved))
        a.inv_freq, a.rot_mult, a.positions = inv_freq.data_ptr(), float(rot_mult), positions.data_ptr()
    _need(dst.dtype in DT, "head_prepare: dst is float32 or bfloat16")
    a.dst_stride, a.dst_fill, a.copies = int(dst_stride), int(dst_fill or dim), int(copies)
    if dst_head is not None:
        _dev(dst_head, "dst_head", torch.int32)
        _need(dst_head.numel() == copies * n_heads, "head_prepare: dst_head is [copies, heads]")
        a.dst_head = dst_head.data_ptr()
    if isinstance(dst, PagesOut):
        kv = dst.kv
        _need(kv.head_dim == dst_stride and n_heads * copies <= kv.n_kv_heads and dst.token_req.numel() >= n_rows
              and dst.positions.numel() >= n_rows, "head_prepare: the heads do not fit the cache's pages")
        a.dst, a.block_table, a.max_blocks = dst.pages.data_ptr(), dst.block_table.data_ptr(), dst.block_table.shape[1]
        a.page_size, a.page_stride = kv.page_size, kv.page_stride
        a.token_req, a.positions = dst.token_req.data_ptr(), dst.positions.data_ptr()
    else:
        a.ldd, a.dst = _rows2d(dst, "dst"), dst.data_ptr()
        _need(dst.shape[1] >= (n_heads * copies - 1) * dst_stride + a.dst_fill, "head_prepare: dst rows are too short for the heads")
    if conv is not None:
        channels, taps = conv.weight.shape
        _need(src.shape[1] >= channels and conv.token_req.numel() >= n_rows, "head_prepare: the convolution's channels are the source's columns")
        a.conv_w, a.taps, a.conv_channels, a.conv_single = conv.weight.data_ptr(), taps, channels, int(conv.single)
        a.conv_state, a.conv_state_stride, a.conv_offset = conv.state.data_ptr(), conv.state.stride(0), conv.offset
        a.seq_start, a.slot_ids, a.token_req = conv.seq_start.data_ptr(), conv.slot_ids.data_ptr(), conv.token_req.data_ptr()
    return a


def diff_combine(out, att, head_stride, first, second, lam, mult, eps, vdim):
    """``out[t, h] = mult * unit_rms(att[t, first[h]] - lam * att[t, second[h]])`` over the first
    ``vdim`` columns of heads that lie ``head_stride`` apart in ``att``."""
    lib = build.load("head_prepare")
    lda, ldo = _rows2d(att, "att"), _rows2d(out, "out")
    _dev(first, "first", torch.int32)
    _dev(second, "second", torch.int32)
    n_heads = first.numel()
    _need(second.numel() == n_heads and out.dtype == att.dtype and att.dtype in DT and att.shape[0] >= out.shape[0], "diff_combine: shapes")
    rc = lib.diff_combine(_ptr(att), _c_int(lda), _c_int(head_stride), _ptr(first), _ptr(second), _c_float(lam), _c_float(mult),
                          _c_float(eps), _c_int(out.shape[0]), _c_int(n_heads), _c_int(vdim), _ptr(out), _c_int(ldo),
                          _c_int(DT[out.dtype]), _stream())
    build.check(lib, rc, "diff_combine")
    return out


def head_gate(x, head_stride, n_heads, gate):
    """``x[t, h, :] *= sigmoid(gate[t, h])`` in place; ``gate`` float32 rows of at least ``n_heads`` columns."""
    lib = build.load("head_prepare")
    ldx, ldg = _rows2d(x, "x"), _f32_rows(gate, "gate", n_heads)
    _need(x.dtype in DT and x.shape[1] >= n_heads * head_stride and gate.shape[0] >= x.shape[0], "head_gate: shapes")
    rc = lib.head_gate(_ptr(x), _c_int(ldx), _c_int(head_stride), _c_int(n_heads), _ptr(gate), _c_int(ldg),
                       _c_int(x.shape[0]), _c_int(DT[x.dtype]), _stream())
    build.check(lib, rc, "head_gate")
    return x


FAST_HEAD_DIMS = (16, 32, 64, 128, 256)


def attention_head_dim(columns):
    """The head size under which a mixer with heads of ``columns`` columns keeps its pages: the
    next size that the matrix-core and the streaming attention kernels take (the columns beyond
    the head's own are zeros in queries, keys and values)."""
    for n in FAST_HEAD_DIMS:
        if columns <= n:
            return n
    raise ValueError(f"heads of {columns} columns: the attention kernels take at most {FAST_HEAD_DIMS[-1]}")


def attend(ctx, out, q, cache, n_heads, n_kv_heads, head_dim, scale, window=0, terms=None):
    """Causal attention of the step's queries ``q`` ``[tokens, n_heads * head_dim]`` over the pages
    of ``cache`` (a ``CacheView``), into ``out``: the native host chooses among the attention kernels
    as it does for the built-in attention part (single rows to the decode kernels, portions to the
    tile kernels), by the step arrays that part declares (``parts.attention.CausalSelfAttention``:
    a mixer that calls this names the same ``step_arrays_key``).  ``terms``: ``ScoreTerms``."""
    from ..parts.attention import CausalSelfAttention as A

    base = native.array_ids(A.step_arrays_key, A.step_array_names)
    qm, om = native.mat(q), native.mat(out)
    t = terms.struct(q, n_heads) if terms is not None else None
    with ctx.enter():
        if t is None:
            rc = native.lib().eng_attend(ctypes.byref(ctx.c), ctypes.byref(om), ctypes.byref(qm), cache.slot, int(n_heads),
                                         int(n_kv_heads), int(head_dim), int(window), float(scale), base)
        else:
            rc = native.lib().eng_attend_terms(ctypes.byref(ctx.c), ctypes.byref(om), ctypes.byref(qm), cache.slot,
                                               int(n_heads), int(n_kv_heads), int(head_dim), int(window), float(scale),
                                               base, ctypes.byref(t))
    native.check(rc, "attend")
    return out


def ssm_prepare(xbc, dt, log_a, u, conv_col, dt_col, conv_w, conv_b, dt_bias, a_log, state, conv_offset, token_req,
                seq_start, slot_ids, single_tokens=False):
    """The causal convolution (with the requests' last inputs from ``state``), bias and silu of
    columns ``conv_col ..`` of the float32 rows ``u`` into ``xbc``; ``dt = softplus(u[:, dt_col + h]
    + dt_bias[h])`` and ``log_a = -exp(a_log[h]) * dt`` (csrc/linear_state.hip).  ``single_tokens``:
    every request brings one token, and the kernel also does what ``conv_state_update`` would."""
    lib = build.load("linear_state")
    ldu = _f32_rows(u, "u", 1)
    T, C = xbc.shape
    H = dt.shape[1]
    taps = conv_w.shape[1]
    for name, t in (("xbc", xbc), ("dt", dt), ("log_a", log_a), ("conv_w", conv_w), ("dt_bias", dt_bias),
                    ("a_log", a_log), ("state", state)):
        _dev(t, name, torch.float32)
    if conv_b is not None:
        _dev(conv_b, "conv_b", torch.float32)
        _need(conv_b.numel() == C, "ssm_prepare: conv_b length")
    _need(tuple(conv_w.shape) == (C, taps) and dt.shape == log_a.shape and dt.shape[0] == T, "ssm_prepare: shapes")
    _need(dt_bias.numel() == H and a_log.numel() == H and u.shape[0] >= T, "ssm_prepare: per-head vectors")
    _need(conv_col + C <= u.shape[1] and dt_col + H <= u.shape[1], "ssm_prepare: columns beyond the rows")
    _need(state.dim() == 2 and conv_offset + (taps - 1) * C <= state.shape[1], "ssm_prepare: the state rows are too short")
    for name, t in (("token_req", token_req), ("seq_start", seq_start), ("slot_ids", slot_ids)):
        _dev(t, name, torch.int32)
    rc = lib.ssm_prepare(_ptr(u), _c_int(ldu), _c_int(conv_col), _c_int(dt_col), _ptr(conv_w), _ptr(conv_b),
                         _c_int(taps), _c_int(C), _c_int(H), _ptr(dt_bias), _ptr(a_log), _ptr(state),
                         _c_size_t(state.stride(0)), _c_size_t(conv_offset), _ptr(token_req), _ptr(seq_start),
                         _ptr(slot_ids), _ptr(xbc), _ptr(dt), _ptr(log_a), _c_int(T), _c_int(int(bool(single_tokens))),
                         _stream())
    build.check(lib, rc, "ssm_prepare")


def conv_state_update(u, conv_col, taps, n_channels, state, conv_offset, seq_start, seq_len, slot_ids, n_requests):
    """Each request's last ``taps - 1`` inputs (columns ``conv_col ..`` of ``u``) into its state row."""
    lib = build.load("linear_state")
    ldu = _f32_rows(u, "u", conv_col + n_channels)
    _dev(state, "state", torch.float32)
    _need(state.dim() == 2 and conv_offset + (taps - 1) * n_channels <= state.shape[1], "conv_state_update: the state rows are too short")
    for name, t in (("seq_start", seq_start), ("seq_len", seq_len), ("slot_ids", slot_ids)):
        _dev(t, name, torch.int32)
        _need(t.numel() >= n_requests, f"conv_state_update: {name} is shorter than the requests")
    rc = lib.conv_state_update(_ptr(u), _c_int(ldu), _c_int(conv_col), _c_int(taps), _c_int(n_channels), _ptr(state),
                               _c_size_t(state.stride(0)), _c_size_t(conv_offset), _ptr(seq_start), _ptr(seq_len),
                               _ptr(slot_ids), _c_int(n_requests), _stream())
    build.check(lib, rc, "conv_state_update")


def gated_group_rmsnorm(out, y, z, weight, groups, eps):
    """``out = RMSnorm(y * silu(z))`` in ``groups`` equal parts of a row, times ``weight``."""
    lib = build.load("linear_state")
    T, width = out.shape
    ldy, ldz, ldo = _f32_rows(y, "y", width), _f32_rows(z, "z", width), _rows2d(out, "out")
    _dev(weight, "weight", torch.float32)
    _need(weight.numel() == width and out.dtype in DT and y.shape[0] >= T and z.shape[0] >= T, "gated_group_rmsnorm: shapes")
    rc = lib.gated_group_rmsnorm(_ptr(y), _c_int(ldy), _ptr(z), _c_int(ldz), _ptr(weight), _c_float(eps), _c_int(T),
                                 _c_int(width), _c_int(groups), _ptr(out), _c_int(ldo), _c_int(DT[out.dtype]), _stream())
    build.check(lib, rc, "gated_group_rmsnorm")
    return out


# ---------------------------------------------------------------------------
# experts chosen per token (csrc/experts.hip)


def router_choice(idx, weight, z, correction, top, renormalize=False, weight_scale=1.0):
    """From float32 router outputs ``z`` ``[tokens, outputs]``: softmax, the ``top`` largest of
    softmax + ``correction`` into ``idx`` (int32 ``[tokens, top]``), their softmax values into
    ``weight``; with ``renormalize`` divided by their sum (+ 1e-20); times ``weight_scale``."""
    lib = build.load("experts")
    ldz = _f32_rows(z, "z", 1)
    T, n_out = z.shape
    _dev(idx, "idx", torch.int32)
    _dev(weight, "weight", torch.float32)
    _need(idx.numel() >= T * top and weight.numel() >= T * top, "router_choice: idx / weight too short")
    if correction is not None:
        _dev(correction, "correction", torch.float32)
        _need(correction.numel() == n_out, "router_choice: correction length")
    rc = lib.router_choice_scaled(_ptr(z), _c_int(ldz), _ptr(correction), _c_int(T), _c_int(n_out), _c_int(top), _ptr(idx),
                                  _ptr(weight), _c_int(int(bool(renormalize))), _c_float(weight_scale), _stream())
    build.check(lib, rc, "router_choice")


def route_and_gate(idx, weight, act, zu, correction, top, n_out, renormalize=False, weight_scale=1.0):
    """``router_choice`` on the first ``n_out`` columns of the float32 rows ``zu`` and ``silu_mul`` on
    the ``2 * act.shape[1]`` columns behind them, in one launch (for steps of few tokens)."""
    lib = build.load("experts")
    ld, ldo = _f32_rows(zu, "zu", 1), _rows2d(act, "act")
    T, F = act.shape
    _need(zu.shape[0] >= T and zu.shape[1] == n_out + 2 * F and act.dtype in DT, "route_and_gate: shapes")
    _dev(idx, "idx", torch.int32)
    _dev(weight, "weight", torch.float32)
    _need(idx.numel() >= T * top and weight.numel() >= T * top, "route_and_gate: idx / weight too short")
    if correction is not None:
        _dev(correction, "correction", torch.float32)
        _need(correction.numel() == n_out, "route_and_gate: correction length")
    rc = lib.route_and_gate_scaled(_ptr(zu), _c_int(ld), _ptr(correction), _c_int(T), _c_int(n_out), _c_int(top), _c_int(F),
                                   _ptr(idx), _ptr(weight), _ptr(act), _c_int(ldo), _c_int(DT[act.dtype]),
                                   _c_int(int(bool(renormalize))), _c_float(weight_scale), _stream())
    build.check(lib, rc, "route_and_gate")


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def silu_mul(out, gate_up, activation="silu"):
    """``out = act(gate_up[:, :F]) * gate_up[:, F:2F]`` with ``F = out.shape[1]``; ``activation``:
    ``silu``, or ``gelu_tanh`` (``0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))``)."""
    lib = build.load("experts")
    ld, ldo = _rows2d(gate_up, "gate_up"), _rows2d(out, "out")
    T, F = out.shape
    _need(gate_up.dtype == out.dtype and out.dtype in DT and gate_up.shape[1] == 2 * F and gate_up.shape[0] >= T, "silu_mul: shapes")
    _need(activation in GATE_ACTIVATIONS, f"silu_mul: activation {activation!r} (known: {sorted(GATE_ACTIVATIONS)})")
    rc = lib.act_mul(_ptr(gate_up), _c_int(ld), _ptr(out), _c_int(ldo), _c_int(T), _c_int(F), _c_int(DT[out.dtype]),
                     _c_int(GATE_ACTIVATIONS[activation]), _stream())
    build.check(lib, rc, "silu_mul")
    return out


def expert_rows(y, x, w_gate, w_up, w_down, idx, weight, top, act, accumulate=True):
    """``y (+)= sum over a token's picks of weight * expert(x)``, reading only the picked experts'
    weights (``w_gate``, ``w_up``: ``[experts, F, width]``, ``w_down``: ``[experts, width, F]``); a
    pick at or beyond the number of experts gives ``weight * x``.  ``act``: room for ``[tokens *
    top, F]`` of ``x``'s dtype."""
    lib = build.load("experts")
    ldx, ldy = _rows2d(x, "x"), _rows2d(y, "y")
    T, width = x.shape
    n_experts = 0 if w_gate is None else w_gate.shape[0]
    F = 1 if w_gate is None else w_gate.shape[1]
    _need(y.dtype == torch.float32 and tuple(y.shape) == (T, width) and x.dtype in DT, "expert_rows: x / y")
    if n_experts:
        for name, t, shape in (("w_gate", w_gate, (n_experts, F, width)), ("w_up", w_up, (n_experts, F, width)),
                               ("w_down", w_down, (n_experts, width, F))):
            _dev(t, name, x.dtype)
            _need(tuple(t.shape) == shape, f"expert_rows: {name} is {tuple(t.shape)}, want {shape}")
        _dev(act, "act", x.dtype)
        _need(act.numel() >= T * top * F, "expert_rows: act too small")
    _dev(idx, "idx", torch.int32)
    _dev(weight, "weight", torch.float32)
    _need(idx.numel() >= T * top and weight.numel() >= T * top, "expert_rows: idx / weight too short")
    rc = lib.expert_rows(_ptr(x), _c_int(ldx), _ptr(w_gate), _ptr(w_up), _ptr(w_down), _ptr(idx), _ptr(weight),
                         _c_int(T), _c_int(n_experts), _c_int(top), _c_int(F), _c_int(width), _ptr(act), _ptr(y),
                         _c_int(ldy), _c_int(int(bool(accumulate))), _c_int(DT[x.dtype]), _stream())
    build.check(lib, rc, "expert_rows")
    return y


def expert_tiles_takes(inner, width, dtype):
    """Whether ``expert_tiles`` takes experts of this inner size at this width."""
    return bool(build.load("experts").expert_tiles_takes(_c_int(inner), _c_int(width), _c_int(DT[dtype])))


def expert_tiles(y, x, w_gate, w_up, w_down, idx, weight, top, alloc, accumulate=True):
    """What ``expert_rows`` computes, for many tokens: the picks are sorted by expert on the device
    and every tile of up to 64 picks of one expert is a small product on the matrix cores.
    ``alloc(shape, dtype)`` gives the work memory (the sorted list, the tiles, the activations
    and a float32 row for every pick)."""
    lib = build.load("experts")
    ldx, ldy = _rows2d(x, "x"), _rows2d(y, "y")
    T, width = x.shape
    n_experts, F = w_gate.shape[0], w_gate.shape[1]
    _need(y.dtype == torch.float32 and tuple(y.shape) == (T, width) and x.dtype in DT, "expert_tiles: x / y")
    for name, t, shape in (("w_gate", w_gate, (n_experts, F, width)), ("w_up", w_up, (n_experts, F, width)),
                           ("w_down", w_down, (n_experts, width, F))):
        _dev(t, name, x.dtype)
        _need(tuple(t.shape) == shape, f"expert_tiles: {name} is {tuple(t.shape)}, want {shape}")
    _dev(idx, "idx", torch.int32)
    _dev(weight, "weight", torch.float32)
    _need(idx.numel() >= T * top and weight.numel() >= T * top, "expert_tiles: idx / weight too short")
    most = lib.expert_tiles_most(_c_int(T * top), _c_int(n_experts))
    order, tiles, n_tiles = alloc((T * top,), torch.int32), alloc((3 * most,), torch.int32), alloc((1,), torch.int32)
    act, out = alloc((T * top, F), x.dtype), alloc((T * top, width), torch.float32)
    rc = lib.expert_tiles(_ptr(x), _c_int(ldx), _ptr(w_gate), _ptr(w_up), _ptr(w_down), _ptr(idx), _ptr(weight), _c_int(T),
                          _c_int(n_experts), _c_int(top), _c_int(F), _c_int(width), _ptr(order), _ptr(tiles), _ptr(n_tiles),
                          _ptr(act), _ptr(out), _ptr(y), _c_int(ldy), _c_int(int(bool(accumulate))), _c_int(DT[x.dtype]),
                          _stream())
    build.check(lib, rc, "expert_tiles")
    return y


# ---------------------------------------------------------------------------
# a layer whose sublayers share one norm and whose outgoing stream is a sum over depth (csrc/parallel_block.hip)


class CanonArgs(ctypes.Structure):
    """Mirror of ``CanonArgs`` in csrc/parallel_block.hip."""

    _fields_ = [("w", _vp), ("taps", _c_int), ("state", _vp), ("state_stride", _c_size_t), ("state_offset", _c_size_t),
                ("token_req", _vp), ("seq_start", _vp), ("slot_ids", _vp), ("mixed", _vp)]


class InputConvolution:
    """A causal convolution over time on a mixer's input, added to it: ``m_t = h_t + sum_j weight[:, j]
    h_(t - taps + 1 + j)`` per channel over a request's own rows (``weight`` float32 ``[width, taps]``);
    rows of earlier steps come from the request's row of ``state`` (``[taps - 1, width]`` from
    ``offset`` on, the latest last).  ``mixed``: where ``m`` goes, ``[rows, width]`` in the compute dtype."""

    def __init__(self, weight, state, offset, token_req, seq_start, slot_ids, mixed):
        _dev(weight, "weight", torch.float32)
        _dev(state, "state", torch.float32)
        for name, t in (("token_req", token_req), ("seq_start", seq_start), ("slot_ids", slot_ids)):
            _dev(t, name, torch.int32)
        width, taps = weight.shape
        _need(state.dim() == 2 and offset + (taps - 1) * width <= state.shape[1], "a convolution's state rows hold taps - 1 inputs of every channel")
        _need(mixed.is_contiguous() and mixed.dtype in DT and mixed.shape[1] == width and token_req.numel() >= mixed.shape[0],
              "the convolution's output is contiguous [rows, width]")
        self.mixed, self.width = mixed, width
        self._keep = (weight, state, token_req, seq_start, slot_ids)
        c = self.c = CanonArgs()
        c.w, c.taps, c.state, c.state_stride, c.state_offset = weight.data_ptr(), taps, state.data_ptr(), state.stride(0), int(offset)
        c.token_req, c.seq_start, c.slot_ids, c.mixed = token_req.data_ptr(), seq_start.data_ptr(), slot_ids.data_ptr(), mixed.data_ptr()


CANON_FUSED_MAX_WIDTH = 8192  # up to this width the norm's kernel keeps a row in registers and can run the convolution too


def canon_rows(h, canon):
    """``canon`` (an ``InputConvolution``) over the float32 rows ``h`` of a step of any shape; the
    requests' state rows are not touched (``conv_state_update`` keeps the last inputs afterwards)."""
    lib = build.load("parallel_block")
    _dev(h, "h", torch.float32)
    _need(h.dim() == 2 and h.shape[1] == canon.width and h.shape[0] >= canon.mixed.shape[0], "canon_rows: shapes")
    rc = lib.canon_rows(_ptr(h), _c_int(canon.mixed.shape[0]), _c_int(canon.width), _c_int(DT[canon.mixed.dtype]),
                        ctypes.byref(canon.c), _stream())
    build.check(lib, rc, "canon_rows")
    return canon.mixed


def norm_fanout(out, x, weight, eps, out32=None, copy_a=None, copy_b=None, canon=None):
    """``out = x / sqrt(mean(x^2) + eps) * weight`` over the float32 rows ``x`` (``out``: float32 or
    bfloat16, contiguous); the same as float32 into ``out32``, and ``x`` itself into ``copy_a`` and
    ``copy_b`` (contiguous float32 ``[rows, width]``), each where given.  ``canon`` (an
    ``InputConvolution``, for a step in which every request brings one token): the convolution runs
    here too, and every request's state row moves up by one."""
    lib = build.load("parallel_block")
    n, width = out.shape
    ldx = _f32_rows(x, "x", width)
    _dev(weight, "weight", torch.float32)
    _need(out.is_contiguous() and out.dtype in DT and weight.numel() == width and x.shape[0] >= n, "norm_fanout: shapes")
    for name, t in (("out32", out32), ("copy_a", copy_a), ("copy_b", copy_b)):
        if t is not None:
            _dev(t, name, torch.float32)
            _need(t.is_contiguous() and tuple(t.shape) == (n, width), f"norm_fanout: {name} is contiguous [rows, width]")
    if canon is not None:
        _need(canon.width == width and canon.mixed.shape[0] == n and canon.mixed.dtype == out.dtype and width <= CANON_FUSED_MAX_WIDTH,
              "norm_fanout: the convolution's rows are the norm's")
    rc = lib.norm_fanout(_ptr(x), _c_int(ldx), _ptr(weight), _c_float(eps), _c_int(n), _c_int(width), _ptr(out),
                         _c_int(DT[out.dtype]), _ptr(out32), _ptr(copy_a), _ptr(copy_b),
                         ctypes.byref(canon.c) if canon is not None else None, _stream())
    build.check(lib, rc, "norm_fanout")
    return out


def depth_average(out, kept, weights, n):
    """``out[t] = sum over j < n of weights[j] * kept[j, t]``: ``kept`` float32 ``[>= n, rows, width]``,
    ``weights`` float32 on the device, ``out`` contiguous float32 ``[rows, width]``."""
    lib = build.load("parallel_block")
    _dev(out, "out", torch.float32)
    _dev(kept, "kept", torch.float32)
    _dev(weights, "weights", torch.float32)
    _need(kept.dim() == 3 and kept.shape[0] >= n and kept.is_contiguous() and out.is_contiguous()
          and tuple(kept.shape[1:]) == tuple(out.shape) and weights.numel() >= n, "depth_average: shapes")
    rc = lib.depth_average(_ptr(out), _ptr(kept), _c_size_t(kept.stride(0)), _ptr(weights), _c_int(n), _c_int(out.shape[0]),
                           _c_int(out.shape[1]), _stream())
    build.check(lib, rc, "depth_average")
    return out


# ---------------------------------------------------------------------------
# between a projection's float rows and a recurrence, and behind it (csrc/state_gates.hip)


def silu_columns(u, col, n):
    """``u[:, col:col + n] <- silu(...)`` in place on float32 rows."""
    lib = build.load("state_gates")
    ld = _f32_rows(u, "u", col + n)
    rc = lib.silu_columns(_ptr(u), _c_int(ld), _c_int(u.shape[0]), _c_int(col), _c_int(n), _stream())
    build.check(lib, rc, "silu_columns")
    return u


def forget_gate(u, q_col, z_col, n, lower, keys):
    """A forget gate with a floor, ``f = lower + (1 - lower) * sigmoid(z)``, for ``S <- diag(f) S +
    (1 - f) v^T``: the logits ``u[:, z_col:z_col + n]`` become ``log f`` in place, ``1 - f`` goes to
    ``keys`` (float32 ``[rows, >= n]``), and the queries ``u[:, q_col:q_col + n]`` pass a silu in place."""
    lib = build.load("state_gates")
    ld, ldk = _f32_rows(u, "u", max(q_col, z_col) + n), _f32_rows(keys, "keys", n)
    _dev(lower, "lower", torch.float32)
    _need(lower.numel() == n and keys.shape[0] >= u.shape[0], "forget_gate: a floor a channel, a row of keys a row")
    rc = lib.forget_gate(_ptr(u), _c_int(ld), _c_int(u.shape[0]), _c_int(q_col), _c_int(z_col), _c_int(n), _ptr(lower),
                         _ptr(keys), _c_int(ldk), _stream())
    build.check(lib, rc, "forget_gate")
    return keys


def normed_gate(out, y, gate, weight, eps):
    """``out = y / sqrt(mean(y^2) + eps) * weight * sigmoid(gate)`` over whole float32 rows; ``out``
    float32 or bfloat16 ``[rows, width]`` (its rows may be wider apart)."""
    lib = build.load("state_gates")
    n, width = out.shape
    ldy, ldg, ldo = _f32_rows(y, "y", width), _f32_rows(gate, "gate", width), _rows2d(out, "out")
    _dev(weight, "weight", torch.float32)
    _need(out.dtype in DT and weight.numel() == width and y.shape[0] >= n and gate.shape[0] >= n, "normed_gate: shapes")
    rc = lib.normed_gate(_ptr(y), _c_int(ldy), _ptr(gate), _c_int(ldg), _ptr(weight), _c_float(eps), _c_int(n), _c_int(width),
                         _ptr(out), _c_int(ldo), _c_int(DT[out.dtype]), _stream())
    build.check(lib, rc, "normed_gate")
    return out
