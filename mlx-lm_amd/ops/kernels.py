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


def embed_gather_add(out, table, ids, add_table=None, add_ids=None):
    """``out[t] = table[ids[t]] (+ add_table[add_ids[t]])`` into float32 ``out``."""
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
    rc = lib.embed_gather_add(
        _ptr(out), _ptr(table), _ptr(ids), _ptr(add_table), _ptr(add_ids),
        _c_int(n), _c_int(width), _c_int(DT[table.dtype]), _stream(),
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
    """The LayerNorm of float32 rows, not computed yet.

    ``linear`` takes it as its input and, where its kernel can, norms the rows
    itself while the first weights are on their way; anything else calls
    ``materialize()`` and gets the tensor.
    """

    def __init__(self, alloc, x, gamma, beta, eps, dtype):
        self.alloc, self.x, self.gamma, self.beta, self.eps, self.dtype = alloc, x, gamma, beta, eps, dtype
        self.shape = tuple(x.shape)
        self._out = None

    def materialize(self):
        if self._out is None:
            self._out = self.alloc(self.shape, self.dtype)
            layernorm(self._out, self.x, self.gamma, self.beta, self.eps)
        return self._out


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


def linear(out, a, w, bias=None, gelu=False, accumulate=False, variant=0, scatter=None, splits=None,
           pending=None):
    """``out = epilogue(a @ w.T + bias)``.

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
        call.a.lazy, call.a.ldx = 1, a.x.stride(0)
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
    call.gelu, call.accumulate, call.variant, call.splits = int(gelu), int(accumulate), int(variant), int(splits or 0)
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


def attn_tile(out, q, kv, block_table, token_req, positions, tiles, n_tiles, n_heads, scale, window=0):
    """Attention for tiles of up to 16 consecutive queries of one request each.

    ``tiles`` is int32 ``[n_tiles, 2]``: first flat row and number of rows.
    """
    lib = build.load("attention")
    ldq, ldo = _rows2d(q, "q"), _rows2d(out, "out")
    _need(q.shape[1] == n_heads * kv.head_dim, "attn_tile: q width must be n_heads*head_dim")
    _need(out.shape[1] == n_heads * kv.head_dim and out.dtype == q.dtype, "attn_tile: out shape/dtype")
    _attn_common(q, kv, block_table, token_req, positions)
    _dev(tiles, "tiles", torch.int32)
    _need(tiles.numel() >= 2 * n_tiles, "attn_tile: tile list too short")
    rc = lib.attn_tile(
        _ptr(out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(tiles), _c_int(n_tiles), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), _c_int(DT[q.dtype]), _stream(),
    )
    build.check(lib, rc, "attn_tile")
    return out


ATTN_ROW_MAX_HEAD_DIM = 144  # beyond this the per-wave key tiles do not fit in LDS


def attn_row(out, q, kv, block_table, token_req, positions, rows, n_rows, n_heads, scale,
             window=0, n_splits=1, part_o=None, part_ml=None):
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
    rc = lib.attn_row(
        _ptr(out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(rows), _c_int(n_rows), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), _c_int(n_splits), _ptr(part_o), _ptr(part_ml), _c_int(DT[q.dtype]),
        _stream(),
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
    return q_dtype == torch.bfloat16 and kv.head_dim in (32, 64, 128)


def attn_prefill(out, q, kv, block_table, token_req, positions, tiles, n_tiles, n_heads, scale, window=0):
    """``attn_tile`` on the matrix cores: bfloat16, head_dim 32/64/128, tiles of up to 128 queries."""
    lib = build.load("attention_prefill")
    ldq, ldo = _rows2d(q, "q"), _rows2d(out, "out")
    _need(q.dtype == torch.bfloat16, "attn_prefill: bfloat16 only")
    _need(q.shape[1] == n_heads * kv.head_dim, "attn_prefill: q width must be n_heads*head_dim")
    _need(out.shape[1] == n_heads * kv.head_dim and out.dtype == q.dtype, "attn_prefill: out shape/dtype")
    _attn_common(q, kv, block_table, token_req, positions)
    _dev(tiles, "tiles", torch.int32)
    _need(tiles.numel() >= 2 * n_tiles, "attn_prefill: tile list too short")
    rc = lib.attn_prefill(
        _ptr(out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(tiles), _c_int(n_tiles), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), _stream(),
    )
    build.check(lib, rc, "attn_prefill")
    return out


def attn_decode_takes(q_dtype, kv):
    """Whether the register-streaming decode kernel takes this cache geometry."""
    if q_dtype not in (torch.bfloat16, torch.float32):
        return False
    key_bytes = kv.head_dim * q_dtype.itemsize
    return key_bytes in (64, 128, 256) and kv.page_size % (1024 // key_bytes) == 0


def attn_decode(out, q, kv, block_table, token_req, positions, rows, n_rows, n_heads, scale,
                window=0, n_splits=1, part_o=None, part_ml=None, n_waves=4, ahead=None, ahead_chunks=0,
                rows_are_requests=False, key_tile=32, join_in_kernel=0):
    """``attn_row`` for keys of 64, 128 or 256 bytes (bfloat16 with head_dim 32, 64 or 128, float32
    with 16, 32 or 64): keys stream into registers.

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
    rc = lib.attn_decode_rows(
        _ptr(out.data if packed_out else out), _ptr(q), _c_int(ldq), _c_int(ldo), _ptr(kv.k), _ptr(kv.v),
        _c_size_t(kv.page_stride), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(token_req), _ptr(positions), _ptr(rows), _c_int(n_rows), _c_int(n_heads),
        _c_int(kv.n_kv_heads), _c_int(kv.head_dim), _c_int(kv.page_size), _c_int(window),
        _c_float(scale), _c_int(n_splits), _ptr(part_o), _ptr(part_ml), _c_int(n_waves),
        _ptr(ahead.packed if ahead is not None else None),
        _c_size_t(ahead.chunk_bytes if ahead is not None else 0),
        _c_int(min(ahead_chunks, ahead.n_chunks) if ahead is not None else 0),
        _c_int(1 if rows_are_requests else 0), _c_int(DT[q.dtype]), _c_int(key_tile),
        _c_int(int(join_in_kernel)), _stream(),
    )
    build.check(lib, rc, "attn_decode")
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
