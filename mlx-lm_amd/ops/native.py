"""The Python face of the native host (``csrc/engine.hip``): struct layouts, the library, the
two hooks it calls back through.

The native side walks a model's parts and issues a step's launches from one call.  Python
describes: every built-in part makes its native twin from its sizes, constants and device
pointers; a part that exists only in Python is wrapped as a *callback part*, and the native
walk calls its ``forward`` where its turn comes.  The hooks: ``_resolve`` loads (and, where
needed, builds) a kernel library when the native side first asks for one of its entry points;
``_callback`` runs a Python part's method, or grows the scratch buffer.
"""

import ctypes
import weakref
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int, c_long, c_size_t, c_void_p

import torch

from . import build

MAX_ARRAYS = 32
MAX_GROUPS = 8

DT = {torch.float32: 0, torch.bfloat16: 1, torch.int32: 2}
TORCH_DT = {0: torch.float32, 1: torch.bfloat16, 2: torch.int32}

# kinds of part and callback methods (csrc/engine.h)
NORM, MIXER, FFN, BLOCK, POSITION, EMBEDDING, HEAD, MODEL = range(1, 9)
CB_NORM, CB_MIXER, CB_FFN, CB_BLOCK, CB_ROTATE, CB_EMBEDDING_TERM, CB_EMBEDDING, CB_HEAD, CB_GROW = range(1, 10)
ACCEPTS_LAZY, SETTLES_PENDING, HANDLES_PENDING, READS_AHEAD = 1, 2, 4, 8


class EngMat(Structure):
    _fields_ = [("p", c_void_p), ("rows", c_int), ("cols", c_int), ("ld", c_int), ("dtype", c_int)]


class EngWeight(Structure):
    _fields_ = [("w", c_void_p), ("packed", c_void_p), ("N", c_int), ("K", c_int), ("ldw", c_int),
                ("dtype", c_int), ("chunk_bytes", c_size_t), ("n_chunks", c_int), ("pad_", c_int)]


class EngValue(Structure):
    _fields_ = [("m", EngMat), ("lazy", c_int), ("ldx", c_int), ("x", c_void_p), ("gamma", c_void_p),
                ("beta", c_void_p), ("eps", c_float), ("packed", c_int)]


class EngPending(Structure):
    _fields_ = [("target", c_void_p), ("rows", c_int), ("cols", c_int), ("ld", c_int), ("n_splits", c_int),
                ("ws", c_void_p), ("bias", c_void_p), ("allowed", c_int), ("pad_", c_int)]


class EngSlot(Structure):
    _fields_ = [("k", c_void_p), ("v", c_void_p), ("page_stride", c_size_t), ("v_page_stride", c_size_t),
                ("n_kv_heads", c_int), ("head_dim", c_int), ("page_size", c_int), ("dtype", c_int),
                ("group", c_int), ("v_head_dim", c_int)]


class EngScratch(Structure):
    _fields_ = [("base", c_void_p), ("size", c_size_t), ("offset", c_size_t), ("peak", c_size_t),
                ("frozen", c_int), ("pad_", c_int)]


class EngStats(Structure):
    _fields_ = [("launches", c_long), ("settle_normed", c_long), ("settle_plain", c_long),
                ("callbacks", c_long), ("steps", c_long), ("key_splits_most", c_long)]


class EngCtx(Structure):
    _fields_ = [
        ("stream", c_void_p), ("dtype", c_int), ("n_tokens", c_int), ("n_requests", c_int),
        ("n_wanted", c_int), ("wants_every_row", c_int), ("force_splits", c_int),
        ("token_ids", c_void_p), ("positions", c_void_p), ("token_req", c_void_p),
        ("wanted_rows", c_void_p), ("slot_ids", c_void_p),
        ("arrays", c_void_p * MAX_ARRAYS), ("counts", c_long * MAX_ARRAYS),
        ("block_tables", c_void_p * MAX_GROUPS), ("table_width", c_int * MAX_GROUPS),
        ("slots", POINTER(EngSlot)), ("n_slots", c_int), ("n_compute_units", c_int),
        ("scratch", POINTER(EngScratch)), ("split_ws", c_void_p), ("split_ws_floats", c_size_t),
        ("logits", c_void_p), ("logits_rows", c_long), ("pending", EngPending),
        ("read_ahead", POINTER(EngWeight)), ("stats", POINTER(EngStats)), ("py", c_void_p),
    ]


class EngCall(Structure):
    _fields_ = [("x", EngMat), ("residual", EngMat), ("out", EngMat), ("q", EngMat), ("k", EngMat),
                ("rows", c_void_p), ("n_rows", c_int), ("cache_slot", c_int), ("writes_cache", c_int),
                ("lazy", c_int), ("result", EngMat), ("index", c_void_p), ("nbytes", c_size_t)]


class EngScatter(Structure):
    _fields_ = [("k", c_void_p), ("v", c_void_p), ("page_stride", c_size_t), ("n_kv_heads", c_int),
                ("head_dim", c_int), ("page_size", c_int), ("dtype", c_int), ("block_table", c_void_p),
                ("token_req", c_void_p), ("positions", c_void_p), ("max_blocks", c_int), ("q_width", c_int),
                ("kv_width", c_int), ("pad_", c_int)]


class EngLinear(Structure):
    _fields_ = [("out", EngMat), ("a", EngValue), ("w", EngWeight), ("bias", c_void_p),
                ("scatter", POINTER(EngScatter)), ("gelu", c_int), ("accumulate", c_int), ("variant", c_int),
                ("splits", c_int), ("out_packed", c_int), ("pad_", c_int)]


_RESOLVER = ctypes.CFUNCTYPE(c_void_p, c_char_p, c_char_p)
_CALLBACK = ctypes.CFUNCTYPE(c_int, c_int, c_int, POINTER(EngCtx), POINTER(EngCall))

_lib = None
_hooks = None  # the two callback objects, kept alive
_raised = []  # an exception a hook caught, to be raised again where the native call returns
_py_parts = weakref.WeakValueDictionary()  # id -> part, for callback parts
_next_id = [1]
_running = []  # the StepContext of each native call in progress, innermost last


class NativeError(RuntimeError, ValueError):
    """The native host refused a call; the text says which check failed.  (Both a refused
    value and a failed launch come back this way, hence both bases.)"""


def _resolve(lib_name, symbol):
    try:
        handle = build.load(lib_name.decode())
        return ctypes.cast(getattr(handle, symbol.decode()), c_void_p).value
    except BaseException as e:  # noqa: BLE001 (raised again by check())
        _raised.append(e)
        return None


def _callback(part_id, method, cctx, call):
    try:
        ctx = _running[-1]
        if method == CB_GROW:
            ctx._scratch.grow(call.contents.nbytes)
            return 0
        part = _py_parts[part_id]
        run_python_part(part, method, ctx, call.contents)
        return 0
    except BaseException as e:  # noqa: BLE001
        _raised.append(e)
        return 1


def lib():
    """The native library, loaded (and built) at first use, with its hooks set."""
    global _lib, _hooks
    if _lib is not None:
        return _lib
    L = build.load("engine")
    P = c_void_p
    sig = {
        "eng_set_hooks": (None, [_RESOLVER, _CALLBACK]),
        "eng_compute_units": (c_int, []),
        "eng_make_callback": (P, [c_int, c_int, c_int]),
        "eng_make_layernorm": (P, [c_int, c_float, P, P]),
        "eng_make_attention": (P, [c_int, c_int, c_int, c_int, c_float, c_int, POINTER(EngWeight), P,
                                   POINTER(EngWeight), P, P, c_int]),
        "eng_make_gelu_mlp": (P, [c_int, c_int, POINTER(EngWeight), P, POINTER(EngWeight), P]),
        "eng_make_pre_norm_block": (P, [P, P, P, P]),
        "eng_make_token_embedding": (P, [P, c_int, c_int, c_int]),
        "eng_make_learned_positions": (P, [P, c_int, c_int, c_int]),
        "eng_make_linear_head": (P, [POINTER(EngWeight)]),
        "eng_make_model": (P, [c_int, c_int, P, P, c_int, POINTER(P), c_int, POINTER(c_int), POINTER(c_int),
                               POINTER(c_int), P, P]),
        "eng_free": (None, [P]),
        "eng_model_forward": (c_int, [P, POINTER(EngCtx)]),
        "eng_block_forward": (c_int, [P, POINTER(EngCtx), POINTER(EngMat), c_int, c_int]),
        "eng_norm_forward": (c_int, [P, POINTER(EngCtx), POINTER(EngMat), P, c_int, c_int, POINTER(EngWeight),
                                     POINTER(EngValue)]),
        "eng_mixer_forward": (c_int, [P, POINTER(EngCtx), POINTER(EngValue), POINTER(EngMat), c_int, c_int]),
        "eng_ffn_forward": (c_int, [P, POINTER(EngCtx), POINTER(EngValue), POINTER(EngMat)]),
        "eng_embedding_forward": (c_int, [P, POINTER(EngCtx), POINTER(EngMat), P]),
        "eng_head_forward": (c_int, [P, POINTER(EngCtx), POINTER(EngValue), POINTER(EngMat)]),
        "eng_settle": (c_int, [POINTER(EngCtx)]),
        "eng_linear": (c_int, [POINTER(EngCtx), POINTER(EngLinear), POINTER(EngPending)]),
        "eng_linear_norms_itself": (c_int, [POINTER(EngCtx), c_int, c_int, c_int, c_int, c_int]),
        "eng_pending_settle": (c_int, [POINTER(EngCtx), POINTER(EngPending)]),
        "eng_pending_can_norm": (c_int, [POINTER(EngPending), POINTER(EngMat)]),
        "eng_pending_settle_normed": (c_int, [POINTER(EngCtx), POINTER(EngPending), POINTER(EngMat), P, P,
                                              c_float, POINTER(EngWeight), c_int]),
        "eng_read_ahead_pays": (c_int, [POINTER(EngCtx), POINTER(EngWeight), c_int, c_int]),
        "eng_wants_packed_rows": (c_int, [POINTER(EngCtx), POINTER(EngWeight), c_int]),
        "eng_host": (P, []),
        "eng_attn_tile_sizes": (None, [POINTER(c_int), POINTER(c_int)]),
        "eng_rows_split_from": (c_int, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    mirrored = [EngMat, EngWeight, EngValue, EngPending, EngSlot, EngScratch, EngStats, EngCtx, EngCall,
                EngScatter, EngLinear]
    want = [ctypes.sizeof(t) for t in mirrored] + [EngCtx.pending.offset, EngCall.nbytes.offset]
    got = (c_long * len(want))()
    L.eng_struct_sizes.argtypes = [POINTER(c_long), c_int]
    if L.eng_struct_sizes(got, len(want)) != len(want) or list(got) != want:
        raise build.ExtensionError(f"struct layouts of csrc/engine.h and ops/native.py differ: {list(got)} and {want}")
    _hooks = (_RESOLVER(_resolve), _CALLBACK(_callback))
    L.eng_set_hooks(*_hooks)
    _lib = L
    return L


def check(rc, what="the native host"):
    """Raise what a native call reported: a hook's own exception first, else the library's text."""
    if _raised:
        e = _raised.pop()
        _raised.clear()
        raise e
    if rc != 0:
        raise NativeError(lib().mlxlm_last_error().decode() or f"{what} failed")


def host():
    """The host's table of routines (``EngHost`` of csrc/engine.h), for the maker of a native part
    that lives in a library of its own (csrc/engine_parts.h)."""
    return lib().eng_host()


def made(handle, what):
    """A handle that an ``eng_make_*`` call returned, or its error."""
    if not handle:
        check(1, what)
    return handle


class running:
    """``with running(ctx):`` around a native call that may call Python parts back."""

    def __init__(self, ctx):
        self.ctx = ctx

    def __enter__(self):
        _running.append(self.ctx)
        return self.ctx

    def __exit__(self, *exc):
        _running.pop()
        return False


# ---------------------------------------------------------------------------
# tensors <-> structs


def mat(t):
    """An ``EngMat`` over a 2-D device tensor with contiguous rows (1-D: one row)."""
    if t.dim() == 1:
        t = t[None]
    if t.dim() != 2 or t.stride(1) != 1 or not t.is_cuda:
        raise ValueError("a 2-D GPU tensor with contiguous rows is needed")
    if t.dtype not in DT:
        raise ValueError(f"dtype {t.dtype} is not supported")
    return EngMat(t.data_ptr(), t.shape[0], t.shape[1], t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1]),
                  DT[t.dtype])


def ptr(t):
    return t.data_ptr() if t is not None else None


def register_python_part(part):
    """An id under which the native side can call ``part`` back."""
    pid = _next_id[0]
    _next_id[0] += 1
    _py_parts[pid] = part
    return pid


_array_ids = {}


def array_ids(key, names):
    """The first of ``len(names)`` consecutive ids for a part kind's own step arrays.

    Ids are handed out once per ``key`` for the life of the process; the packer puts array
    ``names[i]`` of that kind at ``EngCtx.arrays[base + i]``."""
    if key in _array_ids:
        base, known = _array_ids[key]
        if list(known) != list(names):
            raise ValueError(f"step arrays of '{key}' were registered as {known}, now {list(names)}")
        return base
    base = sum(len(n) for _, n in _array_ids.values())
    if base + len(names) > MAX_ARRAYS:
        raise ValueError(f"no room for the {len(names)} step arrays of '{key}' (at most {MAX_ARRAYS} in all)")
    _array_ids[key] = (base, list(names))
    return base


def run_python_part(part, method, ctx, call):
    """A callback part's turn: build tensors over the native side's matrices, call the method."""
    T = ctx.tensor
    if method == CB_MIXER:
        part.forward(ctx, T(call.x), T(call.residual), ctx.cache_view(call.cache_slot), bool(call.writes_cache))
    elif method == CB_FFN:
        part.forward(ctx, T(call.x), T(call.residual))
    elif method == CB_BLOCK:
        part.forward(ctx, T(call.residual), ctx.cache_view(call.cache_slot), bool(call.writes_cache))
    elif method == CB_NORM:
        x = T(call.x)
        if call.rows:
            rows = ctx.int_array(call.rows, call.n_rows)
            out = part.forward(ctx, x, rows=rows, n_rows=call.n_rows)
        else:
            out = part.forward(ctx, x)
        if not isinstance(out, torch.Tensor):
            out = out.materialize()
        ctx.keep(out)
        call.result = mat(out)
    elif method == CB_ROTATE:
        part.rotate(ctx, T(call.q), T(call.k))
    elif method == CB_EMBEDDING_TERM:
        term = part.embedding_term(ctx)
        if term is not None:
            table, index = term
            ctx.keep(table, index)
            call.result = mat(table)
            call.index = index.data_ptr()
    elif method == CB_EMBEDDING:
        add = None
        if call.result.p:
            add = (ctx.tensor(call.result), ctx.int_array(call.index, call.out.rows))
        part.forward(ctx, T(call.out), add)
    elif method == CB_HEAD:
        part.forward(ctx, T(call.x), T(call.out))
    else:
        raise ValueError(f"unknown callback method {method}")
