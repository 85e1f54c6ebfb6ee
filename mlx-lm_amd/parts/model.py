"""A decoder-only model built from a plan: embedding, scheduled layers, final norm, head."""

import ctypes

from ..config.plan import CacheNeed, ModelPlan, StateNeed
from ..ops import native
from .base import BLOCKS, EMBEDDINGS, FAMILIES, HEADS, NORMS, POSITION_ENCODINGS, build_part


class DecoderModel:
    """The parts a ``ModelPlan`` names, and the forward pass over one step's tokens.

    The order of the reference's forward (mlx_lm/models/gpt2.py:125-151,
    161-168): embeddings, the layers, final norm, head; except that the norm
    and the head run only on the rows whose logits are wanted, and that the
    order of layers is the plan's schedule.
    """

    _native = None

    def __init__(self, plan: ModelPlan):
        self.plan = plan.validate()
        self.width, self.vocab_size = plan.width, plan.vocab_size
        self.max_positions = plan.max_positions
        self.embedding = build_part(EMBEDDINGS, "embedding", plan.embedding)
        self.embedding_positions = (
            build_part(POSITION_ENCODINGS, "position encoding", plan.embedding_positions)
            if plan.embedding_positions is not None
            else None
        )
        self.layers = []
        for spec in plan.layers:
            if spec.arrangement not in BLOCKS:
                raise ValueError(
                    f"unknown block arrangement '{spec.arrangement}' (known: {sorted(BLOCKS)})"
                )
            cls = BLOCKS[spec.arrangement]
            if set(spec.parts) != set(cls.PARTS):
                raise ValueError(
                    f"arrangement '{spec.arrangement}' arranges {sorted(cls.PARTS)}, the plan gives {sorted(spec.parts)}"
                )
            built = {name: build_part(*FAMILIES[cls.PARTS[name]], part_spec) for name, part_spec in spec.parts.items()}
            self.layers.append(cls(**built))
        self.schedule = list(plan.schedule)
        self.final_norm = build_part(NORMS, "norm", plan.final_norm)
        self.head = build_part(HEADS, "output head", plan.head)
        self._native = None

    # -- tensors ------------------------------------------------------------

    def parts(self):
        yield self.embedding
        if self.embedding_positions is not None:
            yield self.embedding_positions
        for block in self.layers:
            yield from block.parts()
        yield self.final_norm
        yield self.head

    def expected_tensors(self):
        """Every tensor the model wants, by full name.  A name may be wanted by
        two parts (a tied head) if they agree on shape and role."""
        want = {}
        for part in self.parts():
            for name, spec in part.tensors().items():
                if name in want and want[name] != spec:
                    raise ValueError(f"tensor '{name}' is wanted as {want[name]} and as {spec}")
                want[name] = spec
        return want

    def load_tensors(self, tensors):
        """Hand every part its device tensors.  The native twins keep the tensors' addresses, and
        so do the steps an engine has recorded: once a twin exists, other weights need a new model."""
        if self._native is not None or any(p._native is not None for p in self.parts()):
            raise RuntimeError(
                "this model has run (its native parts and recorded steps hold the addresses of its "
                "weights): build a new model to load other weights")
        for part in self.parts():
            part.load(tensors)

    def bytes_read_per_step(self, dtype_size):
        """Bytes of the tensors that a step reads whole, each counted once.  A table that a part
        reads row by row (``reads_rows_of()`` names it: an embedding, a position table) does not
        count unless another part reads all of it (a tied head does)."""
        whole, by_rows = {}, {}
        for part in self.parts():
            rows = set(part.reads_rows_of()) if hasattr(part, "reads_rows_of") else set()
            for name, spec in part.tensors().items():
                (by_rows if name in rows else whole)[name] = spec
        total = 0
        for spec in whole.values():
            n = 1
            for s in spec.shape:
                n *= s
            total += n * (dtype_size if spec.role == "matrix" else 4)
        return total

    # -- cache ---------------------------------------------------------------

    def cache_needs(self):
        """What each cache slot has to hold, from the mixer of the run that writes it."""
        needs = {}
        for run in self.schedule:
            need = self.layers[run.layer].cache_need()
            if run.writes_cache:
                needs[run.cache] = need
            elif needs[run.cache] != need:
                raise ValueError(
                    f"layer {run.layer} reads cache slot {run.cache} but wants {need}, "
                    f"the slot holds {needs[run.cache]}"
                )
        out = [needs[i] for i in range(len(needs))]
        for need in out:
            if need is not None and not isinstance(need, (CacheNeed, StateNeed)):
                raise TypeError(f"cache_need() must give a CacheNeed, a StateNeed or None, got {need!r}")
        return out

    # -- the step arrays that parts ask for ------------------------------------

    def array_providers(self):
        """``[(first array id, key, names, function of a HostBatch)]``: one entry for each kind of
        part that declared ``step_arrays`` (parts that share a key share the arrays)."""
        seen, out = set(), []
        for part in self.parts():
            key = getattr(part, "step_arrays_key", None)
            if key is None or key in seen:
                continue
            seen.add(key)
            names = tuple(part.step_array_names)
            out.append((native.array_ids(key, names), key, names, part.step_arrays))
        return out

    # -- forward -------------------------------------------------------------

    def native(self):
        """The native model: the tree of the parts' native twins (made at first use, after ``load``)."""
        if self._native is None:
            L = native.lib()
            layers = (ctypes.c_void_p * len(self.layers))(*[b.native() for b in self.layers])
            n = len(self.schedule)
            ints = ctypes.c_int * n
            self._native = native.made(L.eng_make_model(
                self.width, self.vocab_size, self.embedding.native(),
                self.embedding_positions.native() if self.embedding_positions is not None else None,
                len(self.layers), layers, n, ints(*[r.layer for r in self.schedule]),
                ints(*[r.cache for r in self.schedule]), ints(*[int(r.writes_cache) for r in self.schedule]),
                self.final_norm.native(), self.head.native()), "model")
        return self._native

    def __del__(self):
        handle, self._native = self._native, None
        if handle:
            try:
                native.lib().eng_free(handle)
            except Exception:  # noqa: BLE001 (the interpreter may be shutting down)
                pass

    def forward(self, ctx):
        """Run the step's tokens; returns float32 logits ``[n_wanted, vocab]`` or ``None``.

        One call into the native host, which walks the parts: embedding (+ position term),
        the scheduled blocks, the final norm on the wanted rows only, the head."""
        logits = None
        if ctx.n_wanted:
            logits = ctx.logits_out(ctx.n_wanted, self.vocab_size)
            ctx.c.logits, ctx.c.logits_rows = logits.data_ptr(), logits.shape[0]
        with ctx.enter():
            rc = native.lib().eng_model_forward(self.native(), ctypes.byref(ctx.c))
        native.check(rc, "the model's step")
        return logits
