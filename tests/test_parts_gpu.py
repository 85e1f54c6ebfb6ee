"""Each part alone against the plain implementation, and toy parts defined here
that are registered, built and stepped without touching the framework's files."""

import json
import os
from dataclasses import dataclass

import pytest
import torch

import helpers
import plain_gpt2 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {"float32": 2e-5, "bfloat16": 2.5e-2}


def _close(got, want, dtype, what=""):
    scale = max(want.abs().max().item(), 1e-6)
    err = (got.double().cpu() - want).abs().max().item()
    assert err <= TOL[dtype] * scale, f"{what}: max error {err:.3e} against scale {scale:.3e}"


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("partsB"))
    config, weights = helpers.make_folder(d, "B", 8.0)
    return d, config, weights


def _engine(folder, dtype, n_pages=32):
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.utils import load_model

    model, _ = load_model(folder, dtype=dtype)
    return Engine(model, dtype=dtype, page_size=16, n_pages=n_pages, max_requests=4)


def _context(engine, entries):
    """Pages and a step context for ``entries`` without running the model."""
    for e in entries:
        if not engine.has_request(e.request_id):
            engine.add_request(e.request_id)
        engine.cache.reserve(e.request_id, len(e.tokens))
    ctx = engine._build_context(entries)
    engine.scratch.reset()
    return ctx


def _commit(engine, entries):
    for e in entries:
        engine.cache.commit(e.request_id, len(e.tokens))


def _w(weights, dtype):
    w = helpers.round_matrices_to_bf16(weights) if dtype == "bfloat16" else weights
    return {k: v.double() for k, v in w.items()}


def _act(x, dtype):
    return x.to(torch.bfloat16 if dtype == "bfloat16" else torch.float32).to(DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_parts_alone(folder_b, dtype):
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = folder_b
    w = _w(weights, dtype)
    eng = _engine(folder, dtype)
    dec = eng.decoder
    D, H, V = config["n_embd"], config["n_head"], config["vocab_size"]
    eps = config["layer_norm_epsilon"]
    g = torch.Generator().manual_seed(1)

    # embedding with learned positions, the second request starting at position 30
    first = [StepEntry("b", helpers.random_tokens(30, V, 2), [])]
    ctx = _context(eng, first)
    _commit(eng, first)
    toks_a, toks_b = helpers.random_tokens(21, V, 3), helpers.random_tokens(5, V, 4)
    entries = [StepEntry("a", toks_a, [0, 20]), StepEntry("b", toks_b, [4])]
    ctx = _context(eng, entries)
    h = ctx.scratch((26, D), "float32")
    dec.embedding.forward(ctx, h, dec.embedding_positions.embedding_term(ctx))
    want = torch.cat([
        plain.add_learned_positions(plain.embed_tokens(w["model.wte.weight"], torch.tensor(toks_a)), w["model.wpe.weight"], 0),
        plain.add_learned_positions(plain.embed_tokens(w["model.wte.weight"], torch.tensor(toks_b)), w["model.wpe.weight"], 30),
    ])
    _close(h, want, "float32", "embedding")  # exact sums of stored values

    # norm, on all rows and on the wanted rows only
    x = (torch.randn(26, D, generator=g) * 2 + 0.5)
    norm = dec.layers[1].ffn_norm
    y = norm.forward(ctx, x.to(DEV))
    want = plain.layer_norm(x.double(), w["model.h.1.ln_2.weight"], w["model.h.1.ln_2.bias"], eps)
    _close(y, want, dtype, "layernorm")
    y = norm.forward(ctx, x.to(DEV), rows=ctx.wanted_rows, n_rows=ctx.n_wanted)
    _close(y, want[[0, 20, 25]], dtype, "layernorm on wanted rows")

    # feed-forward adds into the residual stream
    xin = _act(torch.randn(26, D, generator=g), dtype)
    res0 = torch.randn(26, D, generator=g)
    res = res0.clone().to(DEV)
    dec.layers[2].ffn.forward(ctx, xin, res)
    want = res0.double() + plain.mlp(xin.double().cpu(), w, "model.h.2.mlp.")
    _close(res, want, dtype, "feed-forward")

    # head
    xin = _act(torch.randn(3, D, generator=g), dtype)
    logits = torch.empty(3, V, dtype=torch.float32, device=DEV)
    dec.head.forward(ctx, xin, logits)
    _close(logits, plain.tied_head(xin.double().cpu(), w["model.wte.weight"]), dtype, "head")
    eng.cache.release_all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_part_and_block_in_portions(folder_b, dtype):
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = folder_b
    w = _w(weights, dtype)
    eng = _engine(folder, dtype)
    dec = eng.decoder
    D, H = config["n_embd"], config["n_head"]
    g = torch.Generator().manual_seed(2)
    n = 75
    x = _act(torch.randn(n, D, generator=g), dtype)
    res0 = torch.randn(n, D, generator=g)
    want = res0.double() + plain.self_attention(x.double().cpu(), w, "model.h.1.attn.", H)
    attn = dec.layers[1].mixer
    got, i = [], 0
    for cut in (37, 2, 1, 20, 1, 14):  # tiles, short portions and single rows
        e = [StepEntry("r", [0] * cut, [])]
        ctx = _context(eng, e)
        res = res0[i : i + cut].clone().to(DEV)
        attn.forward(ctx, x[i : i + cut], res, ctx.cache_view(1), True)
        got.append(res.clone())
        _commit(eng, e)
        i += cut
    _close(torch.cat(got), want, dtype, "attention part in portions")
    eng.cache.release_all()

    # a whole block
    h0 = torch.randn(n, D, generator=g)
    e = [StepEntry("s", [0] * n, [])]
    ctx = _context(eng, e)
    h = h0.clone().to(DEV)
    dec.layers[0].forward(ctx, h, ctx.cache_view(0), True)
    _close(h, plain.block(h0.double(), w, 0, H, config["layer_norm_epsilon"]), dtype, "block")
    eng.cache.release_all()
    eng.cache.check()


# ---------------------------------------------------------------------------
# toy parts: a mixer with state of its own, a rotating position encoding, a feed-forward
# with experts chosen per token, grouped key heads, a window, a layer that runs twice and a
# layer that reads another's cache


def _register_toys():
    from mlx_lm_amd.config import BaseModelArgs, LayerSpec, ModelPlan, PartSpec, RunEntry, StateNeed, register_model
    from mlx_lm_amd.ops import kernels
    from mlx_lm_amd.parts import (DecoderModel, FeedForward, Mixer, PositionEncoding, TensorSpec,
                                  register_feed_forward, register_mixer, register_position_encoding)

    class DecayMixer(Mixer):
        """``s_t = decay * s_{t-1} + x_t``; adds ``s_t`` to the residual.  Its state
        ``s`` lives in the request's state slot between steps."""

        def __init__(self, width, prefix=""):
            super().__init__(prefix)
            self.width = width

        def cache_need(self):
            return StateNeed((self.width,), "float32")

        def tensors(self):
            return {self._name("decay"): TensorSpec((self.width,), "vector")}

        def load(self, tensors):
            self.decay = tensors[self._name("decay")]

        def forward(self, ctx, x, residual, cache, writes_cache=True):
            for start, n, slot in zip(ctx.q_starts, ctx.q_lens, ctx.state_slots):
                s = cache.state[slot]
                for t in range(start, start + n):
                    s = self.decay * s + x[t].float()
                    residual[t] += s
                cache.state[slot] = s

    class PairRotation(PositionEncoding):
        """Rotates pairs of head columns by ``position * theta^(-2i/d)`` (written with torch ops)."""

        def __init__(self, head_dim, theta, prefix=""):
            super().__init__(prefix)
            self.head_dim, self.theta = head_dim, theta

        def rotate(self, ctx, q, k):
            half = self.head_dim // 2
            freq = self.theta ** (-torch.arange(half, device=q.device, dtype=torch.float32) / half)
            ang = ctx.positions.float()[:, None] * freq[None]
            cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
            for t in (q, k):
                v = t.float().reshape(t.shape[0], -1, self.head_dim)
                a, b = v[..., :half], v[..., half:]
                out = torch.cat([a * cos - b * sin, a * sin + b * cos], -1)
                t.copy_(out.reshape(t.shape).to(t.dtype))

    class HashedExperts(FeedForward):
        """``n_experts`` GELU feed-forwards; a token goes to expert ``token_id % n_experts``
        (routing by a hash of the token, so that rounding cannot change the choice).  The
        tokens of an expert are gathered, run through the framework's ``linear`` and added
        back into the residual stream."""

        def __init__(self, width, inner, n_experts, prefix=""):
            super().__init__(prefix)
            self.width, self.inner, self.n_experts = width, inner, n_experts

        def tensors(self):
            return {self._name("up"): TensorSpec((self.n_experts, self.inner, self.width), "matrix"),
                    self._name("down"): TensorSpec((self.n_experts, self.width, self.inner), "matrix")}

        def load(self, tensors):
            self.up, self.down = tensors[self._name("up")], tensors[self._name("down")]

        def forward(self, ctx, x, residual):
            expert = ctx.token_ids % self.n_experts
            for e in range(self.n_experts):
                rows = torch.nonzero(expert == e).flatten()
                if rows.numel() == 0:
                    continue
                xe = x[rows].contiguous()
                act = torch.empty((rows.numel(), self.inner), dtype=x.dtype, device=x.device)
                kernels.linear(act, xe, self.up[e], gelu=True)
                out = torch.empty((rows.numel(), self.width), dtype=torch.float32, device=x.device)
                kernels.linear(out, act, self.down[e])
                residual.index_add_(0, rows, out)

    register_mixer("toy_decay", DecayMixer)
    register_position_encoding("toy_pair_rotation", PairRotation)
    register_feed_forward("toy_hashed_experts", HashedExperts)

    @dataclass
    class ToyArgs(BaseModelArgs):
        model_type: str
        width: int
        vocab: int
        max_len: int
        heads: int
        kv_heads: int
        head_dim: int
        window: int
        inner: int
        eps: float
        theta: float
        experts: int

    class ToyModel:
        def __init__(self, args):
            self.args, self.model_type = args, args.model_type
            self.decoder = DecoderModel(self.plan(args))

        @property
        def layers(self):
            return self.decoder.layers

        @staticmethod
        def plan(a):
            def norm(p):
                return PartSpec("layernorm", {"width": a.width, "eps": a.eps}, p)

            def attention(p, window):
                return PartSpec("attention", {
                    "width": a.width, "n_heads": a.heads, "n_kv_heads": a.kv_heads, "head_dim": a.head_dim,
                    "window": window, "bias": False, "qkv_name": "qkv", "out_name": "o",
                    "position": PartSpec("toy_pair_rotation", {"head_dim": a.head_dim, "theta": a.theta})}, p)

            def ffn(p):
                return PartSpec("gelu_mlp", {"width": a.width, "inner": a.inner}, p)

            mixers = [attention("l0.mix.", 0), attention("l1.mix.", a.window),
                      PartSpec("toy_decay", {"width": a.width}, "l2.mix.")]
            ffns = [ffn("l0.ff."), PartSpec("toy_hashed_experts", {"width": a.width, "inner": a.inner,
                                                                     "n_experts": a.experts}, "l1.ff."),
                    ffn("l2.ff.")]
            layers = [LayerSpec("pre_norm", dict(mixer_norm=norm(f"l{i}.n1."), mixer=m, ffn_norm=norm(f"l{i}.n2."), ffn=f))
                      for i, (m, f) in enumerate(zip(mixers, ffns))]
            # layer 0 runs twice (two cache slots); the last run of layer 1 reads the
            # keys and values that its first run wrote
            schedule = [RunEntry(0, 0), RunEntry(1, 1), RunEntry(2, 2), RunEntry(0, 3),
                        RunEntry(1, 1, writes_cache=False)]
            return ModelPlan(
                width=a.width, vocab_size=a.vocab, max_positions=a.max_len,
                embedding=PartSpec("token", {"vocab_size": a.vocab, "width": a.width}, "emb."),
                embedding_positions=None, layers=layers, schedule=schedule,
                final_norm=norm("nf."), head=PartSpec("linear", {"vocab_size": a.vocab, "width": a.width,
                                                                  "weight_name": "head.weight"}))

    register_model("toy_hybrid", ToyModel, ToyArgs)
    return ToyModel, ToyArgs


TOY = dict(model_type="toy_hybrid", width=80, vocab=211, max_len=160, heads=6, kv_heads=2, head_dim=32,
           window=24, inner=120, eps=1e-4, theta=100.0, experts=3)


def _toy_folder(path):
    from safetensors.torch import save_file

    ToyModel, ToyArgs = _register_toys()
    model = ToyModel(ToyArgs.from_dict(TOY))
    g = torch.Generator().manual_seed(7)
    tensors = {}
    for name, spec in model.decoder.expected_tensors().items():
        if name.endswith("decay"):
            t = 0.5 + 0.4 * torch.rand(spec.shape, generator=g)
        elif spec.role == "vector":
            t = 1.0 + 0.1 * torch.randn(spec.shape, generator=g) if "weight" in name else 0.05 * torch.randn(spec.shape, generator=g)
        else:
            t = torch.randn(spec.shape, generator=g) * (0.25 if "qkv" in name else 0.05)
        tensors[name] = t
    os.makedirs(path, exist_ok=True)
    json.dump(TOY, open(os.path.join(path, "config.json"), "w"))
    save_file(tensors, os.path.join(path, "model.safetensors"))
    return tensors


def _toy_plain(t, ids):
    """The toy model on one whole sequence, from the plain parts."""
    a = TOY
    w = {k: v.double() for k, v in t.items()}
    L = len(ids)
    H, Hkv, hd = a["heads"], a["kv_heads"], a["head_dim"]
    pos = torch.arange(L, dtype=torch.float64)
    half = hd // 2
    freq = a["theta"] ** (-torch.arange(half, dtype=torch.float64) / half)
    ang = pos[:, None] * freq[None]

    def rotate(v):  # [heads, L, hd]
        x, y = v[..., :half], v[..., half:]
        return torch.cat([x * ang.cos() - y * ang.sin(), x * ang.sin() + y * ang.cos()], -1)

    def ln(x, p):
        return plain.layer_norm(x, w[p + "weight"], w[p + "bias"], a["eps"])

    def ffn(x, p):
        if p + "up" in w:  # experts by token id
            out = torch.zeros_like(x)
            for i, tok in enumerate(ids):
                e = tok % a["experts"]
                out[i] = plain.linear(plain.gelu_tanh(plain.linear(x[i : i + 1], w[p + "up"][e])), w[p + "down"][e])[0]
            return out
        return plain.mlp(x, w, p)

    kv_store = {}

    def attention(x, p, window, slot, writes):
        qkv = plain.linear(x, w[p + "qkv.weight"])
        q = qkv[:, : H * hd].reshape(L, H, hd).permute(1, 0, 2)
        if writes:
            k = qkv[:, H * hd : (H + Hkv) * hd].reshape(L, Hkv, hd).permute(1, 0, 2)
            v = qkv[:, (H + Hkv) * hd :].reshape(L, Hkv, hd).permute(1, 0, 2)
            kv_store[slot] = (rotate(k), v)
        k, v = kv_store[slot]
        o = plain.attention(rotate(q), k, v, hd**-0.5, plain.causal_mask(L, 0, window or None))
        return plain.linear(plain.merge_heads(o), w[p + "o.weight"])

    def decay(x, p):
        s, out = torch.zeros(a["width"], dtype=torch.float64), []
        for i in range(L):
            s = w[p + "decay"] * s + x[i]
            out.append(s)
        return torch.stack(out)

    h = plain.embed_tokens(w["emb.weight"], torch.tensor(ids))
    runs = [(0, 0, True), (1, 1, True), (2, 2, True), (0, 3, True), (1, 1, False)]
    for layer, slot, writes in runs:
        p = f"l{layer}."
        x = ln(h, p + "n1.")
        if layer == 2:
            h = h + decay(x, p + "mix.")
        else:
            h = h + attention(x, p + "mix.", a["window"] if layer == 1 else 0, slot, writes)
        h = h + ffn(ln(h, p + "n2."), p + "ff.")
    return plain.tied_head(ln(h, "nf."), w["head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(tmp_path, dtype):
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    tensors = _toy_folder(str(tmp_path))
    model, config = load_model(str(tmp_path), dtype=dtype)  # found by config.json's model_type
    assert model.model_type == "toy_hybrid" and len(model.layers) == 3
    cm_needs = model.decoder.cache_needs()
    assert len(cm_needs) == 4 and cm_needs[2].shape == (80,) and cm_needs[1].window == 24
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=14, max_requests=3)
    assert len(eng.cache.groups) == 2  # all keys, and a window of them: pages of their own

    ref = helpers.round_matrices_to_bf16(tensors) if dtype == "bfloat16" else tensors
    seqs = {"a": helpers.random_tokens(150, TOY["vocab"], 1), "b": helpers.random_tokens(61, TOY["vocab"], 2)}
    want = {k: _toy_plain(ref, v) for k, v in seqs.items()}
    # the bfloat16 tolerance is wider here: the toy mixers written with torch ops round again
    tol = dict(TOL, bfloat16=6e-2)

    def check(got, rid, what):
        scale = want[rid].abs().max().item()
        err = (got.double().cpu() - want[rid]).abs().max().item()
        assert err <= tol[dtype] * scale, f"{what}: {err:.3e} against {scale:.3e}"

    # whole
    eng.add_request("a")
    check(eng.step([StepEntry("a", seqs["a"], list(range(150)))]), "a", "whole")
    eng.end_request("a")
    # in portions, the two requests mixed, pages of the windowed group coming back on the way
    fed = {"a": 0, "b": 0}
    got = {"a": [], "b": []}
    cuts = {"a": [40, 2, 1, 1, 30, 1, 1, 17, 3, 54], "b": [1, 1, 25, 2, 1, 31]}
    eng.add_request("a")
    eng.add_request("b")
    for i in range(10):
        entries = []
        for rid in ("a", "b"):
            if i < len(cuts[rid]):
                n = cuts[rid][i]
                entries.append(StepEntry(rid, seqs[rid][fed[rid] : fed[rid] + n], list(range(n))))
                fed[rid] += n
        eng.cache.poison_free_pages()
        out = eng.step(entries)
        j = 0
        for e in entries:
            got[e.request_id].append(out[j : j + len(e.tokens)].clone())
            j += len(e.tokens)
        eng.cache.check()
    for rid in ("a", "b"):
        check(torch.cat(got[rid]), rid, f"portions, request {rid}")
    # the window let pages go: the windowed group holds fewer than the full group
    full, windowed = eng.cache.groups
    if full.need.window:
        full, windowed = windowed, full
    assert windowed.pool.n_held < full.pool.n_held
    eng.end_request("a")
    eng.end_request("b")
    assert eng.cache.free_pages() == 14


# ---------------------------------------------------------------------------
# a mixer that keeps state and launches kernels only: its steps are recorded and replayed


def _register_running_sum():
    from mlx_lm_amd.config import BaseModelArgs, LayerSpec, ModelPlan, PartSpec, RunEntry, StateNeed, register_model
    from mlx_lm_amd.parts import DecoderModel, Mixer, register_mixer

    class RunningSum(Mixer):
        """``s += sum of the portion's rows``; every row of the portion adds the new ``s`` to the
        residual.  Device-side indexing only (no value comes to the host), so a step with it can
        be recorded; a step that ran twice would add its rows to the state twice."""

        graph_safe = True

        def __init__(self, width, prefix=""):
            super().__init__(prefix)
            self.width = width

        def cache_need(self):
            return StateNeed((self.width,), "float32")

        def forward(self, ctx, x, residual, cache, writes_cache=True):
            slots = ctx.slot_ids.long()[ctx.token_req.long()]
            cache.state.index_add_(0, slots, x.float())
            residual += cache.state[slots]

    register_mixer("toy_running_sum", RunningSum)

    class NativeRunningSum(RunningSum):
        """The same mixer with a native twin in a library of its own (tests/native_parts/
        running_sum.hip, which includes csrc/engine_parts.h): the native walk calls it without a
        trip through Python, and no file of the framework names it."""

        def make_native(self):
            import ctypes

            from mlx_lm_amd.ops import build, native

            lib = build.load(build.add_source(os.path.join(os.path.dirname(__file__), "native_parts", "running_sum.hip")))
            lib.make_running_sum.restype, lib.make_running_sum.argtypes = ctypes.c_void_p, [ctypes.c_void_p, ctypes.c_int]
            return native.made(lib.make_running_sum(native.host(), self.width), "running sum")

        def forward(self, ctx, x, residual, cache, writes_cache=True):
            raise AssertionError("the native twin runs, not this")

    register_mixer("toy_running_sum_native", NativeRunningSum)

    @dataclass
    class SumArgs(BaseModelArgs):
        model_type: str
        width: int
        vocab: int
        max_len: int
        inner: int
        mixer: str = "toy_running_sum"

    class SumModel:
        def __init__(self, args):
            self.args, self.model_type = args, args.model_type
            self.decoder = DecoderModel(self.plan(args))

        @property
        def layers(self):
            return self.decoder.layers

        @staticmethod
        def plan(a):
            def norm(p):
                return PartSpec("layernorm", {"width": a.width, "eps": 1e-5}, p)

            layers = [
                LayerSpec("pre_norm", dict(
                    mixer_norm=norm("l0.n1."), mixer=PartSpec(a.mixer, {"width": a.width}, "l0.mix."),
                    ffn_norm=norm("l0.n2."), ffn=PartSpec("gelu_mlp", {"width": a.width, "inner": a.inner}, "l0.ff."))),
                LayerSpec("pre_norm", dict(
                    mixer_norm=norm("l1.n1."),
                    mixer=PartSpec("attention", {"width": a.width, "n_heads": 2, "head_dim": a.width // 2}, "l1.mix."),
                    ffn_norm=norm("l1.n2."), ffn=PartSpec("gelu_mlp", {"width": a.width, "inner": a.inner}, "l1.ff."))),
            ]
            return ModelPlan(
                width=a.width, vocab_size=a.vocab, max_positions=a.max_len,
                embedding=PartSpec("token", {"vocab_size": a.vocab, "width": a.width}, "emb."),
                embedding_positions=None, layers=layers, schedule=[RunEntry(0, 0), RunEntry(1, 1)],
                final_norm=norm("nf."), head=PartSpec("linear", {"vocab_size": a.vocab, "width": a.width,
                                                                  "weight_name": "emb.weight"}))

    register_model("toy_sum", SumModel, SumArgs)
    return SumModel, SumArgs


@pytest.mark.parametrize("mixer", ["toy_running_sum", "toy_running_sum_native"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_recorded_step_takes_its_tokens_once(tmp_path, dtype, mixer):
    """Steps of a model whose mixer keeps state, replayed from graphs, against the same steps
    run eagerly, bit for bit: the step that records a graph counts once, like any other.  The
    mixer is a Python part that launches kernels only, or a native part in a library of its own
    that the native walk calls directly (both give the same logits up to the order of a sum)."""
    from safetensors.torch import save_file

    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    cfg = dict(model_type="toy_sum", width=64, vocab=97, max_len=96, inner=80, mixer=mixer)
    SumModel, SumArgs = _register_running_sum()
    g = torch.Generator().manual_seed(3)
    tensors = {}
    for name, spec in SumModel(SumArgs.from_dict(cfg)).decoder.expected_tensors().items():
        if spec.role == "vector":
            tensors[name] = (1.0 if name.endswith("weight") else 0.0) + 0.05 * torch.randn(spec.shape, generator=g)
        else:
            tensors[name] = 0.1 * torch.randn(spec.shape, generator=g)
    json.dump(cfg, open(os.path.join(tmp_path, "config.json"), "w"))
    save_file(tensors, os.path.join(tmp_path, "model.safetensors"))
    model, _ = load_model(str(tmp_path), dtype=dtype)
    seqs = {"a": helpers.random_tokens(40, 97, 11), "b": helpers.random_tokens(33, 97, 12)}
    results, states = {}, {}
    for use_graphs in (True, False):
        eng = Engine(model, dtype=dtype, page_size=16, n_pages=8, max_requests=3, use_graphs=use_graphs,
                     record_prompt_steps=use_graphs)
        assert eng.use_graphs == use_graphs  # every part launches kernels only
        out = []
        for r in seqs:
            eng.add_request(r)
        out.append(eng.step([StepEntry("a", seqs["a"][:9], [8]), StepEntry("b", seqs["b"][:2], [1])]).clone())
        for i in range(24):  # decode steps of both (recorded at the first), then portions of one shape
            out.append(eng.step([StepEntry("a", [seqs["a"][9 + i]], [0]), StepEntry("b", [seqs["b"][2 + i]], [0])]).clone())
        for i in range(3):  # (recorded at the third sighting of the shape)
            out.append(eng.step([StepEntry("a", seqs["a"][33 + 2 * i : 35 + 2 * i], [0, 1])]).clone())
        if use_graphs:
            assert helpers.decode_graphs(eng, 2)[0].graph is not None
            assert any(sg.graph is not None for sg in eng._step_graphs.values())
        results[use_graphs] = torch.cat(out)
        states[use_graphs] = eng.cache.state(0)[[eng.cache.requests[r].state_slot for r in seqs]].clone()
    assert torch.equal(states[True], states[False])
    assert torch.equal(results[True], results[False])
    if mixer == "toy_running_sum_native":
        assert eng.stats.callbacks == 0  # no part of this model is called back in Python
        assert model.layers[0].mixer._native is not None
    _SUM_RESULTS[dtype, mixer] = results[False].float().cpu()
    other = _SUM_RESULTS.get((dtype, "toy_running_sum" if mixer.endswith("native") else "toy_running_sum_native"))
    if other is not None:
        tol = 1e-4 if dtype == "float32" else 5e-2
        assert (other - _SUM_RESULTS[dtype, mixer]).abs().max().item() <= tol * other.abs().max().item()


_SUM_RESULTS = {}


# ---------------------------------------------------------------------------
# windowed attention under recorded steps


def _register_windowed():
    from mlx_lm_amd.config import BaseModelArgs, LayerSpec, ModelPlan, PartSpec, RunEntry, register_model
    from mlx_lm_amd.parts import DecoderModel

    @dataclass
    class WinArgs(BaseModelArgs):
        model_type: str
        width: int
        vocab: int
        max_len: int
        heads: int
        kv_heads: int
        window: int
        inner: int

    class WinModel:
        """Built-in parts only (so its steps are recorded): a layer that sees every key and one
        that sees a window of them, grouped key heads, no position term at all."""

        def __init__(self, args):
            self.args, self.model_type = args, args.model_type
            self.decoder = DecoderModel(self.plan(args))

        @property
        def layers(self):
            return self.decoder.layers

        @staticmethod
        def plan(a):
            def norm(p):
                return PartSpec("layernorm", {"width": a.width, "eps": 1e-5}, p)

            def layer(i, window):
                p = f"l{i}."
                return LayerSpec("pre_norm", dict(
                    mixer_norm=norm(p + "n1."),
                    mixer=PartSpec("attention", {"width": a.width, "n_heads": a.heads, "n_kv_heads": a.kv_heads,
                                                 "head_dim": a.width // a.heads, "window": window, "bias": True}, p + "mix."),
                    ffn_norm=norm(p + "n2."), ffn=PartSpec("gelu_mlp", {"width": a.width, "inner": a.inner}, p + "ff.")))

            return ModelPlan(
                width=a.width, vocab_size=a.vocab, max_positions=a.max_len,
                embedding=PartSpec("token", {"vocab_size": a.vocab, "width": a.width}, "emb."),
                embedding_positions=None, layers=[layer(0, 0), layer(1, a.window)],
                schedule=[RunEntry(0, 0), RunEntry(1, 1)], final_norm=norm("nf."),
                head=PartSpec("linear", {"vocab_size": a.vocab, "width": a.width, "weight_name": "emb.weight"}))

    register_model("toy_windowed", WinModel, WinArgs)
    return WinModel, WinArgs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_window_under_recorded_steps(tmp_path, dtype):
    """Decoding far past a window of 24 keys under recorded steps: the windowed group's pages go
    back as the window passes them (their table entries turn to -1 and stay in the recorded
    step's table), pages are used again by a second request, and the logits equal the eager
    engine's bit for bit and the plain implementation's with the window's mask."""
    from safetensors.torch import save_file

    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    cfg = dict(model_type="toy_windowed", width=64, vocab=131, max_len=160, heads=4, kv_heads=2, window=24, inner=96)
    WinModel, WinArgs = _register_windowed()
    g = torch.Generator().manual_seed(5)
    tensors = {}
    for name, spec in WinModel(WinArgs.from_dict(cfg)).decoder.expected_tensors().items():
        if spec.role == "vector":
            tensors[name] = (1.0 if name.endswith("n1.weight") or name.endswith("n2.weight") or name == "nf.weight"
                             else 0.0) + 0.05 * torch.randn(spec.shape, generator=g)
        else:
            tensors[name] = torch.randn(spec.shape, generator=g) * (0.15 if "c_attn" in name else 0.08)
    json.dump(cfg, open(os.path.join(tmp_path, "config.json"), "w"))
    save_file(tensors, os.path.join(tmp_path, "model.safetensors"))
    model, _ = load_model(str(tmp_path), dtype=dtype)
    ref = helpers.round_matrices_to_bf16(tensors) if dtype == "bfloat16" else tensors
    w = {k: v.double() for k, v in ref.items()}
    H, Hkv, hd = cfg["heads"], cfg["kv_heads"], cfg["width"] // cfg["heads"]

    def plain_logits(ids):
        L = len(ids)
        h = plain.embed_tokens(w["emb.weight"], torch.tensor(ids))
        for i, window in ((0, None), (1, cfg["window"])):
            p = f"l{i}."
            x = plain.layer_norm(h, w[p + "n1.weight"], w[p + "n1.bias"], 1e-5)
            qkv = plain.linear(x, w[p + "mix.c_attn.weight"], w[p + "mix.c_attn.bias"])
            q = qkv[:, : H * hd].reshape(L, H, hd).permute(1, 0, 2)
            k = qkv[:, H * hd : (H + Hkv) * hd].reshape(L, Hkv, hd).permute(1, 0, 2).repeat_interleave(H // Hkv, 0)
            v = qkv[:, (H + Hkv) * hd :].reshape(L, Hkv, hd).permute(1, 0, 2).repeat_interleave(H // Hkv, 0)
            o = plain.attention(q, k, v, hd**-0.5, plain.causal_mask(L, 0, window))
            h = h + plain.linear(plain.merge_heads(o), w[p + "mix.c_proj.weight"], w[p + "mix.c_proj.bias"])
            h = h + plain.mlp(plain.layer_norm(h, w[p + "n2.weight"], w[p + "n2.bias"], 1e-5), w, p + "ff.")
        return plain.tied_head(plain.layer_norm(h, w["nf.weight"], w["nf.bias"], 1e-5), w["emb.weight"])

    seqs = {"a": helpers.random_tokens(150, cfg["vocab"], 21), "b": helpers.random_tokens(90, cfg["vocab"], 22)}
    results = {}
    for use_graphs in (True, False):
        eng = Engine(model, dtype=dtype, page_size=16, n_pages=16, max_requests=3, use_graphs=use_graphs)
        assert eng.use_graphs == use_graphs and len(eng.cache.groups) == 2
        got = {r: [] for r in seqs}
        eng.add_request("a")
        got["a"].append(eng.step([StepEntry("a", seqs["a"][:20], list(range(20)))]).clone())
        for i in range(20, 100):  # alone, one by one: the window passes pages of the windowed group
            got["a"].append(eng.step([StepEntry("a", [seqs["a"][i]], [0])]).clone())
        windowed = next(g for g in eng.cache.groups if g.need.window)
        full = next(g for g in eng.cache.groups if not g.need.window)
        assert windowed.pool.n_held < full.pool.n_held and -1 in eng.cache.requests["a"].blocks[eng.cache.groups.index(windowed)]
        eng.add_request("b")  # takes pages that the window gave back
        got["b"].append(eng.step([StepEntry("b", seqs["b"][:30], list(range(30)))]).clone())
        for i in range(50):
            out = eng.step([StepEntry("a", [seqs["a"][100 + i]], [0]), StepEntry("b", [seqs["b"][30 + i]], [0])])
            got["a"].append(out[0:1].clone())
            got["b"].append(out[1:2].clone())
            eng.cache.check()
        for i in range(80, 90):
            got["b"].append(eng.step([StepEntry("b", [seqs["b"][i]], [0])]).clone())
        if use_graphs:
            assert all(helpers.decode_graphs(eng, n)[0].graph is not None for n in (1, 2))
        results[use_graphs] = {r: torch.cat(v) for r, v in got.items()}
    for r, toks in seqs.items():
        _close(results[True][r], plain_logits(toks[: results[True][r].shape[0]]), dtype, f"a window under recorded steps, request {r}")
        assert torch.equal(results[True][r], results[False][r]), r


# ---------------------------------------------------------------------------
# a mixer whose values are narrower than its keys: the cache slot's layout is the mixer's choice


def _register_narrow_values():
    from mlx_lm_amd.config import BaseModelArgs, CacheNeed, LayerSpec, ModelPlan, PartSpec, RunEntry, register_model
    from mlx_lm_amd.parts import DecoderModel, Mixer, TensorSpec, register_mixer

    class NarrowValueAttention(Mixer):
        """One head; keys of ``key_dim`` columns, values of ``value_dim`` (written with torch ops
        over the slot's pages, which it reaches through the step's block table)."""

        def __init__(self, width, key_dim, value_dim, prefix=""):
            super().__init__(prefix)
            self.width, self.key_dim, self.value_dim = width, key_dim, value_dim

        def cache_need(self):
            return CacheNeed(1, self.key_dim, 0, v_head_dim=self.value_dim)

        def tensors(self):
            n = self._name
            return {n("q"): TensorSpec((self.key_dim, self.width), "matrix"),
                    n("k"): TensorSpec((self.key_dim, self.width), "matrix"),
                    n("v"): TensorSpec((self.value_dim, self.width), "matrix"),
                    n("o"): TensorSpec((self.width, self.value_dim), "matrix")}

        def load(self, tensors):
            self.q, self.k, self.v, self.o = (tensors[self._name(t)] for t in "qkvo")

        def forward(self, ctx, x, residual, cache, writes_cache=True):
            assert cache.kv is None and cache.keys.shape[-1] == self.key_dim and cache.values.shape[-1] == self.value_dim
            ps = cache.keys.shape[2]
            xf = x.float()
            q, k, v = xf @ self.q.float().t(), xf @ self.k.float().t(), xf @ self.v.float().t()
            pos, req = ctx.positions.long(), ctx.token_req.long()
            pages = cache.block_table[req, pos // ps].long()
            cache.keys[pages, 0, pos % ps] = k.to(cache.keys.dtype)
            cache.values[pages, 0, pos % ps] = v.to(cache.values.dtype)
            for t in range(x.shape[0]):
                n = int(pos[t]) + 1
                pg = cache.block_table[req[t], : (n + ps - 1) // ps].long()
                keys = cache.keys[pg, 0].reshape(-1, self.key_dim)[:n].float()
                values = cache.values[pg, 0].reshape(-1, self.value_dim)[:n].float()
                p = torch.softmax(keys @ q[t] * self.key_dim**-0.5, 0)
                residual[t] += (p @ values) @ self.o.float().t()

    register_mixer("toy_narrow_values", NarrowValueAttention)

    @dataclass
    class NarrowArgs(BaseModelArgs):
        model_type: str
        width: int
        vocab: int
        max_len: int
        key_dim: int
        value_dim: int
        inner: int

    class NarrowModel:
        def __init__(self, args):
            self.args, self.model_type = args, args.model_type
            self.decoder = DecoderModel(self.plan(args))

        @property
        def layers(self):
            return self.decoder.layers

        @staticmethod
        def plan(a):
            def norm(p):
                return PartSpec("layernorm", {"width": a.width, "eps": 1e-5}, p)

            layers = [LayerSpec("pre_norm", dict(
                mixer_norm=norm(f"l{i}.n1."),
                mixer=PartSpec("toy_narrow_values", {"width": a.width, "key_dim": a.key_dim, "value_dim": a.value_dim}, f"l{i}.mix."),
                ffn_norm=norm(f"l{i}.n2."), ffn=PartSpec("gelu_mlp", {"width": a.width, "inner": a.inner}, f"l{i}.ff.")))
                for i in range(2)]
            return ModelPlan(width=a.width, vocab_size=a.vocab, max_positions=a.max_len,
                             embedding=PartSpec("token", {"vocab_size": a.vocab, "width": a.width}, "emb."),
                             embedding_positions=None, layers=layers, schedule=[RunEntry(0, 0), RunEntry(1, 1)],
                             final_norm=norm("nf."),
                             head=PartSpec("linear", {"vocab_size": a.vocab, "width": a.width, "weight_name": "emb.weight"}))

    register_model("toy_narrow", NarrowModel, NarrowArgs)
    return NarrowModel, NarrowArgs


def test_a_mixer_whose_values_are_narrower_than_its_keys(tmp_path):
    """``CacheNeed(v_head_dim=...)``: the manager keeps keys and values of such a slot as tensors of
    their own widths and the step hands both to the mixer; whole, in portions and token by token
    give the plain computation, with pages used again."""
    from safetensors.torch import save_file

    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    cfg = dict(model_type="toy_narrow", width=48, vocab=97, max_len=96, key_dim=32, value_dim=16, inner=64)
    Model, Args = _register_narrow_values()
    g = torch.Generator().manual_seed(3)
    tensors = {}
    for name, spec in Model(Args.from_dict(cfg)).decoder.expected_tensors().items():
        if spec.role == "vector":
            tensors[name] = torch.ones(spec.shape) if name.endswith("weight") else torch.zeros(spec.shape)
        else:
            tensors[name] = torch.randn(spec.shape, generator=g) * (0.4 if name.endswith((".q", ".k")) else 0.1)
    json.dump(cfg, open(os.path.join(tmp_path, "config.json"), "w"))
    save_file(tensors, os.path.join(tmp_path, "model.safetensors"))
    model, _ = load_model(str(tmp_path), dtype="float32")
    eng = Engine(model, dtype="float32", page_size=16, n_pages=8, max_requests=2)
    assert len(eng.cache.groups) == 1 and eng.cache.kv(1)[1].shape[-1] == 16

    w = {k: v.double() for k, v in tensors.items()}
    ids = helpers.random_tokens(70, cfg["vocab"], 5)

    def ln(x, p):
        return plain.layer_norm(x, w[p + "weight"], w[p + "bias"], 1e-5)

    h = plain.embed_tokens(w["emb.weight"], torch.tensor(ids))
    for i in range(2):
        x = ln(h, f"l{i}.n1.")
        q, k, v = (plain.linear(x, w[f"l{i}.mix.{t}"]) for t in "qkv")
        o = plain.attention(q[None], k[None], v[None], cfg["key_dim"] ** -0.5, plain.causal_mask(len(ids)))[0]
        h = h + plain.linear(o, w[f"l{i}.mix.o"])
        h = h + plain.mlp(ln(h, f"l{i}.n2."), w, f"l{i}.ff.")
    want = plain.tied_head(ln(h, "nf."), w["emb.weight"])
    for cuts in ([70], [33, 2, 1, 1, 20, 13], [64] + [1] * 6):
        eng.add_request("r")
        eng.cache.poison_free_pages()
        rows, i = [], 0
        for n in cuts:
            rows.append(eng.step([StepEntry("r", ids[i : i + n], list(range(n)))]).clone())
            i += n
        eng.end_request("r")
        _close(torch.cat(rows), want, "float32", f"portions {cuts}")
    eng.cache.check()
    assert eng.cache.free_pages() == 8
