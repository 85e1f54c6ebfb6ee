"""The plain implementation pinned by what fixes it beside the reference's text:
library routines it must reduce to, invariants, and the vectors of the
reference's own tests."""


import pytest
import torch
import torch.nn.functional as F

import helpers
import plain_gpt2 as plain

torch.manual_seed(0)


def _weights(name):
    from mlx_lm_amd.config import get_model_classes

    config, seed, scheme = helpers.TINY[name]
    model_cls, args_cls = get_model_classes(config)
    args = args_cls.from_dict(config)
    t = model_cls.random_weights(args, seed, scheme)
    return config, plain.from_checkpoint_layout({k: v.double() for k, v in t.items()}, config["n_layer"])


def test_layer_norm_is_the_library_routine_and_eps_matters():
    x = torch.randn(5, 96, dtype=torch.float64) * 3 + 1
    x[2] *= 1e-3
    g, b = torch.randn(96, dtype=torch.float64), torch.randn(96, dtype=torch.float64)
    for eps in (1e-5, 1e-6):
        assert torch.allclose(plain.layer_norm(x, g, b, eps), F.layer_norm(x, (96,), g, b, eps), atol=1e-12)
    # gamma=1, beta=0: mean 0 and biased variance var/(var+eps)
    y = plain.layer_norm(x, torch.ones(96, dtype=torch.float64), torch.zeros(96, dtype=torch.float64), 1e-5)
    assert y.mean(-1).abs().max() < 1e-12
    var = x.var(-1, unbiased=False)
    assert torch.allclose((y**2).mean(-1), var / (var + 1e-5), atol=1e-12)
    # on the low-variance row the two eps differ visibly
    a = plain.layer_norm(x[2], g, b, 1e-5)
    c = plain.layer_norm(x[2], g, b, 1e-6)
    assert (a - c).abs().max() > 1e-3


def test_linear_layout_and_conv1d_transpose():
    x, w, b = torch.randn(4, 6), torch.randn(3, 6), torch.randn(3)
    assert torch.allclose(plain.linear(x, w, b), F.linear(x, w, b))
    assert torch.equal(plain.linear(x, torch.zeros(3, 6), b), b.expand(4, 3))
    conv = {"h.0.attn.c_attn.weight": w.t().contiguous(), "h.0.attn.bias": torch.ones(1)}
    back = plain.from_checkpoint_layout(conv, 1)
    assert torch.equal(back["model.h.0.attn.c_attn.weight"], w) and len(back) == 1


def test_gelu_is_the_tanh_form():
    x = torch.linspace(-6, 6, 241, dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-12)
    assert torch.allclose(plain.gelu_tanh(x) - plain.gelu_tanh(-x), x, atol=1e-12)
    assert plain.gelu_tanh(torch.zeros(1)).item() == 0
    # and not the erf form: they differ by a few 1e-4 around |x| = 2
    assert (plain.gelu_tanh(x) - F.gelu(x)).abs().max() > 1e-4


def test_attention_reduces_to_sdpa():
    H, L, hd = 3, 11, 16
    q, k, v = (torch.randn(H, L, hd, dtype=torch.float64) for _ in range(3))
    want = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    got = plain.attention(q, k, v, hd**-0.5, plain.causal_mask(L))
    assert torch.allclose(got, want, atol=1e-12)
    # no mask, one query, one key: the value itself
    assert torch.allclose(plain.attention(q[:, :1], k[:, :1], v[:, :1], hd**-0.5), v[:, :1])
    # equal keys: the mean of the visible values
    k_same = k[:, :1].expand(H, L, hd)
    got = plain.attention(q, k_same, v, hd**-0.5, plain.causal_mask(L))
    want = torch.cumsum(v, 1) / torch.arange(1, L + 1, dtype=torch.float64)[None, :, None]
    assert torch.allclose(got, want, atol=1e-12)
    # grouped key heads repeat over their group
    q6 = torch.randn(6, L, hd, dtype=torch.float64)
    got = plain.attention(q6, k[:2], v[:2], 0.3, plain.causal_mask(L))
    want = plain.attention(q6, k[:2].repeat_interleave(3, 0), v[:2].repeat_interleave(3, 0), 0.3, plain.causal_mask(L))
    assert torch.equal(got, want)


def test_causal_mask_vectors():
    # mlx_lm tests/test_prompt_cache.py:435-438: 4 queries on 16 cached keys
    m = plain.causal_mask(4, 16)
    assert tuple(m.shape) == (4, 20)
    assert m[0].sum() == 17 and m[3].sum() == 20
    # a window of 3: every row sees at most 3 keys, ending at its own position
    m = plain.causal_mask(5, 2, window=3)
    assert m.sum(-1).tolist() == [3, 3, 3, 3, 3]
    assert m[0].nonzero().flatten().tolist() == [0, 1, 2]
    assert torch.equal(plain.causal_mask(3), torch.tril(torch.ones(3, 3, dtype=torch.bool)))


def test_split_heads_order_and_head_permutation_invariance():
    config, w = _weights("B")
    D, H = config["n_embd"], config["n_head"]
    hd = D // H
    qkv = torch.arange(2 * 3 * D, dtype=torch.float64).reshape(2, 3 * D)
    q, k, v = plain.split_heads(qkv, H)
    assert q[1, 0, 0] == hd and k[0, 0, 0] == D and v[2, 1, 3] == 3 * D + 2 * D + 2 * hd + 3
    ids = helpers.random_tokens(12, config["vocab_size"], 1)
    base = plain.forward(w, config, ids)
    # permute whole heads of q, k, v rows of c_attn with the columns of c_proj: nothing changes
    perm = torch.tensor([2, 0, 1])
    idx = (perm[:, None] * hd + torch.arange(hd)[None]).flatten()
    w2 = dict(w)
    ca, cb = w["model.h.1.attn.c_attn.weight"].clone(), w["model.h.1.attn.c_attn.bias"].clone()
    for part in range(3):
        ca[part * D : (part + 1) * D] = w["model.h.1.attn.c_attn.weight"][part * D + idx]
        cb[part * D : (part + 1) * D] = w["model.h.1.attn.c_attn.bias"][part * D + idx]
    w2["model.h.1.attn.c_attn.weight"], w2["model.h.1.attn.c_attn.bias"] = ca, cb
    w2["model.h.1.attn.c_proj.weight"] = w["model.h.1.attn.c_proj.weight"][:, idx]
    assert torch.allclose(plain.forward(w2, config, ids), base, atol=1e-10)
    # permuting only the key rows does change the result
    w3 = dict(w)
    ck = w["model.h.1.attn.c_attn.weight"].clone()
    ck[D : 2 * D] = w["model.h.1.attn.c_attn.weight"][D + idx]
    w3["model.h.1.attn.c_attn.weight"] = ck
    assert (plain.forward(w3, config, ids) - base).abs().max() > 1e-6


def test_causality_and_position_table():
    config, w = _weights("B")
    ids = helpers.random_tokens(20, config["vocab_size"], 2)
    base = plain.forward(w, config, ids)
    changed = list(ids)
    changed[13] = (changed[13] + 1) % config["vocab_size"]
    other = plain.forward(w, config, changed)
    assert torch.equal(other[:13], base[:13]) and (other[13:] - base[13:]).abs().max() > 1e-6
    # positions enter through the learned table only: rolling the table by one
    # row equals feeding the sequence one position later
    h = plain.embed_tokens(w["model.wte.weight"], torch.tensor(ids))
    a = plain.add_learned_positions(h, w["model.wpe.weight"], 5)
    b = plain.add_learned_positions(h, torch.roll(w["model.wpe.weight"], -5, 0), 0)
    assert torch.equal(a, b)
    with pytest.raises(IndexError):
        plain.add_learned_positions(h, w["model.wpe.weight"], config["n_positions"] - 3)


def test_identity_blocks_give_closed_form_and_head_is_tied():
    config, w = _weights("A")
    w = dict(w)
    for i in range(config["n_layer"]):
        for t in ("attn.c_proj", "mlp.c_proj"):
            w[f"model.h.{i}.{t}.weight"] = torch.zeros_like(w[f"model.h.{i}.{t}.weight"])
            w[f"model.h.{i}.{t}.bias"] = torch.zeros_like(w[f"model.h.{i}.{t}.bias"])
    ids = torch.tensor(helpers.random_tokens(9, config["vocab_size"], 3))
    x = w["model.wte.weight"][ids] + w["model.wpe.weight"][:9]
    want = F.layer_norm(x, (config["n_embd"],), w["model.ln_f.weight"], w["model.ln_f.bias"],
                        config["layer_norm_epsilon"]) @ w["model.wte.weight"].t()
    assert torch.allclose(plain.forward(w, config, ids), want, atol=1e-12)
    # one buffer for embedding and head: a changed row moves both
    w["model.wte.weight"] = w["model.wte.weight"].clone()
    j = int(ids[4])
    w["model.wte.weight"][j] += torch.randn(config["n_embd"], dtype=torch.float64)  # (a uniform shift would vanish in the norm)
    moved = plain.forward(w, config, ids)
    assert (moved[:, j] - want[:, j]).abs().min() > 1e-3  # the column of the logits
    unused = next(t for t in range(config["vocab_size"]) if t not in ids.tolist())
    assert torch.allclose(moved[:4, unused], want[:4, unused], atol=1e-12)  # rows before token j unchanged


def test_log_softmax_and_greedy():
    x = torch.randn(3, 50, dtype=torch.float64)
    lp = plain.log_softmax(x)
    assert torch.allclose(lp, torch.log_softmax(x, -1)) and (lp <= 0).all()
    assert torch.allclose(lp.exp().sum(-1), torch.ones(3, dtype=torch.float64))
    config, w = _weights("A")
    out = plain.greedy_generate(w, config, [1, 2, 3], 4)
    assert len(out) == 4
    again = plain.forward(w, config, [1, 2, 3] + out[:3])
    assert [int(again[i].argmax()) for i in (2, 3, 4, 5)] == out


def test_sampler_filters_on_the_reference_vectors():
    # mlx_lm tests/test_sample_utils.py:19-105
    lp = torch.log(torch.tensor([0.9, 0.0, 0.0, 0.1]))
    assert plain.top_p_filter(lp, 0.3).exp().tolist() == pytest.approx([0.9, 0, 0, 0])
    lp = torch.log(torch.tensor([0.0, 0.5, 0.4, 0.1]))
    got = plain.top_p_filter(lp, 0.6).exp()
    assert (got / got.sum()).tolist() == pytest.approx([0, 0.5556, 0.4444, 0], abs=1e-3)
    got = plain.top_p_filter(lp, 0.95).exp()
    assert got.tolist() == pytest.approx([0, 0.5, 0.4, 0.1])
    lp = torch.log(torch.tensor([0.6, 0.0, 0.1, 0.3]))
    got = plain.top_k_filter(lp, 2).exp()
    assert (got / got.sum()).tolist() == pytest.approx([0.6667, 0, 0, 0.3333], abs=1e-3)
    lp = torch.log(torch.tensor([0.9, 0.0, 0.0, 0.1]))
    assert plain.min_p_filter(lp, 0.8).exp().tolist() == pytest.approx([0.9, 0, 0, 0])
    assert plain.min_p_filter(lp, 0.05).exp().tolist() == pytest.approx([0.9, 0, 0, 0.1])
    # batched rows are independent
    rows = torch.log(torch.tensor([[0.9, 0.0, 0.0, 0.1], [0.1, 0.8, 0.0, 0.1]]))
    got = plain.top_k_filter(rows, 1).exp()
    assert got.tolist() == [pytest.approx([0.9, 0, 0, 0]), pytest.approx([0, 0.8, 0, 0])]
    # xtc: tokens above the threshold go, except the least likely of them
    probs = torch.tensor([0.4, 0.3, 0.2, 0.1])
    got = plain.xtc_filter(torch.log(probs), 0.15)
    assert torch.isfinite(got).tolist() == [False, False, True, True]
    got = plain.xtc_filter(torch.log(probs), 0.15, special_tokens=[0])
    assert torch.isfinite(got).tolist() == [True, False, True, True]


def test_penalties():
    x = torch.tensor([1.0, -1.0, 2.0, 0.5])
    assert plain.repetition_penalty(x, [0, 1, 0], 2.0).tolist() == [0.5, -2.0, 2.0, 0.5]
    assert plain.presence_penalty(x, [0, 0, 2], 0.5).tolist() == [0.5, -1.0, 1.5, 0.5]
    assert plain.frequency_penalty(x, [0, 0, 2], 0.5).tolist() == [0.0, -1.0, 1.5, 0.5]
    assert plain.frequency_penalty(x, [0, 0, 2], 0.5, context_size=1).tolist() == [1.0, -1.0, 1.5, 0.5]


def _library_block(x, w, i, n_head, eps):
    """One block put together from library routines only, in the order the reference's text
    gives (mlx_lm/models/gpt2.py:98-108; inside attention :52-68, the MLP :71-80)."""
    p = f"model.h.{i}."
    D = x.shape[-1]
    L = x.shape[0]
    a = F.layer_norm(x, (D,), w[p + "ln_1.weight"], w[p + "ln_1.bias"], eps)
    qkv = F.linear(a, w[p + "attn.c_attn.weight"], w[p + "attn.c_attn.bias"])
    q, k, v = (t.reshape(L, n_head, D // n_head).transpose(0, 1)[None] for t in qkv.split(D, dim=-1))
    o = F.scaled_dot_product_attention(q, k, v, is_causal=True)[0].transpose(0, 1).reshape(L, D)
    h = x + F.linear(o, w[p + "attn.c_proj.weight"], w[p + "attn.c_proj.bias"])
    m = F.layer_norm(h, (D,), w[p + "ln_2.weight"], w[p + "ln_2.bias"], eps)
    m = F.gelu(F.linear(m, w[p + "mlp.c_fc.weight"], w[p + "mlp.c_fc.bias"]), approximate="tanh")
    return h + F.linear(m, w[p + "mlp.c_proj.weight"], w[p + "mlp.c_proj.bias"])


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_model_is_the_library_routines_in_the_reference_s_order(name):
    config, w = _weights(name)
    D, H, eps = config["n_embd"], config["n_head"], config["layer_norm_epsilon"]
    ids = torch.tensor(helpers.random_tokens(23, config["vocab_size"], 6))
    h = F.embedding(ids, w["model.wte.weight"]) + w["model.wpe.weight"][: len(ids)]
    for i in range(config["n_layer"]):
        want = _library_block(h, w, i, H, eps)
        assert torch.allclose(plain.block(h, w, i, H, eps), want, atol=1e-11)
        h = want
    want = F.linear(F.layer_norm(h, (D,), w["model.ln_f.weight"], w["model.ln_f.bias"], eps), w["model.wte.weight"])
    assert torch.allclose(plain.forward(w, config, ids), want, atol=1e-10)


def test_block_wiring_by_invariants():
    """What a mis-wired block would break: each sub-layer reads the *norm* of the stream (so its
    contribution does not change when the stream is scaled), adds to the stream *unnormed*, the
    attention sub-layer comes first with ``ln_1`` and the feed-forward reads its result with
    ``ln_2``, and the last norm stands between the blocks and the head."""
    config, w = _weights("B")
    H, eps, D = config["n_head"], 0.0, config["n_embd"]  # (eps 0: the norm of c*x is the norm of x exactly)
    x = torch.randn(9, D, dtype=torch.float64)
    base = plain.block(x, w, 1, H, eps)
    # pre-norm: block(c x) - c x == block(x) - x would hold only if the second sub-layer saw a
    # scaled stream too; with the feed-forward's output projection off it is exact
    off_mlp = dict(w)
    off_mlp["model.h.1.mlp.c_proj.weight"] = torch.zeros_like(w["model.h.1.mlp.c_proj.weight"])
    off_mlp["model.h.1.mlp.c_proj.bias"] = torch.zeros_like(w["model.h.1.mlp.c_proj.bias"])
    d1 = plain.block(x, off_mlp, 1, H, eps) - x
    assert torch.allclose(plain.block(3.0 * x, off_mlp, 1, H, eps) - 3.0 * x, d1, atol=1e-10)
    assert d1.abs().max() > 1e-3
    # the attention sub-layer uses ln_1, not ln_2: with the MLP off, ln_2 does not matter, ln_1 does
    changed = dict(off_mlp)
    changed["model.h.1.ln_2.weight"] = w["model.h.1.ln_2.weight"] * 1.7
    assert torch.equal(plain.block(x, changed, 1, H, eps) - x, d1)
    changed = dict(off_mlp)
    changed["model.h.1.ln_1.bias"] = w["model.h.1.ln_1.bias"] + 0.3
    assert (plain.block(x, changed, 1, H, eps) - x - d1).abs().max() > 1e-4
    # attention off: what is left is x + mlp(ln_2(x)), row by row (no mixing of positions)
    off_attn = dict(w)
    off_attn["model.h.1.attn.c_proj.weight"] = torch.zeros_like(w["model.h.1.attn.c_proj.weight"])
    off_attn["model.h.1.attn.c_proj.bias"] = torch.zeros_like(w["model.h.1.attn.c_proj.bias"])
    d2 = plain.block(x, off_attn, 1, H, eps) - x
    assert torch.allclose(plain.block(x[4:5], off_attn, 1, H, eps) - x[4:5], d2[4:5], atol=1e-12)
    assert torch.allclose(plain.block(2.0 * x, off_attn, 1, H, eps) - 2.0 * x, d2, atol=1e-10)
    # the feed-forward reads the stream *after* attention was added: both on is not the sum of each alone
    assert ((base - x) - (d1 + d2)).abs().max() > 1e-4
    # and attention does not read the feed-forward's output: the first row's attention term is
    # the same whatever the feed-forward does (one key: the value itself)
    moved = dict(w)
    moved["model.h.1.mlp.c_proj.bias"] = w["model.h.1.mlp.c_proj.bias"] + 1.0
    assert torch.allclose(plain.block(x, moved, 1, H, eps) - base, torch.ones_like(base), atol=1e-10)
    # the final norm: scaling the last block's output stream leaves the logits unchanged, which
    # holds only if ln_f stands before the head; its scale doubles them
    cfg0 = dict(config, layer_norm_epsilon=0.0)
    ids = helpers.random_tokens(7, config["vocab_size"], 8)
    logits = plain.forward(w, cfg0, ids)
    w2 = dict(w)
    w2["model.ln_f.weight"], w2["model.ln_f.bias"] = 2 * w["model.ln_f.weight"], 2 * w["model.ln_f.bias"]
    assert torch.allclose(plain.forward(w2, cfg0, ids), 2 * logits, atol=1e-9)


def test_query_key_value_order_by_construction():
    """Weights built so that the three thirds of ``c_attn`` can be told apart: the first third
    makes queries that pick out, through the second third's keys, exactly one earlier position,
    and the third third's values carry that position's marker.  Swapping any two thirds moves
    the result (mlx_lm/models/gpt2.py:52-58: q, k, v in this order)."""
    L, D = 6, 16
    w = {k: torch.zeros(s, dtype=torch.float64) for k, s in {
        "a.c_attn.weight": (3 * D, D), "a.c_attn.bias": (3 * D,), "a.c_proj.weight": (D, D), "a.c_proj.bias": (D,)}.items()}
    # rows of x: one-hot of the position in columns 0..5, one-hot of the position to look at in 8..13
    x = torch.zeros(L, D, dtype=torch.float64)
    look = [0, 0, 1, 1, 3, 2]
    for t in range(L):
        x[t, t] = 1.0
        x[t, 8 + look[t]] = 1.0
    big = 60.0
    mark = [9, 7, 12, 6, 15, 10]
    for j in range(L):
        w["a.c_attn.weight"][j, 8 + j] = big          # q_j = big * [looks at j]
        w["a.c_attn.weight"][D + j, j] = 1.0          # k_j = [is position j]
        w["a.c_attn.weight"][2 * D + mark[j], j] = 1.0  # v_j = position j's marker (not its key)
    w["a.c_proj.weight"] = torch.eye(D, dtype=torch.float64)
    out = plain.self_attention(x, w, "a.", 1)
    want = torch.zeros(L, D, dtype=torch.float64)
    for t in range(L):
        want[t, mark[look[t]]] = 1.0
    assert torch.allclose(out, want, atol=1e-6)
    for a, b in ((0, 1), (0, 2), (1, 2)):
        sw = dict(w)
        m = w["a.c_attn.weight"].clone()
        m[a * D:(a + 1) * D], m[b * D:(b + 1) * D] = w["a.c_attn.weight"][b * D:(b + 1) * D], w["a.c_attn.weight"][a * D:(a + 1) * D]
        sw["a.c_attn.weight"] = m
        assert (plain.self_attention(x, sw, "a.", 1) - want).abs().max() > 0.1, (a, b)
