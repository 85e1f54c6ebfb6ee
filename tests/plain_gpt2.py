"""Plain, slow GPT-2: whole sequences, no cache, one function for each part.

Written from the formulas of the reference (ml-explore/mlx-lm), each function
citing the file and lines it follows.  Runs on the CPU in float64 unless asked
otherwise.  It shares no code with the engine: tests import the engine on one
side and this file on the other.

Weights are a dict of torch tensors under the names that the reference's
``sanitize`` produces (``model.wte.weight`` and so on, linear weights laid out
``[out, in]``; mlx_lm/models/gpt2.py:170-196).
"""

import math

import torch


def embed_tokens(wte, ids):
    """``h = wte[ids]`` (mlx_lm/models/gpt2.py:132)."""
    return wte.index_select(0, ids)


def add_learned_positions(h, wpe, offset=0):
    """``h += wpe[arange(L) + offset]`` (mlx_lm/models/gpt2.py:137-144).

    ``offset`` is the number of tokens the request already holds.
    """
    L = h.shape[0]
    pos = torch.arange(L) + offset
    if int(pos[-1]) >= wpe.shape[0]:
        raise IndexError("position beyond n_positions")
    return h + wpe.index_select(0, pos)


def layer_norm(x, gamma, beta, eps):
    """LayerNorm over the last axis, biased variance, eps inside the root.

    The reference calls ``nn.LayerNorm(n_embd, eps=layer_norm_epsilon)``
    (mlx_lm/models/gpt2.py:92-96,123); the formula is the library's.
    """
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * gamma + beta


def linear(x, w, b=None):
    """``x @ w.T + b`` with ``w`` laid out ``[out, in]``.

    ``nn.Linear`` in mlx_lm/models/gpt2.py:41-42,76-77; the ``[out, in]``
    layout is what ``sanitize`` makes from Conv1D's ``[in, out]``
    (mlx_lm/models/gpt2.py:175-190).
    """
    y = x @ w.t()
    if b is not None:
        y = y + b
    return y


def split_heads(qkv, n_head):
    """Split a fused ``[L, 3D]`` projection into q, k, v of ``[H, L, hd]``.

    ``mx.split(qkv, 3, axis=-1)`` then ``reshape(B, L, n_head, -1)`` and
    ``transpose(0, 2, 1, 3)`` (mlx_lm/models/gpt2.py:52-58): q first, then k,
    then v; head ``h`` takes columns ``h*hd .. (h+1)*hd - 1``.
    """
    L, three_d = qkv.shape
    D = three_d // 3
    q, k, v = qkv[:, :D], qkv[:, D : 2 * D], qkv[:, 2 * D :]
    hd = D // n_head

    def heads(t):
        return t.reshape(L, n_head, hd).permute(1, 0, 2)

    return heads(q), heads(k), heads(v)


def causal_mask(n_q, offset=0, window=None):
    """Boolean ``[n_q, offset + n_q]`` mask, true where a query sees a key.

    ``linds >= rinds`` with ``linds = arange(offset, offset+N)`` and
    ``rinds = arange(offset+N)``; a window adds ``linds < rinds + window``
    (mlx_lm/models/base.py:24-35).
    """
    rinds = torch.arange(offset + n_q)[None, :]
    linds = torch.arange(offset, offset + n_q)[:, None]
    mask = linds >= rinds
    if window is not None:
        mask = mask & (linds < rinds + window)
    return mask


def attention(q, k, v, scale, mask=None):
    """``softmax(scale * q k^T + mask) v`` for ``[H, Lq, hd]`` / ``[H, Lk, hd]``.

    mlx_lm/models/base.py:132-139 hands this to the fused kernel; the spelled
    out form is mlx_lm/models/base.py:77-101: scores scaled, masked entries
    set to the lowest finite number, softmax in full precision, times v.
    Fewer key heads than query heads repeat each key head over its group
    (mlx_lm/models/base.py:74-85).
    """
    Hq, Hk = q.shape[0], k.shape[0]
    if Hk != Hq:
        rep = Hq // Hk
        k = k.repeat_interleave(rep, dim=0)
        v = v.repeat_interleave(rep, dim=0)
    scores = (q * scale) @ k.transpose(-1, -2)
    if mask is not None:
        scores = torch.where(mask, scores, torch.finfo(scores.dtype).min)
    p = torch.softmax(scores, dim=-1)
    return p @ v


def merge_heads(o):
    """``[H, L, hd] -> [L, H*hd]`` (mlx_lm/models/gpt2.py:67)."""
    H, L, hd = o.shape
    return o.permute(1, 0, 2).reshape(L, H * hd)


def gelu_tanh(x):
    """``0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))``.

    ``nn.gelu_approx`` in mlx_lm/models/gpt2.py:80; the tanh form is the one
    GPT-2 checkpoints name ``gelu_new``.
    """
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x**3)))


def self_attention(x, w, prefix, n_head, window=None):
    """The attention sub-layer on an already normed input, whole sequence.

    mlx_lm/models/gpt2.py:44-68 with ``scale = head_dim ** -0.5`` (line 39).
    """
    qkv = linear(x, w[prefix + "c_attn.weight"], w[prefix + "c_attn.bias"])
    q, k, v = split_heads(qkv, n_head)
    hd = q.shape[-1]
    L = x.shape[0]
    mask = causal_mask(L, 0, window) if (L > 1 or window is not None) else None
    o = attention(q, k, v, hd**-0.5, mask)
    return linear(merge_heads(o), w[prefix + "c_proj.weight"], w[prefix + "c_proj.bias"])


def mlp(x, w, prefix):
    """``c_proj(gelu(c_fc(x)))`` (mlx_lm/models/gpt2.py:71-80)."""
    h = gelu_tanh(linear(x, w[prefix + "c_fc.weight"], w[prefix + "c_fc.bias"]))
    return linear(h, w[prefix + "c_proj.weight"], w[prefix + "c_proj.bias"])


def block(x, w, i, n_head, eps):
    """Pre-norm residual block (mlx_lm/models/gpt2.py:98-108)."""
    p = f"model.h.{i}."
    r = self_attention(
        layer_norm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], eps), w, p + "attn.", n_head
    )
    h = x + r
    r = mlp(layer_norm(h, w[p + "ln_2.weight"], w[p + "ln_2.bias"], eps), w, p + "mlp.")
    return h + r


def tied_head(h, wte):
    """``logits = h @ wte^T`` (``wte.as_linear``, mlx_lm/models/gpt2.py:167)."""
    return h @ wte.t()


def forward(weights, config, ids, dtype=torch.float64):
    """Logits ``[L, V]`` at every position of one whole sequence.

    mlx_lm/models/gpt2.py:125-151 (embeddings, blocks, final norm) and
    161-168 (tied head).  ``config`` is the dict of config.json.
    """
    h = final_hidden(weights, config, ids, dtype)
    return tied_head(h, weights["model.wte.weight"].to(dtype))


def final_hidden(weights, config, ids, dtype=torch.float64):
    """What the head is applied to, ``[L, D]``: embeddings, blocks, final norm
    (mlx_lm/models/gpt2.py:125-151).  For tests that cannot afford the head at every position."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    ids = torch.as_tensor(ids, dtype=torch.long)
    eps = config["layer_norm_epsilon"]
    h = embed_tokens(w["model.wte.weight"], ids)
    h = add_learned_positions(h, w["model.wpe.weight"], 0)
    for i in range(config["n_layer"]):
        h = block(h, w, i, config["n_head"], eps)
    return layer_norm(h, w["model.ln_f.weight"], w["model.ln_f.bias"], eps)


def log_softmax(logits):
    """``logits - logsumexp(logits)`` (mlx_lm/generate.py:411)."""
    return logits - torch.logsumexp(logits, dim=-1, keepdim=True)


def greedy_generate(weights, config, prompt, max_tokens, dtype=torch.float64):
    """Argmax decoding by re-running the whole sequence for every token.

    ``temp == 0`` means ``argmax`` of the log-probabilities
    (mlx_lm/sample_utils.py:46-47); one token per forward call
    (mlx_lm/generate.py:444-461).
    """
    seq = list(prompt)
    out = []
    for _ in range(max_tokens):
        logits = forward(weights, config, seq, dtype)[-1]
        tok = int(torch.argmax(logits))
        out.append(tok)
        seq.append(tok)
    return out


# ----------------------------------------------------------------------------
# weights in the two layouts


def conv1d_layout(weights, n_layer):
    """The same weights as a GPT-2 checkpoint stores them.

    The inverse of the reference's ``sanitize`` (mlx_lm/models/gpt2.py:170-196):
    no ``model.`` prefix and the four projection matrices of each layer laid
    out ``[in, out]``.
    """
    out = {}
    for k, v in weights.items():
        name = k[len("model.") :] if k.startswith("model.") else k
        out[name] = v
    for i in range(n_layer):
        for t in ("attn.c_attn", "attn.c_proj", "mlp.c_fc", "mlp.c_proj"):
            key = f"h.{i}.{t}.weight"
            out[key] = out[key].t().contiguous()
    return out


def from_checkpoint_layout(tensors, n_layer):
    """Checkpoint tensors to the names and layouts ``forward`` wants.

    What the reference's ``sanitize`` does (mlx_lm/models/gpt2.py:170-196):
    drop ``attn.bias``, transpose the four Conv1D matrices, prefix ``model.``.
    """
    out = {}
    for k, v in tensors.items():
        if k.endswith(".attn.bias"):
            continue
        out[k] = v
    for i in range(n_layer):
        for t in ("attn.c_attn", "attn.c_proj", "mlp.c_fc", "mlp.c_proj"):
            key = f"h.{i}.{t}.weight"
            if key in out:
                out[key] = out[key].t().contiguous()
    return {(k if k.startswith("model.") else "model." + k): v for k, v in out.items()}


# ----------------------------------------------------------------------------
# sampling (plain forms of mlx_lm/sample_utils.py)


def top_p_filter(logprobs, top_p):
    """Keep tokens whose ascending cumulative probability exceeds ``1 - top_p``.

    mlx_lm/sample_utils.py:204-237.
    """
    probs = torch.exp(logprobs)
    order = torch.argsort(logprobs, dim=-1)
    sorted_probs = torch.gather(probs, -1, order)
    cum = torch.cumsum(sorted_probs, dim=-1)
    inv = torch.empty_like(order)
    inv.scatter_(-1, order, torch.arange(order.shape[-1]).expand_as(order))
    cum = torch.gather(cum, -1, inv)
    return torch.where(cum > 1 - top_p, logprobs, torch.tensor(-float("inf"), dtype=logprobs.dtype))


def min_p_filter(logprobs, min_p, min_tokens_to_keep=1):
    """Drop tokens below ``max + log(min_p)`` but keep the best few.

    mlx_lm/sample_utils.py:154-201.
    """
    top = logprobs.max(dim=-1, keepdim=True).values
    remove = logprobs < top + math.log(min_p)
    if min_tokens_to_keep > 1:
        keep_idx = torch.topk(logprobs, min_tokens_to_keep, dim=-1).indices
        remove.scatter_(-1, keep_idx, False)
    return torch.where(remove, torch.tensor(-float("inf"), dtype=logprobs.dtype), logprobs)


def top_k_filter(logprobs, top_k):
    """Keep the ``top_k`` most probable tokens (mlx_lm/sample_utils.py:129-151)."""
    V = logprobs.shape[-1]
    if not (0 < top_k < V):
        raise ValueError("top_k out of range")
    kth = torch.topk(logprobs, top_k, dim=-1).values[..., -1:]
    return torch.where(logprobs < kth, torch.tensor(-float("inf"), dtype=logprobs.dtype), logprobs)


def xtc_filter(logits, threshold, special_tokens=()):
    """Remove every token above the threshold except the least likely of them.

    mlx_lm/sample_utils.py:240-276, the branch in which XTC applies.
    """
    probs = torch.softmax(logits, -1)
    inf = torch.tensor(float("inf"), dtype=probs.dtype)
    lowest = torch.where(probs > threshold, probs, inf).min(dim=-1, keepdim=True).values
    mask = probs > lowest
    for t in special_tokens:
        mask[..., t] = False
    return torch.where(mask, torch.tensor(-float("inf"), dtype=logits.dtype), logits)


def repetition_penalty(logits, tokens, penalty, context_size=20):
    """mlx_lm/sample_utils.py:284-315."""
    logits = logits.clone()
    if len(tokens) > 0:
        idx = torch.as_tensor(list(tokens)[-context_size:], dtype=torch.long)
        sel = logits[idx]
        logits[idx] = torch.where(sel < 0, sel * penalty, sel / penalty)
    return logits


def presence_penalty(logits, tokens, penalty, context_size=20):
    """mlx_lm/sample_utils.py:318-342: once for each token that occurs."""
    logits = logits.clone()
    if len(tokens) > 0:
        idx = torch.as_tensor(sorted(set(list(tokens)[-context_size:])), dtype=torch.long)
        logits[idx] -= penalty
    return logits


def frequency_penalty(logits, tokens, penalty, context_size=20):
    """mlx_lm/sample_utils.py:345-369: once for every occurrence."""
    logits = logits.clone()
    for t in list(tokens)[-context_size:]:
        logits[t] -= penalty
    return logits
