"""GPT-2: arguments, plan, tensor names, random weights.

The architecture of mlx_lm/models/gpt2.py: token and learned position
embeddings, ``n_layer`` pre-LayerNorm blocks of fused-QKV multi-head causal
attention and a tanh-GELU MLP, a final LayerNorm and a head tied to the token
embedding.
"""

import math
from dataclasses import dataclass
from typing import Optional

import torch

from ..config.base import BaseModelArgs
from ..config.plan import LayerSpec, ModelPlan, PartSpec, RunEntry
from ..parts.model import DecoderModel


@dataclass
class ModelArgs(BaseModelArgs):
    """Keys of a GPT-2 config.json (mlx_lm/models/gpt2.py:12-26).

    The reference reads the first eight and ignores the rest; here the rest
    is read too and anything the engine would compute differently is refused.
    ``n_ctx`` is legacy and optional.
    """

    model_type: str
    n_embd: int
    n_head: int
    n_layer: int
    n_positions: int
    layer_norm_epsilon: float
    vocab_size: int
    n_ctx: Optional[int] = None
    n_inner: Optional[int] = None
    num_key_value_heads: Optional[int] = None
    activation_function: str = "gelu_new"
    tie_word_embeddings: bool = True
    scale_attn_weights: bool = True
    scale_attn_by_inverse_layer_idx: bool = False

    def __post_init__(self):
        if self.n_ctx is None:
            self.n_ctx = self.n_positions
        if self.n_inner is None:
            self.n_inner = 4 * self.n_embd  # mlx_lm/models/gpt2.py:76-77
        if self.num_key_value_heads is None:
            self.num_key_value_heads = self.n_head  # mlx_lm/models/gpt2.py:24-26
        for key in ("n_embd", "n_head", "n_layer", "n_positions", "vocab_size", "n_inner"):
            if not isinstance(getattr(self, key), int) or getattr(self, key) <= 0:
                raise ValueError(f"{key} must be a positive integer, got {getattr(self, key)!r}")
        if self.n_embd % self.n_head:
            raise ValueError("n_embd must be divisible by n_head")  # mlx_lm/models/gpt2.py:33
        # num_key_value_heads is read and not used, as in the reference: keys and values are
        # reshaped with n_head (mlx_lm/models/gpt2.py:57-58), and the fused c_attn of
        # [3 n_embd, n_embd] leaves no room for fewer key heads.
        if not self.tie_word_embeddings:
            raise ValueError("an untied output head is not implemented for gpt2")
        if not self.scale_attn_weights or self.scale_attn_by_inverse_layer_idx:
            raise ValueError(
                "only scale_attn_weights=true with scale_attn_by_inverse_layer_idx=false is implemented"
            )
        if self.layer_norm_epsilon <= 0:
            raise ValueError(f"layer_norm_epsilon must be positive, got {self.layer_norm_epsilon}")

    @property
    def head_dim(self):
        return self.n_embd // self.n_head


_CONV1D = ("attn.c_attn", "attn.c_proj", "mlp.c_fc", "mlp.c_proj")


class Model:
    """The GPT-2 model: a ``DecoderModel`` built from the plan below."""

    def __init__(self, args: ModelArgs):
        self.args = args
        self.model_type = args.model_type
        self.decoder = DecoderModel(self.plan(args))

    @property
    def layers(self):
        return self.decoder.layers

    @staticmethod
    def plan(args: ModelArgs) -> ModelPlan:
        D, eps = args.n_embd, args.layer_norm_epsilon

        def norm(prefix):
            return PartSpec("layernorm", {"width": D, "eps": eps, "bias": True}, prefix)

        layers = []
        for i in range(args.n_layer):
            p = f"model.h.{i}."
            attention = PartSpec(
                "attention",
                {
                    "width": D,
                    "n_heads": args.n_head,
                    "n_kv_heads": args.n_head,  # mlx_lm/models/gpt2.py:57-58
                    "head_dim": args.head_dim,
                    "scale": args.head_dim**-0.5,  # mlx_lm/models/gpt2.py:39
                    "bias": True,
                    "window": 0,
                    "position": None,
                },
                p + "attn.",
            )
            mlp = PartSpec(
                "gelu_mlp",
                {"width": D, "inner": args.n_inner, "activation": args.activation_function},
                p + "mlp.",
            )
            layers.append(
                LayerSpec(
                    arrangement="pre_norm",  # mlx_lm/models/gpt2.py:98-108
                    parts=dict(mixer_norm=norm(p + "ln_1."), mixer=attention, ffn_norm=norm(p + "ln_2."), ffn=mlp),
                )
            )
        return ModelPlan(
            width=D,
            vocab_size=args.vocab_size,
            max_positions=args.n_positions,
            embedding=PartSpec("token", {"vocab_size": args.vocab_size, "width": D}, "model.wte."),
            embedding_positions=PartSpec(
                "learned", {"max_positions": args.n_positions, "width": D}, "model.wpe."
            ),
            layers=layers,
            schedule=[RunEntry(layer=i, cache=i) for i in range(args.n_layer)],
            final_norm=norm("model.ln_f."),
            head=PartSpec(
                "linear",
                {"vocab_size": args.vocab_size, "width": D, "weight_name": "model.wte.weight"},
            ),
        )

    def sanitize(self, weights):
        """Checkpoint names and layouts to the model's.

        As mlx_lm/models/gpt2.py:170-196: drop each layer's ``attn.bias`` (the
        checkpoint's mask buffer), transpose the four Conv1D matrices
        ``[in, out] -> [out, in]`` where the un-prefixed name is present, and
        put ``model.`` before every name that lacks it.  Beyond the reference:
        a leading ``transformer.`` is stripped, ``attn.masked_bias`` is
        dropped, and an ``lm_head.weight`` is accepted only if it equals
        ``wte.weight`` (the head is tied).
        """
        w = {}
        for k, v in weights.items():
            w[k[len("transformer.") :] if k.startswith("transformer.") else k] = v
        head = w.pop("lm_head.weight", None)
        if head is None:
            head = w.pop("model.lm_head.weight", None)
        for i in range(self.args.n_layer):
            for drop in (f"h.{i}.attn.bias", f"h.{i}.attn.masked_bias"):
                w.pop(drop, None)
            for t in _CONV1D:
                key = f"h.{i}.{t}.weight"
                if key in w:
                    w[key] = w[key].transpose(1, 0)
        out = {}
        for k, v in w.items():
            out[k if k.startswith("model.") else "model." + k] = v
        if head is not None:
            wte = out.get("model.wte.weight")
            if wte is None or head.shape != wte.shape or not torch.equal(head, wte):
                raise ValueError("lm_head.weight differs from wte.weight, but GPT-2's head is tied")
        return out

    @staticmethod
    def random_weights(args: ModelArgs, seed, scheme="a"):
        """Seeded tensors in a checkpoint's names and layouts (Conv1D ``[in, out]``).

        Embeddings and linear weights ~ N(0, 0.02); both ``c_proj`` weights
        ~ N(0, 0.02 / sqrt(2 n_layer)).  Scheme ``a``: biases 0, norm scale 1,
        shift 0.  Scheme ``b``: biases and shifts ~ N(0, 0.02), scales
        ~ 1 + N(0, 0.1).  Drawn in float32 in a fixed order of names.
        """
        if scheme not in ("a", "b"):
            raise ValueError(f"unknown random-weight scheme '{scheme}'")
        g = torch.Generator().manual_seed(int(seed))
        D, F = args.n_embd, args.n_inner
        proj_std = 0.02 / math.sqrt(2 * args.n_layer)

        def normal(shape, std):
            return torch.randn(shape, generator=g, dtype=torch.float32) * std

        def bias(n):
            return normal((n,), 0.02) if scheme == "b" else torch.zeros(n)

        def scale(n):
            return 1.0 + normal((n,), 0.1) if scheme == "b" else torch.ones(n)

        t = {"wte.weight": normal((args.vocab_size, D), 0.02), "wpe.weight": normal((args.n_positions, D), 0.02)}
        for i in range(args.n_layer):
            p = f"h.{i}."
            t[p + "ln_1.weight"], t[p + "ln_1.bias"] = scale(D), bias(D)
            t[p + "attn.c_attn.weight"], t[p + "attn.c_attn.bias"] = normal((D, 3 * D), 0.02), bias(3 * D)
            t[p + "attn.c_proj.weight"], t[p + "attn.c_proj.bias"] = normal((D, D), proj_std), bias(D)
            t[p + "ln_2.weight"], t[p + "ln_2.bias"] = scale(D), bias(D)
            t[p + "mlp.c_fc.weight"], t[p + "mlp.c_fc.bias"] = normal((D, F), 0.02), bias(F)
            t[p + "mlp.c_proj.weight"], t[p + "mlp.c_proj.bias"] = normal((F, D), proj_std), bias(D)
        t["ln_f.weight"], t["ln_f.bias"] = scale(D), bias(D)
        return t
