"""GPT-2: the architecture's own config.json keys, typed, and the model as a DecoderSpec.

Configuration.  The reference reads n_embd, n_head, n_ctx, vocab_size, n_layer and eos_token_id
(crates/denno-engine/src/model/gpt2.rs:51-56) and fixes eps = 1e-5 (gpt2.rs:154), an MLP
width of 4*n_embd (gpt2.rs:80-82), the tanh GELU (tensor.rs:1156-1161) and a score scale
of 1/sqrt(head) (gpt2.rs:174) in code.  Those four are config keys of the architecture
(layer_norm_epsilon, n_inner, activation_function, scale_attn_weights /
scale_attn_by_inverse_layer_idx); they are read here, and a key that is absent falls
back to what the reference computes.

Model.  Learned token and position tables, pre-LayerNorm blocks of fused-QKV causal attention
with biases and a GELU MLP, final LayerNorm, tied head (gpt2.rs:50-119 for names and shapes,
:135-233 for the order).  Checkpoints store the four matrices of a block [in, out] (Conv1D); they
are transposed once at load.  Names are read with or without the `transformer.` prefix; the
`attn.bias` and `attn.masked_bias` buffers of some files are not weights; `lm_head.weight`, if a
file has it, repeats the token table.
"""
from __future__ import annotations

import math
from dataclasses import asdict, dataclass
from typing import Optional

from ..config.base import ConfigError, read_bool, read_float, read_int, read_str
from ..config.registry import register_architecture
from ..parts.model import DecoderSpec, LayerCall, LayerSpec

ACTIVATION_ALIASES = {
    "gelu_new": "gelu_tanh",
    "gelu_pytorch_tanh": "gelu_tanh",
    "gelu_fast": "gelu_tanh",
    "gelu": "gelu_erf",
}


@dataclass(frozen=True)
class GPT2Config:
    vocab_size: int
    n_positions: int
    n_embd: int
    n_layer: int
    n_head: int
    n_inner: Optional[int]
    activation_function: str
    layer_norm_epsilon: float
    scale_attn_weights: bool
    scale_attn_by_inverse_layer_idx: bool
    tie_word_embeddings: bool
    eos_token_id: Optional[int]
    bos_token_id: Optional[int]

    architecture = "GPT2LMHeadModel"
    model_type = "gpt2"

    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    @property
    def inner_dim(self) -> int:
        return self.n_inner if self.n_inner is not None else 4 * self.n_embd

    @property
    def activation(self) -> str:
        return ACTIVATION_ALIASES[self.activation_function]

    @property
    def max_positions(self) -> int:
        return self.n_positions

    @classmethod
    def from_dict(cls, d: dict) -> "GPT2Config":
        vocab = read_int(d, "vocab_size", minimum=1)
        # the reference's default end-of-sequence id (gpt2.rs:56), where the vocabulary has it
        eos_default = 50256 if vocab > 50256 else None
        cfg = cls(
            vocab_size=vocab,
            n_positions=read_int(d, "n_positions", aliases=("n_ctx",), minimum=1),
            n_embd=read_int(d, "n_embd", minimum=1),
            n_layer=read_int(d, "n_layer", minimum=1),
            n_head=read_int(d, "n_head", minimum=1),
            n_inner=read_int(d, "n_inner", default=None, minimum=1),
            activation_function=read_str(d, "activation_function", default="gelu_new",
                                         choices=ACTIVATION_ALIASES),
            layer_norm_epsilon=read_float(d, "layer_norm_epsilon", default=1e-5),
            scale_attn_weights=read_bool(d, "scale_attn_weights", True),
            scale_attn_by_inverse_layer_idx=read_bool(d, "scale_attn_by_inverse_layer_idx", False),
            tie_word_embeddings=read_bool(d, "tie_word_embeddings", True),
            eos_token_id=read_int(d, "eos_token_id", default=eos_default, minimum=0),
            bos_token_id=read_int(d, "bos_token_id", default=None, minimum=0),
        )
        cfg.validate()
        return cfg

    def validate(self):
        if self.n_embd % self.n_head != 0:
            raise ConfigError(
                f"config.json: n_embd ({self.n_embd}) is not a multiple of n_head ({self.n_head})")
        if self.layer_norm_epsilon < 0:
            raise ConfigError(f"config.json: layer_norm_epsilon must be >= 0, got {self.layer_norm_epsilon}")
        if not self.tie_word_embeddings:
            raise ConfigError(
                "config.json: tie_word_embeddings = false: this architecture's head is the "
                "transposed token table (crates/denno-engine/src/model/gpt2.rs:90-91)")
        if self.eos_token_id is not None and self.eos_token_id >= self.vocab_size:
            raise ConfigError(
                f"config.json: eos_token_id ({self.eos_token_id}) is outside the vocabulary "
                f"({self.vocab_size})")

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = [self.architecture]
        d["model_type"] = self.model_type
        return d


def attention_scale(cfg: GPT2Config, layer_idx: int) -> float:
    """1/sqrt(head) as the reference (gpt2.rs:174) unless scale_attn_weights is false;
    divided by (layer index + 1) if scale_attn_by_inverse_layer_idx."""
    s = 1.0 / math.sqrt(cfg.head_dim) if cfg.scale_attn_weights else 1.0
    if cfg.scale_attn_by_inverse_layer_idx:
        s /= float(layer_idx + 1)
    return s


def build_gpt2(cfg: GPT2Config) -> DecoderSpec:
    E = cfg.n_embd
    layers = []
    for i in range(cfg.n_layer):
        p = f"h.{i}."
        layers.append(LayerSpec(arrangement="pre_norm", parts=dict(
            norm1=("layernorm", dict(width=E, eps=cfg.layer_norm_epsilon, weight_name=p + "ln_1.weight",
                                     bias_name=p + "ln_1.bias")),
            mixer=("causal_attention", dict(
                width=E, n_heads=cfg.n_head, n_kv_heads=cfg.n_head, head_dim=cfg.head_dim,
                scale=attention_scale(cfg, i), qkv_weight=p + "attn.c_attn.weight", qkv_bias=p + "attn.c_attn.bias",
                out_weight=p + "attn.c_proj.weight", out_bias=p + "attn.c_proj.bias", stored_in_out=True,
                window=0)),
            norm2=("layernorm", dict(width=E, eps=cfg.layer_norm_epsilon, weight_name=p + "ln_2.weight",
                                     bias_name=p + "ln_2.bias")),
            ffn=("dense_mlp", dict(
                width=E, inner=cfg.inner_dim, activation=cfg.activation, up_weight=p + "mlp.c_fc.weight",
                up_bias=p + "mlp.c_fc.bias", down_weight=p + "mlp.c_proj.weight", down_bias=p + "mlp.c_proj.bias",
                stored_in_out=True)),
        )))
    return DecoderSpec(
        vocab=cfg.vocab_size, width=E, max_positions=cfg.n_positions,
        token_table="wte.weight",
        position=("learned_absolute", dict(n_positions=cfg.n_positions, width=E, name="wpe.weight")),
        layers=layers,
        run_order=[LayerCall(layer=i, cache=i) for i in range(cfg.n_layer)],
        final_norm=("layernorm", dict(width=E, eps=cfg.layer_norm_epsilon, weight_name="ln_f.weight",
                                      bias_name="ln_f.bias")),
        head_weight=None,
        eos_token_ids=(cfg.eos_token_id,) if cfg.eos_token_id is not None else (),
        name_prefixes=("", "transformer."),
        ignore_tensors=(r"(^|\.)h\.\d+\.attn\.(masked_)?bias$",),
        tied_tensors={"lm_head.weight": "wte.weight"},
    )


register_architecture(["GPT2LMHeadModel", "gpt2"], GPT2Config, build_gpt2)
