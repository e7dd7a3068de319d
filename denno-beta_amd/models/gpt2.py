"""GPT-2 as a DecoderSpec: learned token and position tables, pre-LayerNorm blocks of fused-QKV
causal attention with biases and a GELU MLP, final LayerNorm, tied head
(crates/denno-engine/src/model/gpt2.rs:50-119 for names and shapes, :135-233 for the order).

Checkpoints store the four matrices of a block [in, out] (Conv1D); they are transposed once
at load.  Names are read with or without the `transformer.` prefix; the `attn.bias` and
`attn.masked_bias` buffers of some files are not weights; `lm_head.weight`, if a file has it,
repeats the token table.
"""
from __future__ import annotations

import math

from ..config.gpt2 import GPT2Config
from ..config.registry import register_architecture
from ..parts.model import DecoderSpec, LayerCall, LayerSpec


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
        layers.append(LayerSpec(
            arrangement="pre_norm",
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
        ))
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
