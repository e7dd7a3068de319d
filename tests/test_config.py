import json

import pytest

from conftest import TINY_A, TINY_B
from denno_beta_amd.config import (ConfigError, EngineOptions, known_architectures, load_config,
                                   resolve_architecture)
from denno_beta_amd.models.gpt2 import GPT2Config


def test_reads_every_key():
    c = GPT2Config.from_dict(TINY_B)
    assert (c.n_layer, c.n_embd, c.n_head, c.head_dim, c.inner_dim) == (3, 96, 2, 48, 320)
    assert (c.vocab_size, c.n_positions, c.layer_norm_epsilon) == (1000, 256, 1e-6)
    assert c.activation == "gelu_erf" and c.scale_attn_by_inverse_layer_idx and c.scale_attn_weights
    a = GPT2Config.from_dict(TINY_A)
    assert a.activation == "gelu_tanh" and a.inner_dim == 256 and not a.scale_attn_by_inverse_layer_idx


def test_defaults_are_the_reference_s_fixed_values():
    # crates/denno-engine/src/model/gpt2.rs:80-82, 154, 174; tensor.rs:1156-1161
    c = GPT2Config.from_dict(dict(n_layer=1, n_embd=32, n_head=2, vocab_size=60000, n_ctx=64))
    assert c.inner_dim == 128 and c.layer_norm_epsilon == 1e-5 and c.activation == "gelu_tanh"
    assert c.n_positions == 64                      # n_ctx, the key the reference reads (gpt2.rs:53)
    assert c.eos_token_id == 50256                  # gpt2.rs:56
    assert GPT2Config.from_dict(dict(TINY_A)).eos_token_id is None   # a vocabulary without that id


@pytest.mark.parametrize("key", ["n_layer", "n_embd", "n_head", "vocab_size", "n_positions"])
def test_missing_key_is_named(key):
    d = dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        GPT2Config.from_dict(d)


def test_bad_values():
    with pytest.raises(ConfigError, match="n_head"):
        GPT2Config.from_dict(dict(TINY_A, n_head=5))
    with pytest.raises(ConfigError, match="activation_function"):
        GPT2Config.from_dict(dict(TINY_A, activation_function="relu"))
    with pytest.raises(ConfigError, match="integer"):
        GPT2Config.from_dict(dict(TINY_A, n_layer="2"))
    with pytest.raises(ConfigError, match="tie_word_embeddings"):
        GPT2Config.from_dict(dict(TINY_A, tie_word_embeddings=False))


def test_registry():
    assert resolve_architecture({"architectures": ["GPT2LMHeadModel"]}).name == "GPT2LMHeadModel"
    assert resolve_architecture({"model_type": "gpt2"}).name == "GPT2LMHeadModel"    # model/mod.rs:94-95
    with pytest.raises(ConfigError, match="LlamaForCausalLM"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="names no architecture"):
        resolve_architecture({})
    assert "GPT2LMHeadModel" in known_architectures()


def test_load_config_from_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, cfg = load_config(str(tmp_path))
    spec = arch.build(cfg)
    assert len(spec.layers) == 3 and spec.vocab == 1000 and spec.max_positions == 256
    # every size of the spec comes from the config
    assert spec.layers[2].parts["mixer"][1]["scale"] == pytest.approx(1 / (48 ** 0.5) / 3)
    assert spec.layers[0].parts["ffn"][1]["inner"] == 320 and spec.layers[0].parts["norm1"][1]["eps"] == 1e-6
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path / "nowhere"))


def test_engine_options():
    EngineOptions().validate()
    with pytest.raises(ValueError, match="dtype"):
        EngineOptions(dtype="float16").validate()
    with pytest.raises(ValueError, match="kv_policy"):
        EngineOptions(kv_policy="swap").validate()
