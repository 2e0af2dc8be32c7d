"""Configuration and registry."""
import json

import pytest

from trapetum_amd.config import ConfigError, Gemma2Config
from trapetum_amd.registry import architecture, architectures, config_from_folder

from .tiny import TINY_A, TINY_B


def test_reads_its_keys():
    c = Gemma2Config.from_kwargs(**TINY_B)
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (3, 96, 6, 1, 32)
    assert c.final_logit_softcapping is None and c.attn_logit_softcapping == 20.0
    assert c.eos_token_id == (1, 107)
    assert Gemma2Config.from_kwargs(**TINY_A).eos_token_id == (1,)            # a number or a list (serve.rs:88-101)
    assert [c.layer_is_local(l) for l in range(3)] == [True, False, True]


def test_round_trip_through_config_json(tmp_path):
    c = Gemma2Config.from_kwargs(**TINY_B)
    d = c.to_dict()
    assert d["architectures"] == ["Gemma2ForCausalLM"] and d["final_logit_softcapping"] is None
    (tmp_path / "config.json").write_text(json.dumps(d))
    arch, again = config_from_folder(str(tmp_path))
    assert arch.name == "Gemma2ForCausalLM" and again == c


@pytest.mark.parametrize("key", ["num_hidden_layers", "hidden_size", "head_dim", "rms_norm_eps", "rope_theta",
                                 "sliding_window", "query_pre_attn_scalar", "vocab_size", "intermediate_size"])
def test_missing_key_is_named(key):
    d = dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Gemma2Config.from_kwargs(**d)


def test_bad_values():
    with pytest.raises(ConfigError, match="no multiple"):
        Gemma2Config.from_kwargs(**dict(TINY_A, num_attention_heads=5))
    with pytest.raises(ConfigError, match="integer"):
        Gemma2Config.from_kwargs(**dict(TINY_A, hidden_size="64"))
    with pytest.raises(ConfigError, match="even"):
        Gemma2Config.from_kwargs(**dict(TINY_A, head_dim=15))
    with pytest.raises(ConfigError, match="gelu"):
        Gemma2Config.from_kwargs(**dict(TINY_A, hidden_activation="silu"))
    with pytest.raises(ConfigError, match="layer_types"):
        Gemma2Config.from_kwargs(**dict(TINY_A, layer_types=["full_attention"]))
    assert Gemma2Config.from_kwargs(**dict(TINY_A, attn_logit_softcapping=0.0)).attn_logit_softcapping is None
    with pytest.raises(ConfigError, match="attention_bias"):          # read, and refused: never dropped in silence
        Gemma2Config.from_kwargs(**dict(TINY_A, attention_bias=True))
    assert Gemma2Config.from_kwargs(**dict(TINY_A, attention_bias=False)).attention_bias is False
    c = Gemma2Config.from_kwargs(**dict(TINY_A, layer_types=["full_attention", "sliding_attention"]))
    assert [c.layer_is_local(l) for l in range(2)] == [False, True]


def test_registry(tmp_path):
    assert "Gemma2ForCausalLM" in architectures()
    with pytest.raises(ConfigError, match="unsupported architecture 'LlamaForCausalLM'"):
        architecture("LlamaForCausalLM")
    (tmp_path / "config.json").write_text(json.dumps({"hidden_size": 8}))
    with pytest.raises(ConfigError, match="architectures"):
        config_from_folder(str(tmp_path))
    with pytest.raises(FileNotFoundError):
        config_from_folder(str(tmp_path / "nothing"))


def test_spec_follows_the_configuration():
    spec = architecture("Gemma2ForCausalLM").build_spec(Gemma2Config.from_kwargs(**TINY_B))
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    m0, m1 = spec.layers[0].mixer[1], spec.layers[1].mixer[1]
    assert m0["window"] == 16 and m1["window"] is None
    assert abs(m0["query_scale"] - 24 ** -0.5) < 1e-12 and m0["softcap"] == 20.0
    assert spec.head[1]["softcap"] is None and spec.head_prefix == spec.embedding_prefix
    assert spec.layers[2].prefixes["post_ff_norm"] == "model.layers.2.post_feedforward_layernorm."
    assert spec.stop_ids == (1, 107)
