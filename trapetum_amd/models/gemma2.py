"""Gemma-2 as data: which parts stand where, under which tensor names.

Formulas and their order follow the reference's Gemma path (runtime/src/lib.rs:
4450-4605); tensor names are the checkpoint's own, as the reference's exporter
walks them (model/export_gemma.py:60-73).  What the reference leaves out is set
here from config.json: the query scale 1/sqrt(query_pre_attn_scalar) (the reference
refuses models where it differs from head_dim, model/export_gemma.py:47) and the
sliding window on local layers (runtime/src/lib.rs:4455).
"""
import math

from ..config.gemma2 import Gemma2Config
from ..registry import register_architecture
from .spec import LayerSpec, ModelSpec, ScheduleEntry


def build_spec(c: Gemma2Config) -> ModelSpec:
    norm = ("rms_norm", {"size": c.hidden_size, "eps": c.rms_norm_eps, "weight_offset": 1.0})
    layers = []
    for l in range(c.num_hidden_layers):
        p = f"model.layers.{l}."
        mixer = ("attention", {
            "hidden_size": c.hidden_size, "num_heads": c.num_attention_heads,
            "num_kv_heads": c.num_key_value_heads, "head_dim": c.head_dim,
            "query_scale": 1.0 / math.sqrt(c.query_pre_attn_scalar),
            "softcap": c.attn_logit_softcapping,
            "window": c.sliding_window if c.layer_is_local(l) else None,
            "position": ("rope", {"rotary_dim": c.head_dim, "theta": c.rope_theta}),
        })
        ff = ("gated_mlp", {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size,
                            "activation": "gelu_tanh"})
        layers.append(LayerSpec(
            block=("sandwich", {}), mixer=mixer, feed_forward=ff, norm=norm,
            prefixes={"pre_mixer_norm": p + "input_layernorm.", "mixer": p + "self_attn.",
                      "post_mixer_norm": p + "post_attention_layernorm.",
                      "pre_ff_norm": p + "pre_feedforward_layernorm.", "feed_forward": p + "mlp.",
                      "post_ff_norm": p + "post_feedforward_layernorm."}))
    head_prefix = "model.embed_tokens." if c.tie_word_embeddings else "lm_head."
    return ModelSpec(
        architecture=c.architecture, hidden_size=c.hidden_size, vocab_size=c.vocab_size,
        embedding=("scaled_embedding", {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size,
                                        "scale": math.sqrt(c.hidden_size)}),
        embedding_prefix="model.embed_tokens.",
        layers=layers,
        schedule=[ScheduleEntry(l) for l in range(c.num_hidden_layers)],
        final_norm=norm, final_norm_prefix="model.norm.",
        head=("linear_head", {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size,
                              "softcap": c.final_logit_softcapping}),
        head_prefix=head_prefix,
        stop_ids=tuple(c.eos_token_id))


register_architecture(Gemma2Config.architecture, Gemma2Config, build_spec)
