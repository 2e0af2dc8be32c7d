"""Gemma-2's configuration, by its config.json keys.

The reference's exporter reads the same attributes (model/export_gemma.py:40-46)
and refuses models whose query_pre_attn_scalar differs from head_dim
(model/export_gemma.py:47) or whose sizes are no multiple of 256 (:48-49);
neither limit exists here.  Which layers are local is not in the reference at
all (runtime/src/lib.rs:4455: "not modeled"): even layers use the sliding
window, odd layers see every key, unless config.json lists `layer_types`.
"""
import dataclasses

from .base import ConfigError, ModelConfig, key

_GELU_TANH_NAMES = ("gelu_pytorch_tanh", "gelu_tanh", "gelu_new")


@dataclasses.dataclass
class Gemma2Config(ModelConfig):
    architecture = "Gemma2ForCausalLM"

    num_hidden_layers: int = key("num_hidden_layers", "int", doc="number of decoder layers")
    hidden_size: int = key("hidden_size", "int", doc="width of the residual stream")
    num_attention_heads: int = key("num_attention_heads", "int", doc="query heads")
    num_key_value_heads: int = key("num_key_value_heads", "int", doc="key/value heads")
    head_dim: int = key("head_dim", "int", doc="size of one head (not hidden_size / heads)")
    intermediate_size: int = key("intermediate_size", "int", doc="feed-forward width")
    vocab_size: int = key("vocab_size", "int", doc="rows of the embedding table")
    rms_norm_eps: float = key("rms_norm_eps", "float", doc="epsilon inside every RMSNorm")
    rope_theta: float = key("rope_theta", "float", doc="base of the rotary frequencies")
    sliding_window: int = key("sliding_window", "int", doc="keys a local layer sees, the query's own included")
    query_pre_attn_scalar: float = key("query_pre_attn_scalar", "float", doc="scores are scaled by its inverse square root")
    attn_logit_softcapping: float = key("attn_logit_softcapping", "opt_float", None, doc="cap of attention scores; null = off")
    final_logit_softcapping: float = key("final_logit_softcapping", "opt_float", None, doc="cap of the logits; null = off")
    hidden_activation: str = key("hidden_activation", "str", "gelu_pytorch_tanh", doc="gate activation")
    tie_word_embeddings: bool = key("tie_word_embeddings", "bool", True, doc="head shares the embedding table")
    max_position_embeddings: int = key("max_position_embeddings", "opt_int", None, doc="longest trained context")
    eos_token_id: tuple = key("eos_token_id", "int_list", (), doc="stop tokens")
    bos_token_id: int = key("bos_token_id", "opt_int", None, doc="begin-of-sequence token")
    pad_token_id: int = key("pad_token_id", "opt_int", None, doc="padding token")
    layer_types: tuple = key("layer_types", "str_list", None, doc="per layer: sliding_attention or full_attention")
    attention_bias: bool = key("attention_bias", "bool", False, doc="biases on the attention projections (Gemma-2 has none)")

    def validate(self):
        for name in ("hidden_size", "num_attention_heads", "num_key_value_heads",
                     "head_dim", "intermediate_size", "vocab_size", "sliding_window"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config key '{name}' must be positive, found {getattr(self, name)}")
        if self.num_hidden_layers < 0:      # none at all is a model too: embedding, final norm, head
            raise ConfigError(f"config key 'num_hidden_layers' must not be negative, found {self.num_hidden_layers}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) is no multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotary pairs")
        if self.rms_norm_eps <= 0 or self.rope_theta <= 0 or self.query_pre_attn_scalar <= 0:
            raise ConfigError("rms_norm_eps, rope_theta and query_pre_attn_scalar must be positive")
        if self.hidden_activation not in _GELU_TANH_NAMES:
            raise ConfigError(
                f"hidden_activation '{self.hidden_activation}' is not a tanh-approximated gelu "
                f"(one of {', '.join(_GELU_TANH_NAMES)})")
        for name in ("attn_logit_softcapping", "final_logit_softcapping"):
            v = getattr(self, name)
            if v is not None and v <= 0:          # the reference writes 0 for "off" (model/export_gemma.py:44-45)
                setattr(self, name, None)
        if self.attention_bias:               # no released Gemma-2 has them, and the reference's exporter reads none (model/export_gemma.py:53-61)
            raise ConfigError("attention_bias is true: projections with a bias are not built (the products have no bias operand)")
        if self.layer_types is not None:
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError(
                    f"layer_types has {len(self.layer_types)} entries for {self.num_hidden_layers} layers")
            for t in self.layer_types:
                if t not in ("sliding_attention", "full_attention"):
                    raise ConfigError(f"layer_types entry '{t}' is neither sliding_attention nor full_attention")

    def layer_is_local(self, layer):
        if self.layer_types is not None:
            return self.layer_types[layer] == "sliding_attention"
        return layer % 2 == 0

    def to_dict(self):
        d = super().to_dict()
        d["model_type"] = "gemma2"
        if d.get("layer_types") is None:
            d.pop("layer_types", None)
        if not d.get("attention_bias"):
            d.pop("attention_bias", None)
        return d
