"""The tests' own small Gemma-2 configurations; they differ in every size and option."""
import os

import torch

from trapetum_amd.config import Gemma2Config
from trapetum_amd.weights import write_model_folder

TINY_A = dict(
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    intermediate_size=128, vocab_size=256, rms_norm_eps=1e-6, rope_theta=10000.0, sliding_window=8,
    query_pre_attn_scalar=16, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
    hidden_activation="gelu_pytorch_tanh", max_position_embeddings=8192, eos_token_id=1, bos_token_id=2)
TINY_A_INIT = dict(seed=0, sigma=0.02, sigma_norm=0.1)
TINY_A_PROMPTS = (5, 11, 17)

TINY_B = dict(
    num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
    intermediate_size=320, vocab_size=512, rms_norm_eps=1e-5, rope_theta=500.0, sliding_window=16,
    query_pre_attn_scalar=24, attn_logit_softcapping=20.0, final_logit_softcapping=None,
    hidden_activation="gelu_pytorch_tanh", max_position_embeddings=4096, eos_token_id=[1, 107])
TINY_B_INIT = dict(seed=1, sigma=0.05, sigma_norm=0.2)
TINY_B_PROMPTS = (1, 9, 23, 40)

# head size 48 (a step of 16 that is no power of two), three query heads on three kv heads, a window
# that is no multiple of anything, a width and a vocabulary that are no power of two
TINY_C = dict(
    num_hidden_layers=4, hidden_size=88, num_attention_heads=3, num_key_value_heads=3, head_dim=48,
    intermediate_size=200, vocab_size=331, rms_norm_eps=1e-4, rope_theta=37.0, sliding_window=5,
    query_pre_attn_scalar=31.0, attn_logit_softcapping=8.0, final_logit_softcapping=11.0,
    hidden_activation="gelu_pytorch_tanh", eos_token_id=7)
TINY_C_INIT = dict(seed=5, sigma=0.08, sigma_norm=0.3)

# sizes that the matrix-core kernels do not take (a width that is no multiple of 8, a head size that is no multiple
# of 16): the plain kernels must carry the whole model, in both precisions
TINY_D = dict(
    num_hidden_layers=2, hidden_size=100, num_attention_heads=5, num_key_value_heads=5, head_dim=24,
    intermediate_size=52, vocab_size=101, rms_norm_eps=1e-6, rope_theta=100.0, sliding_window=7,
    query_pre_attn_scalar=24, attn_logit_softcapping=30.0, final_logit_softcapping=None,
    hidden_activation="gelu_pytorch_tanh", eos_token_id=3)
TINY_D_INIT = dict(seed=6, sigma=0.06, sigma_norm=0.2)

CONFIGS = {"A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT), "C": (TINY_C, TINY_C_INIT), "D": (TINY_D, TINY_D_INIT)}


def make_folder(tmp_path, which, name=None, **overrides):
    """A model folder of one of the tiny configurations; `overrides` replace config keys (folder `name` then)."""
    cfg_kw, init = CONFIGS[which]
    cfg = Gemma2Config.from_kwargs(**dict(cfg_kw, **overrides))
    folder = os.path.join(str(tmp_path), name or f"tiny_{which}")
    write_model_folder(cfg, folder, **init)
    return folder


def random_tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_l2(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float(torch.linalg.norm(got - ref) / torch.linalg.norm(ref))
