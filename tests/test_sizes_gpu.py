"""Real layer sizes on the GPU: two layers of the 2B configuration (head size 256, width 2304, a vocabulary that
is no power of two) and the 27B head geometry (head size 128, query scale that differs from the head size), the
bfloat16 engine against the float32 engine on the same weights, prefill and decode, with a window small enough
to cut in."""
import pytest
import torch

from trapetum_amd.config import Gemma2Config
from trapetum_amd.engine import Engine

from .tiny import random_tokens, rel_l2

pytestmark = pytest.mark.gpu

SIZES = {
    "2b": dict(num_hidden_layers=2, hidden_size=2304, num_attention_heads=8, num_key_value_heads=4, head_dim=256,
               intermediate_size=9216, vocab_size=25601, rms_norm_eps=1e-6, rope_theta=10000.0, sliding_window=96,
               query_pre_attn_scalar=256, attn_logit_softcapping=50.0, final_logit_softcapping=30.0),
    "9b": dict(num_hidden_layers=2, hidden_size=3584, num_attention_heads=16, num_key_value_heads=8, head_dim=256,
               intermediate_size=14336, vocab_size=32003, rms_norm_eps=1e-6, rope_theta=10000.0, sliding_window=128,
               query_pre_attn_scalar=256, attn_logit_softcapping=50.0, final_logit_softcapping=30.0),
    "27b-heads": dict(num_hidden_layers=2, hidden_size=1152, num_attention_heads=32, num_key_value_heads=16, head_dim=128,
                      intermediate_size=4608, vocab_size=10007, rms_norm_eps=1e-6, rope_theta=10000.0, sliding_window=80,
                      query_pre_attn_scalar=144, attn_logit_softcapping=50.0, final_logit_softcapping=30.0),
}


@pytest.mark.parametrize("which", list(SIZES))
def test_bfloat16_engine_follows_float32_engine(which):
    cfg = Gemma2Config.from_kwargs(**SIZES[which])
    engines = {dt: Engine.from_config(cfg, seed=2, sigma=0.02, dtype=dt, max_tokens_in_cache=2048, use_graph=False)
               for dt in ("float32", "bfloat16")}
    lens = [150, 37, 260]
    seqs = [random_tokens(n + 5, cfg.vocab_size, 40 + i) for i, n in enumerate(lens)]
    out = {}
    for dt, e in engines.items():
        slots = [e.cache.acquire() for _ in lens]
        flat = [t for s, n in zip(seqs, lens) for t in s[:n]]
        rows = [e.model.step(e.cache, slots, flat, counts=lens, want=[lens[0] - 1, lens[0] + lens[1] - 1, sum(lens) - 1, 0, 200])]
        for step in range(5):
            rows.append(e.model.step(e.cache, slots, [s[n + step] for s, n in zip(seqs, lens)]))
        out[dt] = torch.cat(rows).float().cpu()
        for s in slots:
            e.cache.release(s)
    ref, got = out["float32"], out["bfloat16"]
    assert torch.isfinite(ref).all() and torch.isfinite(got).all()
    assert rel_l2(got, ref) < 2e-2
    worst = max(rel_l2(got[i], ref[i]) for i in range(ref.shape[0]))
    assert worst < 4e-2, worst
    # where float32 is sure of its first choice, bfloat16 makes the same one
    top2 = ref.topk(2, dim=-1).values
    sure = (top2[:, 0] - top2[:, 1]) > 0.05 * ref.abs().max()
    assert torch.equal(got.argmax(-1)[sure], ref.argmax(-1)[sure])
