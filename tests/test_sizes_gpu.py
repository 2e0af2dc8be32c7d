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


@pytest.mark.parametrize("which", ["2b", "27b-heads"])
def test_graph_replays_follow_eager_steps_at_real_sizes(which):
    """Decode steps replayed from graphs against eager steps at real head sizes, with sequences on both sides of a
    graph's bound on the lengths (1024): the slices of the attention's keys follow the bound in a graph and the
    lengths in an eager step, so the two agree to rounding; the rows a graph adds to a batch of three change nothing."""
    from trapetum_amd.engine.graphs import GraphedDecode
    cfg = Gemma2Config.from_kwargs(**dict(SIZES[which], sliding_window=600))
    e = Engine.from_config(cfg, seed=2, sigma=0.02, dtype="bfloat16", max_tokens_in_cache=8192, max_context=4096, use_graph=False)
    model = e.model
    lens = [1015, 300, 1040]
    seqs = [random_tokens(n + 20, cfg.vocab_size, 60 + i) for i, n in enumerate(lens)]
    eager_cache, graph_cache = e.cache, model.new_cache(8192, max_context=4096, max_slots=8)
    graphed = GraphedDecode(model, graph_cache)
    flat = [t for s, n in zip(seqs, lens) for t in s[:n]]
    es = [eager_cache.acquire() for _ in lens]
    gs = [graph_cache.acquire() for _ in lens]
    model.step(eager_cache, es, flat, counts=lens)
    model.step(graph_cache, gs, flat, counts=lens)
    for step in range(20):
        toks = [s[n + step] for s, n in zip(seqs, lens)]
        a = model.step(eager_cache, es, toks).float().cpu()
        b = graphed.step(gs, toks).float().cpu()
        assert rel_l2(b, a) < 4e-3, step
        worst = max(rel_l2(b[i], a[i]) for i in range(3))
        assert worst < 8e-3, (step, worst)
    assert {k[:2] for k in graphed.graphs} == {(4, 2048)}       # the longest sequence sets the bound for all
    # the first sequence alone crosses the bound during its steps: two graphs of one row
    graph_cache.release(gs.pop()), graph_cache.release(gs.pop())
    eager_cache.release(es.pop()), eager_cache.release(es.pop())
    g2, e2 = graph_cache.acquire(), eager_cache.acquire()
    n0 = 1015
    model.step(eager_cache, [e2], seqs[0][:n0], counts=[n0])
    model.step(graph_cache, [g2], seqs[0][:n0], counts=[n0])
    for step in range(16):
        a = model.step(eager_cache, [e2], [seqs[0][n0 + step]]).float().cpu()
        b = graphed.step([g2], [seqs[0][n0 + step]]).float().cpu()
        assert rel_l2(b, a) < 4e-3, step
    assert {(1, 1024), (1, 2048)} <= {k[:2] for k in graphed.graphs}


def test_context_beyond_the_real_window():
    """Two layers of the 2B sizes with the real window of 4,096 keys on pages of 64: a prompt of 4,200 tokens and 40
    decoded ones, so that the local layer's ring has wrapped and its window's edge moves through it; the bfloat16
    engine (matrix-core kernels, fused decode step, graphs) against the float32 engine on the same weights."""
    cfg = Gemma2Config.from_kwargs(**dict(SIZES["2b"], sliding_window=4096))
    toks = random_tokens(4240, cfg.vocab_size, 77)
    out = {}
    for dt in ("float32", "bfloat16"):
        e = Engine.from_config(cfg, seed=2, sigma=0.02, dtype=dt, max_tokens_in_cache=8192, max_context=8192, max_batch=4)
        assert [g.pages.rows_cap for g in e.cache.kv_groups] == [4096, None]
        s = e.cache.acquire()
        rows = [e.model.step(e.cache, [s], toks[:4200], counts=[4200], want=[4095, 4096, 4199])]
        for i in range(4200, 4240):
            if dt == "bfloat16" and i % 2:                   # every other step from a graph
                rows.append(e.graphed.step([s], [toks[i]]).clone())
            else:
                rows.append(e.model.step(e.cache, [s], [toks[i]]))
        out[dt] = torch.cat(rows).float().cpu()
        e.cache.release(s)
        del e
        torch.cuda.empty_cache()
    ref, got = out["float32"], out["bfloat16"]
    assert torch.isfinite(ref).all() and torch.isfinite(got).all()
    assert rel_l2(got, ref) < 2e-2
    assert max(rel_l2(got[i], ref[i]) for i in range(ref.shape[0])) < 4e-2
