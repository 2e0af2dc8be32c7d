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
    # where float32 is sure of its first choice, bfloat16 makes the same one; "sure": ahead of the second choice by
    # three times the largest difference the two engines have anywhere, which at these sizes is most of the rows
    top2 = ref.topk(2, dim=-1).values
    sure = (top2[:, 0] - top2[:, 1]) > 3 * (got - ref).abs().max()
    assert float(sure.float().mean()) >= 0.25, float(sure.float().mean())
    assert torch.equal(got.argmax(-1)[sure], ref.argmax(-1)[sure])


def test_float32_engine_meets_the_plain_implementation_at_real_widths(tmp_path):
    """Two layers of the 2B sizes (width 2,304, heads of 256, a feed-forward of 9,216), float32 engine against the plain
    implementation on the same folder: prompts of 40 and 150 tokens in one step, then 5 tokens decoded one by one.
    The bfloat16 engine is held to the float32 engine above, so the chain ends at the plain implementation (the
    reference's forward: runtime/src/lib.rs:4527-4540 for a layer, :1300-1361 for its kernels' order)."""
    import os
    from trapetum_amd import load_model
    from trapetum_amd.weights import write_model_folder
    from .plain import gemma2_plain as plain
    cfg = Gemma2Config.from_kwargs(**dict(SIZES["2b"], vocab_size=5003))
    folder = os.path.join(str(tmp_path), "two_layers_2b")
    write_model_folder(cfg, folder, seed=2, sigma=0.02, sigma_norm=0.1)
    pcfg, pw = plain.read_folder(folder)
    lens = [40, 150]
    seqs = [random_tokens(n + 5, cfg.vocab_size, 90 + i) for i, n in enumerate(lens)]
    ref = [plain.forward(pcfg, pw, s) for s in seqs]
    e = load_model(folder, dtype="float32", max_tokens_in_cache=1024, use_graph=False)
    slots = [e.cache.acquire() for _ in lens]
    out = e.model.step(e.cache, slots, [t for s, n in zip(seqs, lens) for t in s[:n]], counts=lens, want=list(range(sum(lens))))
    got = [[out[:40]], [out[40:]]]
    for step in range(5):
        o = e.model.step(e.cache, slots, [s[n + step] for s, n in zip(seqs, lens)])
        got[0].append(o[0:1]), got[1].append(o[1:2])
    for i in range(2):
        g = torch.cat(got[i]).double().cpu()
        assert rel_l2(g, ref[i]) < 1e-5, i
        assert max(rel_l2(g[r], ref[i][r]) for r in range(g.shape[0])) < 3e-5, i


def test_generate_at_real_sizes_with_and_without_graphs():
    """generate() on two layers of the 2B sizes with the real vocabulary of 256,000: 8 prompts of unequal lengths that
    run into the context's end at different steps (the batch shrinks into smaller graphs), token choice inside the
    captured graph.  float32 steps give the same logits whatever else is in the batch, so the ids with graphs are the
    ids without, greedy and sampled; in bfloat16 (whose decode attention cuts the keys into other slices in a graph than
    in an eager step, so a close call between two tokens may fall the other way) both ways give every request the same
    first token, the same number of tokens and the same reason to end."""
    cfg = Gemma2Config.from_kwargs(**dict(SIZES["2b"], vocab_size=256000))
    lens = [30, 64, 100, 17, 50, 200, 5, 90]
    prompts = [random_tokens(n, cfg.vocab_size, 30 + i) for i, n in enumerate(lens)]
    for dt in ("float32", "bfloat16"):
        got = {}
        for use_graph in (True, False):
            e = Engine.from_config(cfg, seed=2, sigma=0.02, dtype=dt, max_tokens_in_cache=4096, max_context=230, max_batch=8,
                                   use_graph=use_graph, draw_on_device=True)
            got[use_graph] = (e.generate(prompts, max_tokens=220, stop_ids=(), with_reasons=True),
                              e.generate(prompts, max_tokens=220, temperature=0.8, top_k=50, top_p=0.9, seed=3, stop_ids=(),
                                         with_reasons=True))
            assert e.cache.live_slots() == []
            if use_graph:
                assert len({k[0] for k in e.graphed.graphs}) >= 3         # the batch went through graphs of several sizes
            del e
            torch.cuda.empty_cache()
        for a, b in zip(got[True], got[False]):
            assert [r.reason for r in a] == [r.reason for r in b]
            assert [len(r.tokens) for r in a] == [min(220, 231 - n) for n in lens] == [len(r.tokens) for r in b]
            assert {r.reason for r in a} == {"context", "length"}
            assert [r.tokens[0] for r in a] == [r.tokens[0] for r in b]
            if dt == "float32":
                assert [r.tokens for r in a] == [r.tokens for r in b]


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
        assert [g.pages.rows_cap for g in e.cache.token_groups] == [4096, None]
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
        if dt == "bfloat16":
            # the same tokens again in portions of 1,024 (the last ones cross the ring's end and take the places of
            # positions that their own earlier rows still see), then one by one while a second request joins at the
            # tenth step with its whole prompt in the step of the first one's single token
            e = Engine.from_config(cfg, seed=2, sigma=0.02, dtype=dt, max_tokens_in_cache=8192, max_context=8192, max_batch=4,
                                   use_graph=False)
            s = e.cache.acquire()
            rows = []
            for a in range(0, 4200, 1024):
                b = min(4200, a + 1024)
                want = [w - a for w in (4095, 4096, 4199) if a <= w < b]
                o = e.model.step(e.cache, [s], toks[a:b], counts=[b - a], want=want)
                if o is not None:
                    rows.append(o)
            other = random_tokens(300, cfg.vocab_size, 78)
            for i in range(4200, 4240):
                if i == 4210:
                    s2 = e.cache.acquire()
                    o = e.model.step(e.cache, [s, s2], [toks[i]] + other, counts=[1, 300], want=[0, 300])
                    rows.append(o[0:1])
                    joined = o[1:2]
                elif i > 4210:
                    rows.append(e.model.step(e.cache, [s, s2], [toks[i], other[(i * 7) % 300]])[0:1])
                else:
                    rows.append(e.model.step(e.cache, [s], [toks[i]]))
            out["portions"] = torch.cat(rows).float().cpu()
            s3 = e.cache.acquire()                           # the joining request alone: its last logits are the same
            alone = e.model.step(e.cache, [s3], other, counts=[300])
            assert rel_l2(joined, alone) < 4e-3
            del e
            torch.cuda.empty_cache()
    ref, got = out["float32"], out["bfloat16"]
    assert torch.isfinite(ref).all() and torch.isfinite(got).all()
    assert rel_l2(got, ref) < 2e-2
    assert max(rel_l2(got[i], ref[i]) for i in range(ref.shape[0])) < 4e-2
    assert out["portions"].shape == ref.shape
    assert rel_l2(out["portions"], ref) < 2e-2
    assert max(rel_l2(out["portions"][i], ref[i]) for i in range(ref.shape[0])) < 4e-2


class _Tensors:
    """A weight source over a dict of tensors."""

    def __init__(self, tensors):
        self.t = tensors

    def names(self):
        return list(self.t)

    def shape(self, name):
        return tuple(self.t[name].shape)

    def dtype(self, name):
        return self.t[name].dtype

    def tensor(self, name):
        return self.t[name]


def test_the_real_windows_edge_with_a_key_that_stands_out():
    """Random weights make attention near-uniform over 4,096 keys: one key more or less at the window's edge moves the
    logits by a four-thousandth, which no tolerance sees.  Here one (local) layer of the 2B sizes is made so that the
    key of token A is the query of token B (B's embedding is A's with its halves swapped, the key projection is the
    first query head's with its columns swapped the same way, both doubled): A stands once, at position P, and B at
    P + 4,095, where A's key is the oldest one still seen and takes nearly all the weight, and at P + 4,096, where it
    has just left.  Both rows, and their neighbours, must follow the float32 engine through a prompt that ends before
    them and decode steps (the fused kernel, every other step from a graph) and through the whole prompt in one step
    (the prefill kernel); an edge off by one in either direction changes one of the two rows altogether."""
    from trapetum_amd.engine.model import Model
    from trapetum_amd.engine.runtime import Runtime
    from trapetum_amd.registry import architecture
    from trapetum_amd.weights import RandomWeights, load_into
    cfg = Gemma2Config.from_kwargs(**dict(SIZES["2b"], num_hidden_layers=1, sliding_window=4096, vocab_size=2003))
    D, hd, G = cfg.hidden_size, cfg.head_dim, cfg.num_attention_heads // cfg.num_key_value_heads
    P, A, B = 70, 1998, 1999
    toks = [t if t not in (A, B) else 5 for t in random_tokens(P + 4096 + 8, cfg.vocab_size, 79)]
    toks[P], toks[P + 4095], toks[P + 4096] = A, B, B
    arch = architecture(cfg.architecture)
    out = {}
    for dt in ("float32", "bfloat16"):
        model = Model(arch.build_spec(cfg), Runtime(dtype=dt, device="cuda:0"))
        src = RandomWeights(model.tensor_layout(), 2, 0.02, 0.1)
        t = {name: src.tensor(name).clone() for name in src.names()}
        emb, pre = "model.embed_tokens.weight", "model.layers.0."
        t[emb][B] = torch.roll(t[emb][A], D // 2)
        t[pre + "input_layernorm.weight"].zero_()
        q = t[pre + "self_attn.q_proj.weight"]
        q *= 2.0
        for g in range(cfg.num_key_value_heads):
            t[pre + "self_attn.k_proj.weight"][g * hd:(g + 1) * hd] = torch.roll(q[g * G * hd:(g * G + 1) * hd], D // 2, dims=1)
        load_into(model, _Tensors(t))
        e = Engine(model, cfg, max_tokens_in_cache=8192, max_context=8192, max_batch=2)
        s = e.cache.acquire()
        n0 = P + 4090
        rows = [e.model.step(e.cache, [s], toks[:n0], counts=[n0], want=[n0 - 1])]
        for i in range(n0, len(toks)):
            if dt == "bfloat16" and i % 2:
                rows.append(e.graphed.step([s], [toks[i]]).clone())
            else:
                rows.append(e.model.step(e.cache, [s], [toks[i]]))
        e.cache.release(s)
        s = e.cache.acquire()                                # and the whole prompt in one step
        rows.append(e.model.step(e.cache, [s], toks, counts=[len(toks)], want=[P + 4094, P + 4095, P + 4096, P + 4097]))
        out[dt] = torch.cat(rows).float().cpu()
        if dt == "float32":                                  # what the plain implementation makes of the same tensors
            from .plain import gemma2_plain as plain
            # (angles formed in 32-bit, as the reference and the engine form them: at these positions their rounding
            # alone moves the logits by some 1e-5)
            truth = plain.forward(cfg.to_dict(), {name: w.double() for name, w in t.items()}, toks, angle_dtype=torch.float32)
        del e, model
        torch.cuda.empty_cache()
    ref, got = out["float32"], out["bfloat16"]
    base = P + 4089                                          # row r of the decoded part is position base + r
    # the float32 engine at the edge is what the plain implementation (the whole sequence at once, no cache, no ring) gives
    for r in range(ref.shape[0] - 4):
        assert rel_l2(ref[r].double(), truth[base + r]) < 1e-5, r
    inside, outside = ref[P + 4095 - base], ref[P + 4096 - base]
    # the planted key matters: the same query token gives other logits once the key has left the window
    assert rel_l2(inside, outside) > 0.2, rel_l2(inside, outside)
    for r in range(ref.shape[0]):
        assert rel_l2(got[r], ref[r]) < 4e-2, r
    whole = ref[-4:]
    assert rel_l2(whole[1], inside) < 1e-4 and rel_l2(whole[2], outside) < 1e-4      # whole prompt = step by step (float32)
    assert rel_l2(got[-3], got[P + 4095 - base]) < 2e-2 and rel_l2(got[-2], got[P + 4096 - base]) < 2e-2
