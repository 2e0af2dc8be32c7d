"""Generation through the entry point, long decoding, graph replays, sampling: GPU against the plain implementation."""
import pytest
import torch

from .plain import gemma2_plain as plain
from .tiny import make_folder, random_tokens, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("m")
    return {w: make_folder(tmp, w) for w in ("A", "B")}


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_generation_equals_plain_loop(folders, use_graph):
    from trapetum_amd import load_model
    pcfg, pw = plain.read_folder(folders["A"])
    engine = load_model(folders["A"], dtype="float32", max_tokens_in_cache=1024, max_batch=2, use_graph=use_graph)
    prompts = [random_tokens(n, pcfg["vocab_size"], 70 + n) for n in (5, 11, 17, 3, 9)]   # three batches of <= 2
    want = [plain.greedy_generate(pcfg, pw, p, 8) for p in prompts]
    assert engine.generate(prompts, max_tokens=8, stop_ids=()) == want
    assert engine.cache.live_slots() == []
    # a stop token ends its sequence before it is emitted; the others go on
    stop = want[1][3]
    want_stop = [plain.greedy_generate(pcfg, pw, p, 8, stop_ids=(stop,)) for p in prompts]
    got = engine.generate(prompts, max_tokens=8, stop_ids=(stop,), with_reasons=True)
    assert [g.tokens for g in got] == want_stop
    assert got[1].reason == "stop" and len(got[1].tokens) == 3


@pytest.mark.parametrize("top_p,top_k", [(0.9, 50), (1.0, 0)])
def test_sampled_generation_equals_plain_sampler(folders, top_p, top_k):
    """Temperature 0.7, seed 7 (tiny B): with the same uniform numbers the plain sampler picks the same tokens, from a
    nucleus of the 50 largest and from the whole vocabulary."""
    from trapetum_amd import load_model
    from trapetum_amd.sampling import initial_state
    pcfg, pw = plain.read_folder(folders["B"])
    engine = load_model(folders["B"], dtype="float32", max_tokens_in_cache=2048)
    prompts = [random_tokens(n, pcfg["vocab_size"], 80 + n) for n in (1, 9, 23, 40)]
    got = engine.generate(prompts, max_tokens=12, temperature=0.7, top_p=top_p, top_k=top_k, seed=7, stop_ids=())
    for i, p in enumerate(prompts):
        state, seq, out = initial_state(7, i), list(p), []
        for _ in range(12):
            state = plain.xorshift64(state)
            u = float(torch.tensor(plain.uniform_from_state(state), dtype=torch.float32))
            tok = plain.sample(plain.forward(pcfg, pw, seq)[-1], 0.7, top_p, top_k, u)
            out.append(tok)
            seq.append(tok)
        assert got[i] == out, i
    # each request alone gives what it gave in the batch
    alone = engine.generate([prompts[2]], max_tokens=12, temperature=0.7, top_p=top_p, top_k=top_k, seed=7, stop_ids=())
    assert alone[0] != [] and len(alone[0]) == 12


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
def test_long_decoding(folders, dtype, tol):
    """300 tokens one by one after a short prompt: rings wrap many times, pages fill and chain."""
    from .gpu_engine import load_gpu_model
    model, cfg = load_gpu_model(folders["A"], dtype)
    pcfg, pw = plain.read_folder(folders["A"])
    toks = random_tokens(310, cfg.vocab_size, 9)
    ref = plain.forward(pcfg, pw, toks)
    cache = model.new_cache(max_tokens=512, page_size=16)
    s = cache.acquire()
    rows = [model.step(cache, [s], toks[:10], counts=[10], want=list(range(10)))]
    for t in toks[10:]:
        rows.append(model.step(cache, [s], [t]))
    got = torch.cat(rows)
    worst = max(rel_l2(got[i], ref[i]) for i in range(len(toks)))
    assert worst < 3 * tol, worst
    assert rel_l2(got, ref) < tol


def test_graph_replays_equal_eager_steps(folders):
    """Several replays, with eager work and synchronisation between them, each checked against the eager step."""
    from .gpu_engine import load_gpu_model
    from trapetum_amd.engine.graphs import GraphedDecode
    model, cfg = load_gpu_model(folders["B"], "bfloat16")
    toks = [random_tokens(40, cfg.vocab_size, 30 + i) for i in range(3)]
    eager_cache = model.new_cache(max_tokens=1024, page_size=16)
    graph_cache = model.new_cache(max_tokens=1024, page_size=16)
    graphed = GraphedDecode(model, graph_cache)
    es = [eager_cache.acquire() for _ in toks]
    gs = [graph_cache.acquire() for _ in toks]
    lens = [5, 12, 20]
    flat = [t for s, n in zip(toks, lens) for t in s[:n]]
    model.step(eager_cache, es, flat, counts=lens)
    model.step(graph_cache, gs, flat, counts=lens)
    for step in range(12):
        step_toks = [toks[i][lens[i] + step] for i in range(3)]
        a = model.step(eager_cache, es, step_toks).clone()
        torch.cuda.synchronize()
        b = graphed.step(gs, step_toks).clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b), step
        torch.randn(64, 64, device="cuda:0").sum().item()          # unrelated eager work between replays
    # a smaller batch gets its own graph; the larger one still replays afterwards
    graph_cache.release(gs.pop())
    eager_cache.release(es.pop())
    for step in range(12, 16):
        step_toks = [toks[i][lens[i] + step] for i in range(2)]
        assert torch.equal(model.step(eager_cache, es, step_toks), graphed.step(gs, step_toks)), step


def test_graphs_follow_a_sequence_across_their_length_bound(folders):
    """A graph serves lengths up to a bound (1024, 2048, ...); a sequence that grows past it moves to the next graph.
    Replays before, at and after the crossing agree with eager steps (the slices of the keys differ, so to rounding)."""
    from .gpu_engine import load_gpu_model
    from trapetum_amd.engine.graphs import GraphedDecode
    model, cfg = load_gpu_model(folders["B"], "bfloat16")
    lens = [1015, 300]
    toks = [random_tokens(n + 24, cfg.vocab_size, 90 + i) for i, n in enumerate(lens)]
    eager_cache = model.new_cache(max_tokens=4096)
    graph_cache = model.new_cache(max_tokens=4096)
    graphed = GraphedDecode(model, graph_cache)
    es = [eager_cache.acquire() for _ in toks]
    gs = [graph_cache.acquire() for _ in toks]
    flat = [t for s, n in zip(toks, lens) for t in s[:n]]
    model.step(eager_cache, es, flat, counts=lens)
    model.step(graph_cache, gs, flat, counts=lens)
    for step in range(24):
        step_toks = [toks[i][lens[i] + step] for i in range(2)]
        a = model.step(eager_cache, es, step_toks).clone()
        b = graphed.step(gs, step_toks).clone()
        assert rel_l2(b, a) < 3e-3, step
    assert len(graphed.by_batch) == 2


def test_decode_loop_with_and_without_graph(folders):
    """The device-resident greedy loop: the graph that also picks the tokens gives the ids of eager steps and argmax."""
    from .gpu_engine import load_gpu_model
    from trapetum_amd.engine.decode_loop import DecodeLoop
    model, cfg = load_gpu_model(folders["B"], "bfloat16")
    prompts = [random_tokens(n, cfg.vocab_size, 70 + i) for i, n in enumerate((7, 19, 33))]
    runs = []
    for use_graph in (False, True):
        cache = model.new_cache(max_tokens=1024, page_size=16)
        loop = DecodeLoop(model, cache, use_graph=use_graph)
        ids = [loop.start(prompts).cpu().tolist()]
        for _ in range(20):
            ids.append(loop.step().cpu().tolist())
            torch.randn(32, 32, device="cuda:0").sum().item()       # unrelated eager work between replays
        loop.finish()
        runs.append(ids)
    assert runs[0] == runs[1]
