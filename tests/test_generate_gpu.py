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
    # each request alone, under the id it had in the batch, gives what it gave in the batch
    for i in (2, 0):
        alone = engine.generate([prompts[i]], max_tokens=12, temperature=0.7, top_p=top_p, top_k=top_k, seed=7,
                                stop_ids=(), request_ids=[i])
        assert alone[0] == got[i], i
    # and under another id other tokens
    assert engine.generate([prompts[2]], max_tokens=12, temperature=0.7, top_p=top_p, top_k=top_k, seed=7,
                           stop_ids=(), request_ids=[5])[0] != got[2]


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
    # a smaller batch gets a graph of fewer rows
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
    assert len(graphed.graphs) == 2 and graphed.captures == 2


def test_a_shrinking_batch_with_and_without_graphs(folders):
    """Eight requests that reach the context's end one after the other: the graphs' rows that stand for no sequence any
    more, and the moves into graphs of fewer rows, change no token (greedy, and sampled inside the graph)."""
    from trapetum_amd import load_model
    pcfg, pw = plain.read_folder(folders["B"])
    context, most = 48, 40
    prompts = [random_tokens(n, pcfg["vocab_size"], 70 + i) for i, n in enumerate((12, 45, 27, 9, 42, 20, 38, 33))]
    limits = [min(most, context + 1 - len(p)) for p in prompts]          # 37, 4, 22, 40, 7, 29, 11, 16 tokens
    want = [plain.greedy_generate(pcfg, pw, p, n) for p, n in zip(prompts, limits)]
    runs = {}
    for use_graph in (False, True):
        engine = load_model(folders["B"], dtype="float32", max_tokens_in_cache=2048, max_context=context, max_batch=8,
                            use_graph=use_graph)
        got = engine.generate(prompts, max_tokens=most, stop_ids=(), with_reasons=True)
        runs[use_graph] = [g.tokens for g in got]
        assert [g.reason for g in got] == ["context" if n < most else "length" for n in limits]
        assert engine.cache.live_slots() == []
        if use_graph:
            assert {k[0] for k in engine.graphed.graphs} == {8, 4, 2, 1}    # the batch moved through smaller graphs
        sampled = engine.generate(prompts, max_tokens=most, temperature=0.9, top_p=0.9, top_k=30, seed=3, stop_ids=())
        runs[use_graph, "sampled"] = sampled
    assert runs[True] == want and runs[False] == want
    assert runs[True, "sampled"] == runs[False, "sampled"] and [len(t) for t in runs[True, "sampled"]] == limits


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_repetition_penalty_inside_the_graphs(folders, temperature):
    """The penalty over the last 128 tokens, prompt included, when the recent tokens live in rings on the device that
    the graphs extend themselves: the plain loop's tokens, with prompts shorter and longer than the window (a ring
    that fills up, and one that is full from the start and overwrites its oldest place), through a batch that
    shrinks into smaller graphs, and the same tokens as the loop that makes the choice on the host's side."""
    from trapetum_amd import load_model
    from trapetum_amd.sampling import initial_state
    pcfg, pw = plain.read_folder(folders["B"])
    lens, new = (120, 5, 140, 131, 64), 30
    prompts = [random_tokens(n, pcfg["vocab_size"], 90 + i) for i, n in enumerate(lens)]
    want = []
    for i, p in enumerate(prompts):
        state, seq, out = initial_state(11, i), list(p), []
        for _ in range(new):
            z = plain.repetition_penalty(plain.forward(pcfg, pw, seq)[-1], seq[-128:], 1.3)
            if temperature > 0:
                state = plain.xorshift64(state)
                u = float(torch.tensor(plain.uniform_from_state(state), dtype=torch.float32))
                tok = plain.sample(z, temperature, 0.9, 40, u)
            else:
                tok = int(z.argmax())
            out.append(tok)
            seq.append(tok)
        want.append(out)
    # tokens that end three of the requests at different steps, so that the batch shrinks
    stops = {want[1][4], want[3][9], want[0][15]}
    want_cut = [w[:min([w.index(t) for t in stops if t in w] + [new])] for w in want]
    for use_graph in (True, False):
        engine = load_model(folders["B"], dtype="float32", max_tokens_in_cache=4096, max_batch=8, use_graph=use_graph)
        kw = dict(max_tokens=new, temperature=temperature, top_p=0.9, top_k=40, repetition_penalty=1.3, seed=11)
        assert engine.generate(prompts, stop_ids=(), **kw) == want, use_graph
        assert engine.generate(prompts, stop_ids=tuple(stops), **kw) == want_cut, use_graph
        assert engine.cache.live_slots() == []
    assert len(set(len(w) for w in want_cut)) > 2                 # the requests did end at different steps


def test_graphs_are_dropped_beyond_their_number(folders):
    from .gpu_engine import load_gpu_model
    from trapetum_amd.engine.graphs import GraphedDecode
    model, cfg = load_gpu_model(folders["A"], "bfloat16")
    cache = model.new_cache(max_tokens=2048, max_slots=16)
    graphed = GraphedDecode(model, cache, max_graphs=2)
    slots = [cache.acquire() for _ in range(5)]
    model.step(cache, slots, [1] * 5)
    first = graphed.step(slots[:1], [3]).clone()
    for n in (2, 3, 5, 1):                                       # rows 2, 4, 8, 1: the graph of one row was dropped and comes again
        graphed.step(slots[:n], [3] * n)
    assert len(graphed.graphs) == 2 and graphed.captures == 5
    assert set(k[0] for k in graphed.graphs) == {8, 1}
