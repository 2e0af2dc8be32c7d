"""A toy mixer with a state of its own, one that keeps a single tensor per token in a window's ring, another position table, a feed-forward with a router over experts and a
schedule that runs a layer twice and shares a cache: registered, built and stepped without a change to the framework
(host logic, CPU)."""
import pytest
import torch

from trapetum_amd.engine.model import Model
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.registry import config_from_folder
from trapetum_amd.weights import WeightFolder, load_folder, write_model_folder

from . import toy_parts
from .cpu_engine import ref_ops_namespace
from .tiny import random_tokens, rel_l2
from . import trace_schedules as ts


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    toy_parts.register()
    folder = str(tmp_path_factory.mktemp("toy"))
    write_model_folder(toy_parts.ToyConfig.from_kwargs(**toy_parts.TOY), folder, seed=3, sigma=0.15, sigma_norm=0.3)
    arch, cfg = config_from_folder(folder)
    assert arch.name == "ToyEmaForCausalLM"
    model = Model(arch.build_spec(cfg), Runtime(dtype="float32", device="cpu", ops=ref_ops_namespace()))
    load_folder(model, folder)
    src = WeightFolder(folder)
    weights = {n: src.tensor(n).clone() for n in src.names()}
    return model, weights


def test_cache_groups_of_the_toy(toy):
    model, _ = toy
    cache = model.new_cache(max_tokens=256, page_size=16)
    attn, mem = cache.token_groups
    assert attn.entries == [1] and sorted(attn.pools) == ["k", "v"]                  # entry 4 reads entry 1's cache
    # the mixer that keeps one tensor per token has one pool, a ring of its window: nothing else is allocated for it
    assert mem.entries == [2] and list(mem.pools) == ["h"] and mem.pages.rows_cap == 16
    assert tuple(mem.pools["h"].shape) == (1, 16 + 1, 16, toy_parts.TOY["mem"])
    assert cache.bytes() == sum(p.numel() * p.element_size() for g in cache.token_groups for p in g.pools.values()) + \
        sum(g.tensor.numel() * g.tensor.element_size() for g in cache.state_groups)
    assert len(cache.state_groups) == 1 and cache.state_groups[0].entries == [0, 3]  # layer 0 runs twice: two states
    assert cache.site(4) is None
    with pytest.raises(Exception, match="keeps no per-token tensor 'v'"):
        cache.site(2).tensor("v")


def test_toy_whole_stepwise_and_batched(toy):
    model, weights = toy
    seqs = [random_tokens(n, toy_parts.TOY["vocab"], 5 + n) for n in (21, 6, 13)]
    ref = [toy_parts.toy_reference(toy_parts.TOY, weights, s) for s in seqs]
    cache = model.new_cache(max_tokens=256, page_size=16)
    for rounds in range(2):                                                          # slots (and their states) are used again
        s = cache.acquire()
        got = model.step(cache, [s], seqs[0], counts=[len(seqs[0])], want=list(range(len(seqs[0]))))
        assert rel_l2(got, ref[0]) < 2e-5
        cache.release(s)
    s = cache.acquire()
    rows = [model.step(cache, [s], seqs[0][:4], counts=[4], want=[0, 1, 2, 3])]
    rows += [model.step(cache, [s], [t]) for t in seqs[0][4:]]
    assert rel_l2(torch.cat(rows), ref[0]) < 2e-5
    cache.release(s)
    slots = [cache.acquire() for _ in seqs]
    lens = [10, 3, 7]
    out = model.step(cache, slots, [t for q, n in zip(seqs, lens) for t in q[:n]], counts=lens)
    got = {i: [out[i]] for i in range(3)}
    live = [0, 1, 2]
    step = 0
    while live:
        live = [i for i in live if lens[i] + step < len(seqs[i])]
        if not live:
            break
        out = model.step(cache, [slots[i] for i in live], [seqs[i][lens[i] + step] for i in live])
        for j, i in enumerate(live):
            got[i].append(out[j])
        step += 1
    for i in range(3):
        assert rel_l2(torch.stack(got[i]), ref[i][lens[i] - 1:]) < 2e-5, i


def test_toy_portions_and_joining(toy):
    """Steps of any shape reach the toy's parts too: the state mixer scans a portion from the state it kept, and the
    run that reads another run's cache sees the cached positions gathered for that run."""
    model, weights = toy
    vocab = toy_parts.TOY["vocab"]
    requests = {f"r{i}": random_tokens(n, vocab, 60 + i) for i, n in enumerate([33, 5, 18])}
    ref = {rid: toy_parts.toy_reference(toy_parts.TOY, weights, t) for rid, t in requests.items()}
    for steps in (ts.chunked(requests, [4, 1, 9]), ts.joining(requests, every=1, burst=5)):
        cache = model.new_cache(max_tokens=ts.held_tokens(steps, 16), page_size=16)
        got = ts.collect(steps, ts.run_on_model(model, cache, steps), vocab)
        for rid in requests:
            assert rel_l2(torch.from_numpy(got[rid]), ref[rid]) < 2e-5, rid
