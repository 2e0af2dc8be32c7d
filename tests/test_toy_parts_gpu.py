"""The toy architecture of tests/toy_parts.py on the GPU: a mixer with a state of its own (defined in the test),
another position table, a feed-forward with a router over experts, a layer that runs twice and a run that reads
another run's cache."""
import pytest
import torch

from trapetum_amd.engine.model import Model
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.registry import config_from_folder
from trapetum_amd.weights import WeightFolder, load_folder, write_model_folder

from . import toy_parts
from .tiny import random_tokens, rel_l2
from . import trace_schedules as ts

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
def test_toy_model_steps(tmp_path, dtype, tol):
    toy_parts.register()
    folder = str(tmp_path)
    write_model_folder(toy_parts.ToyConfig.from_kwargs(**toy_parts.TOY), folder, seed=3, sigma=0.15, sigma_norm=0.3)
    arch, cfg = config_from_folder(folder)
    model = Model(arch.build_spec(cfg), Runtime(dtype=dtype, device="cuda:0"))
    load_folder(model, folder)
    src = WeightFolder(folder)
    weights = {n: src.tensor(n).clone() for n in src.names()}
    seqs = [random_tokens(n, toy_parts.TOY["vocab"], 5 + n) for n in (40, 6, 13)]
    ref = [toy_parts.toy_reference(toy_parts.TOY, weights, s) for s in seqs]
    cache = model.new_cache(max_tokens=256, page_size=16)
    for _ in range(2):
        s = cache.acquire()
        got = model.step(cache, [s], seqs[0], counts=[len(seqs[0])], want=list(range(len(seqs[0]))))
        assert rel_l2(got, ref[0]) < tol
        cache.release(s)
    s = cache.acquire()
    rows = [model.step(cache, [s], seqs[0][:8], counts=[8], want=list(range(8)))]
    rows += [model.step(cache, [s], [t]) for t in seqs[0][8:]]
    assert rel_l2(torch.cat(rows), ref[0]) < tol
    cache.release(s)
    slots = [cache.acquire() for _ in seqs]
    lens = [10, 3, 7]
    out = model.step(cache, slots, [t for q, n in zip(seqs, lens) for t in q[:n]], counts=lens)
    got = {i: [out[i]] for i in range(3)}
    step = 0
    while True:
        live = [i for i in range(3) if lens[i] + step < len(seqs[i])]
        if not live:
            break
        out = model.step(cache, [slots[i] for i in live], [seqs[i][lens[i] + step] for i in live])
        for j, i in enumerate(live):
            got[i].append(out[j])
        step += 1
    for i in range(3):
        assert rel_l2(torch.stack(got[i]), ref[i][lens[i] - 1:]) < tol, i

    # steps of any shape: portions, and requests that join a running batch
    requests = {f"r{i}": q for i, q in enumerate(seqs)}
    for steps in (ts.chunked(requests, [4, 1, 9]), ts.joining(requests, every=1, burst=5)):
        cache = model.new_cache(max_tokens=ts.held_tokens(steps, 16), page_size=16)
        out = ts.collect(steps, ts.run_on_model(model, cache, steps), toy_parts.TOY["vocab"])
        for i in range(3):
            assert rel_l2(torch.from_numpy(out[f"r{i}"]), ref[i]) < tol, i
