"""Trace replay's host logic on the CPU (plain kernels), and its schedule helpers."""
import numpy as np
import pytest
import torch

from trapetum_amd.cache import CacheError
from trapetum_amd.engine.batch import StepError
from trapetum_amd.engine.trace import TraceError, TraceRunner

from .cpu_engine import ref_ops_namespace
from .plain import gemma2_plain as plain
from .tiny import make_folder, random_tokens, rel_l2
from . import trace_schedules as ts


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    return make_folder(tmp_path_factory.mktemp("m"), "A")


def run(folder, steps, max_tokens):
    r = TraceRunner(folder, "float32", max_tokens, device="cpu", ops=ref_ops_namespace())
    out = {}
    for s in steps:
        a = r.run_step(s)
        if a is not None:
            out[s["step"]] = a
    assert r.cache.live_slots() == []
    return out


def test_schedules_agree(folder):
    pcfg, pw = plain.read_folder(folder)
    vocab = pcfg["vocab_size"]
    requests = {f"r{i}": random_tokens(n, vocab, 20 + i) for i, n in enumerate([70, 9, 41, 1, 66])}
    ref = {rid: plain.forward(pcfg, pw, t) for rid, t in requests.items()}
    for steps in (ts.whole(requests), ts.last_one_by_one(requests, 32), ts.batches(requests, 2),
                  ts.chunked(requests, [16]), ts.chunked(requests, [1, 7, 32]), ts.chunked(requests, [2, 63, 3]),
                  ts.joining(requests)):
        got = ts.collect(steps, run(folder, steps, ts.held_tokens(steps)), vocab)
        for rid in requests:
            assert rel_l2(torch.from_numpy(got[rid]), ref[rid]) < 2e-5


def test_cache_is_sized_by_max_tokens(folder):
    requests = {"a": list(range(65)), "b": list(range(10))}
    steps = ts.batches(requests, 2, prefill_fraction=1.0)
    assert ts.held_tokens(steps) == 128 + 64
    with pytest.raises(CacheError):
        run(folder, steps, 128)
    run(folder, steps, 192)


def test_steps_of_any_shape_and_what_is_still_refused(folder):
    r = TraceRunner(folder, "float32", 256, device="cpu", ops=ref_ops_namespace())
    r.run_step({"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": []}], "end": []})
    # a request continues by two tokens; another joins the batch that has started
    r.run_step({"step": 1, "entries": [{"id": "a", "tokens": [4, 5], "want": []}], "end": []})
    r.run_step({"step": 2, "entries": [{"id": "a", "tokens": [6], "want": []}, {"id": "b", "tokens": [1, 2], "want": []}], "end": []})
    assert r.cache.length(r.slot_of["a"]) == 6 and r.cache.length(r.slot_of["b"]) == 2
    with pytest.raises(TraceError):      # an entry without tokens
        r.run_step({"step": 3, "entries": [{"id": "a", "tokens": [], "want": []}], "end": []})
    with pytest.raises(TraceError):      # a wanted place outside the entry's tokens
        r.run_step({"step": 3, "entries": [{"id": "a", "tokens": [7], "want": [1]}], "end": []})
    with pytest.raises(StepError):       # a token outside the vocabulary; the newcomer's slot is given back
        r.run_step({"step": 3, "entries": [{"id": "a", "tokens": [7], "want": []}, {"id": "c", "tokens": [100000], "want": []}], "end": []})
    assert "c" not in r.slot_of and r.cache.length(r.slot_of["a"]) == 6
    with pytest.raises(CacheError):      # more tokens than the cache was sized for
        r.run_step({"step": 3, "entries": [{"id": "a", "tokens": list(range(200)), "want": []}], "end": []})
    assert r.cache.length(r.slot_of["a"]) == 6
    with pytest.raises(TraceError):
        r.run_step({"step": 4, "entries": [], "end": ["zz"]})
    assert r.run_step({"step": 5, "entries": [{"id": "a", "tokens": [4], "want": []}], "end": ["a", "b"]}) is None
    assert r.cache.live_slots() == []
