"""Host logic of the step function, on the CPU with plain kernels, against the plain implementation."""
import pytest
import torch

from .cpu_engine import load_cpu_model
from .plain import gemma2_plain as plain
from .tiny import CONFIGS, make_folder, random_tokens, rel_l2
from . import trace_schedules as ts


@pytest.fixture(scope="module", params=["A", "B", "C"])
def setup(request, tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("m"), request.param)
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw


def test_whole_prompt_equals_plain(setup):
    model, cfg, pcfg, pw = setup
    toks = random_tokens(45, cfg.vocab_size, 3)
    cache = model.new_cache(max_tokens=256)
    s = cache.acquire()
    got = model.step(cache, [s], toks, counts=[len(toks)], want=list(range(len(toks))))
    ref = plain.forward(pcfg, pw, toks)
    assert rel_l2(got, ref) < 2e-5
    cache.release(s)


@pytest.mark.parametrize("page_size", [16, 64])
def test_token_by_token_equals_whole(setup, page_size):
    model, cfg, pcfg, pw = setup
    toks = random_tokens(40, cfg.vocab_size, 4)
    ref = plain.forward(pcfg, pw, toks)
    cache = model.new_cache(max_tokens=256, page_size=page_size)     # 16: the window's ring wraps
    s = cache.acquire()
    rows = [model.step(cache, [s], toks[:8], counts=[8], want=list(range(8)))]
    for t in toks[8:]:
        rows.append(model.step(cache, [s], [t]))
    got = torch.cat(rows)
    assert rel_l2(got, ref) < 2e-5


def test_unequal_batches_and_slot_reuse(setup):
    model, cfg, pcfg, pw = setup
    cache = model.new_cache(max_tokens=64 * 3, max_slots=3, page_size=16)
    for batch, lens in enumerate([(5, 11, 17), (1, 9, 40), (23, 2, 3)]):
        seqs = [random_tokens(n + 6, cfg.vocab_size, 100 * batch + i) for i, n in enumerate(lens)]
        extra = [6, 3, 1]                        # decoded tokens per sequence: the shorter ones end earlier
        slots = [cache.acquire() for _ in lens]
        flat = [t for s, n in zip(seqs, lens) for t in s[:n]]
        got = {i: [] for i in range(3)}
        out = model.step(cache, slots, flat, counts=list(lens))
        for i in range(3):
            got[i].append(out[i])
        for step in range(max(extra)):
            live = [i for i in range(3) if step < extra[i]]
            out = model.step(cache, [slots[i] for i in live], [seqs[i][lens[i] + step] for i in live])
            for j, i in enumerate(live):
                got[i].append(out[j])
            for i in range(3):
                if step + 1 == extra[i]:
                    cache.release(slots[i])
        for i in range(3):
            n = lens[i] + extra[i]
            ref = plain.forward(pcfg, pw, seqs[i][:n])[lens[i] - 1:n]
            assert rel_l2(torch.stack(got[i]), ref) < 2e-5, (batch, i)
    assert cache.live_slots() == []


@pytest.mark.parametrize("page_size", [16, 64])
def test_portions_and_joining_requests(setup, page_size):
    """A sequence fed in portions of any size, and requests that join a running batch, give the logits of whole
    sequences.  With pages of 16 the windows' rings have no row to spare (B: window 16 in a ring of 16), so a
    portion overwrites ring rows that its own earlier queries still see."""
    model, cfg, pcfg, pw = setup
    requests = {f"r{i}": random_tokens(n, cfg.vocab_size, 40 + i) for i, n in enumerate([70, 9, 41, 2, 35])}
    ref = {rid: plain.forward(pcfg, pw, t) for rid, t in requests.items()}
    for steps in (ts.chunked(requests, [16]), ts.chunked(requests, [1, 7, 32]), ts.chunked(requests, [2, 17, 3]),
                  ts.joining(requests), ts.joining(requests, every=1, burst=9)):
        cache = model.new_cache(max_tokens=ts.held_tokens(steps, page_size), page_size=page_size)
        got = ts.collect(steps, ts.run_on_model(model, cache, steps), cfg.vocab_size)
        assert cache.live_slots() == []
        for rid in requests:
            assert rel_l2(torch.from_numpy(got[rid]), ref[rid]) < 2e-5, rid


def test_debug_dump_lines(setup, monkeypatch, capsys):
    """TRAPETUM_AMD_DEBUG_DUMP=1: one `[ldump]` line per layer and stage in the reference's format
    (runtime/src/lib.rs:1384-1389), the statistics being those of the step's rows, and the five largest logits."""
    import re

    from trapetum_amd import flags
    model, cfg, pcfg, pw = setup
    toks = random_tokens(9, cfg.vocab_size, 8)
    monkeypatch.setenv("TRAPETUM_AMD_DEBUG_DUMP", "1")
    flags._on.cache_clear()
    try:
        cache = model.new_cache(max_tokens=64)
        s = cache.acquire()
        logits = model.step(cache, [s], toks, counts=[9], want=[8])
    finally:
        monkeypatch.delenv("TRAPETUM_AMD_DEBUG_DUMP")
        flags._on.cache_clear()
    lines = [l for l in capsys.readouterr().err.splitlines() if l.startswith("[ldump]")]
    pattern = re.compile(r"^\[ldump\] L=(-?\d+) stage=(\w+) l2=(\S+) absmax=(\S+) mean=(\S+)$")
    rows = [pattern.match(l).groups() for l in lines[:-1]]
    stages = ["mixer_in", "mixer_out", "after_mixer", "ff_out", "layer_out"]
    assert [(int(r[0]), r[1]) for r in rows] == [(-1, "embed")] + [(l, st) for l in range(cfg.num_hidden_layers) for st in stages] \
        + [(-1, "final_norm"), (-1, "logits")]
    assert abs(float(rows[-1][2]) - float(logits.double().norm())) < 1e-4 * float(logits.double().norm())
    x = plain.embed(torch.tensor(toks), pw["model.embed_tokens.weight"], cfg.hidden_size)
    assert abs(float(rows[0][3]) - float(x.abs().max())) < 1e-5 * float(x.abs().max())
    top = lines[-1]
    assert top.startswith("[ldump] top5= ") and int(top.split()[2].split(":")[0]) == int(logits[0].argmax())
    # switched off, nothing is printed
    model.step(cache, [s], [toks[0]])
    assert "[ldump]" not in capsys.readouterr().err
