"""The generation loop's decisions, on the CPU: batching, stops, early ends, slot reuse, limits."""
import pytest
import torch

from trapetum_amd.cache import CacheError
from trapetum_amd.engine.generate import generate, plan_batch
from trapetum_amd.sampling import SamplingParams, initial_state, xorshift64

from .cpu_engine import load_cpu_model
from .plain import gemma2_plain as plain
from .tiny import make_folder, random_tokens


@pytest.fixture(scope="module")
def setup(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("m"), "A")
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw


def test_plan_batch():
    prompts = [[1] * 10, [1] * 100, [1] * 30, [1] * 5]
    # page 64: needs 64, 128, 64, 64 with 20 new tokens
    assert plan_batch([0, 1, 2, 3], prompts, 20, 64, 10_000, 64, 4096) == 4
    assert plan_batch([0, 1, 2, 3], prompts, 20, 2, 10_000, 64, 4096) == 2
    assert plan_batch([0, 1, 2, 3], prompts, 20, 64, 200, 64, 4096) == 2
    assert plan_batch([1, 2, 3], prompts, 20, 64, 128, 64, 4096) == 1
    with pytest.raises(CacheError):
        plan_batch([1], prompts, 20, 64, 64, 64, 4096)
    with pytest.raises(CacheError):
        plan_batch([1], prompts, 20, 64, 10_000, 64, 50)          # prompt longer than the context
    with pytest.raises(ValueError):
        plan_batch([0], [[]], 20, 64, 10_000, 64, 4096)


def test_batches_one_after_another_match_plain(setup):
    model, cfg, pcfg, pw = setup
    prompts = [random_tokens(n, cfg.vocab_size, 40 + n) for n in (5, 11, 17, 2, 8)]
    want = [plain.greedy_generate(pcfg, pw, p, 6) for p in prompts]
    cache = model.new_cache(max_tokens=64 * 2, page_size=64)            # room for two sequences at a time
    seen = []
    got = generate(model, cache, prompts, max_tokens=6, stop_ids=(), on_tokens=lambda s, e: seen.append((s, e)))
    assert got == want
    assert cache.live_slots() == [] and cache.tokens_held() == 0
    assert all(len(e) <= 2 for _, e in seen)                             # never more than two live
    assert [t for _, e in seen for i, t in e if i == 3] == want[3]


def test_stop_tokens_and_reasons(setup):
    model, cfg, pcfg, pw = setup
    prompts = [random_tokens(n, cfg.vocab_size, 50 + n) for n in (5, 11, 17)]
    free = [plain.greedy_generate(pcfg, pw, p, 8) for p in prompts]
    stop = free[0][2]
    want = [plain.greedy_generate(pcfg, pw, p, 8, stop_ids=(stop,)) for p in prompts]
    cache = model.new_cache(max_tokens=1024)
    got = generate(model, cache, prompts, max_tokens=8, stop_ids=(stop,), with_reasons=True)
    assert [g.tokens for g in got] == want
    assert got[0].reason == "stop" and len(got[0].tokens) == 2
    assert all(g.reason in ("stop", "length") for g in got)
    assert cache.live_slots() == []


def test_context_limit_ends_a_sequence(setup):
    model, cfg, pcfg, pw = setup
    prompts = [random_tokens(28, cfg.vocab_size, 1), random_tokens(3, cfg.vocab_size, 2)]
    cache = model.new_cache(max_tokens=256, max_context=32, page_size=16)
    got = generate(model, cache, prompts, max_tokens=20, stop_ids=(), with_reasons=True)
    assert got[0].reason == "context" and len(got[0].tokens) == 5       # 28 + 4 run, the fifth is emitted only
    assert got[1].reason == "length" and len(got[1].tokens) == 20
    assert got[0].tokens == plain.greedy_generate(pcfg, pw, prompts[0], 5)
    assert cache.live_slots() == []


def test_sampling_is_per_request(setup):
    model, cfg, pcfg, pw = setup
    prompts = [random_tokens(n, cfg.vocab_size, 60 + n) for n in (4, 9, 6)]
    params = SamplingParams(temperature=0.8, top_p=0.9, top_k=40, repetition_penalty=1.2)
    cache = model.new_cache(max_tokens=1024)
    together = generate(model, cache, prompts, max_tokens=6, params=params, seed=3, stop_ids=())
    for i, p in enumerate(prompts):
        state, seq, out, recent = initial_state(3, i), list(p), [], list(p)
        for _ in range(6):
            state = plain.xorshift64(state)
            u = float(torch.tensor(plain.uniform_from_state(state), dtype=torch.float32))
            z = plain.repetition_penalty(plain.forward(pcfg, pw, seq)[-1], recent[-128:], 1.2)
            tok = plain.sample(z, 0.8, 0.9, 40, u)
            out.append(tok)
            seq.append(tok)
            recent.append(tok)
        assert together[i] == out, i


def test_generator_matches_reference_xorshift():
    assert xorshift64(1) == plain.xorshift64(1)
    s = 0x9E3779B97F4A7C15
    for _ in range(5):
        assert xorshift64(s) == plain.xorshift64(s)
        s = xorshift64(s)
    assert initial_state(0, 0) != initial_state(0, 1) != initial_state(1, 0)
    assert initial_state(5, 3) & 1
