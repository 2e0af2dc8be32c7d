"""The engine on the GPU against the plain implementation: whole, token by token, unequal batches, reused slots."""
import pytest
import torch

from .plain import gemma2_plain as plain
from .tiny import make_folder, random_tokens, rel_l2
from . import trace_schedules as ts

pytestmark = pytest.mark.gpu
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module", params=[("A", "float32"), ("A", "bfloat16"), ("B", "float32"), ("B", "bfloat16"),
                                        ("C", "float32"), ("C", "bfloat16"), ("D", "float32"), ("D", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def setup(request, tmp_path_factory):
    from .gpu_engine import load_gpu_model
    which, dtype = request.param
    folder = make_folder(tmp_path_factory.mktemp("m"), which)
    model, cfg = load_gpu_model(folder, dtype)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL[dtype]


def test_whole_prompt(setup):
    model, cfg, pcfg, pw, tol = setup
    toks = random_tokens(90, cfg.vocab_size, 3)
    cache = model.new_cache(max_tokens=256, page_size=16)
    s = cache.acquire()
    got = model.step(cache, [s], toks, counts=[len(toks)], want=list(range(len(toks))))
    ref = plain.forward(pcfg, pw, toks)
    assert rel_l2(got, ref) < tol
    cache.release(s)


def test_last_32_one_by_one(setup):
    model, cfg, pcfg, pw, tol = setup
    toks = random_tokens(75, cfg.vocab_size, 4)
    ref = plain.forward(pcfg, pw, toks)
    cache = model.new_cache(max_tokens=256, page_size=16)
    s = cache.acquire()
    n0 = len(toks) - 32
    rows = [model.step(cache, [s], toks[:n0], counts=[n0], want=list(range(n0)))]
    for t in toks[n0:]:
        rows.append(model.step(cache, [s], [t]))
    got = torch.cat(rows)
    assert rel_l2(got, ref) < tol
    for i in range(len(toks)):
        assert rel_l2(got[i], ref[i]) < 3 * tol, i


def test_first_tokens(setup):
    model, cfg, pcfg, pw, tol = setup
    toks = random_tokens(6, cfg.vocab_size, 5)
    ref = plain.forward(pcfg, pw, toks)
    cache = model.new_cache(max_tokens=128)
    s = cache.acquire()
    got = torch.cat([model.step(cache, [s], [t]) for t in toks])
    assert rel_l2(got, ref) < tol


def test_unequal_batches_reused_slots(setup):
    model, cfg, pcfg, pw, tol = setup
    cache = model.new_cache(max_tokens=16 * 12, max_slots=3, page_size=16)
    for batch, lens in enumerate([(5, 11, 17), (1, 9, 40), (23, 2, 3)]):
        seqs = [random_tokens(n + 6, cfg.vocab_size, 100 * batch + i) for i, n in enumerate(lens)]
        extra = [6, 3, 1]
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
            assert rel_l2(torch.stack(got[i]), ref) < tol, (batch, i)
    assert cache.live_slots() == []


def test_steps_repeat_bit_for_bit(setup):
    """The same prefill and the same decode steps, run twice on fresh slots, give the same bits: every reduction has a
    fixed order (no atomics), whatever the timing of the blocks (runtime/src/lib.rs:1433-1457 checks the same)."""
    model, cfg, pcfg, pw, tol = setup
    lens = [41, 7, 23]
    seqs = [random_tokens(n + 6, cfg.vocab_size, 30 + i) for i, n in enumerate(lens)]
    runs = []
    for _ in range(2):
        cache = model.new_cache(max_tokens=512, page_size=16)
        slots = [cache.acquire() for _ in lens]
        flat = [t for s, n in zip(seqs, lens) for t in s[:n]]
        rows = [model.step(cache, slots, flat, counts=lens, want=list(range(sum(lens))))]
        for step in range(6):
            rows.append(model.step(cache, slots, [s[n + step] for s, n in zip(seqs, lens)]))
        runs.append(torch.cat(rows).cpu())
    assert torch.equal(runs[0], runs[1])


@pytest.mark.parametrize("page_size", [16, 64])
def test_portions_and_joining_requests(setup, page_size):
    """A sequence fed in portions of any size, and requests that join a running batch, give the logits of whole
    sequences.  With pages of 16 the windows' rings have no row to spare (B: window 16 in a ring of 16), so a
    portion overwrites ring rows that its own earlier queries still see."""
    model, cfg, pcfg, pw, tol = setup
    requests = {f"r{i}": random_tokens(n, cfg.vocab_size, 40 + i) for i, n in enumerate([70, 9, 41, 2, 35])}
    ref = {rid: plain.forward(pcfg, pw, t) for rid, t in requests.items()}
    for steps in (ts.chunked(requests, [16]), ts.chunked(requests, [1, 7, 32]), ts.chunked(requests, [2, 17, 3]),
                  ts.joining(requests), ts.joining(requests, every=1, burst=9)):
        cache = model.new_cache(max_tokens=ts.held_tokens(steps, page_size), page_size=page_size)
        got = ts.collect(steps, ts.run_on_model(model, cache, steps), cfg.vocab_size)
        assert cache.live_slots() == []
        for rid in requests:
            assert rel_l2(torch.from_numpy(got[rid]), ref[rid]) < tol, rid


class _Tensors:
    """Weights held in memory, for `load_into`."""

    def __init__(self, tensors):
        self.tensors = tensors

    def names(self):
        return list(self.tensors)

    def shape(self, name):
        return tuple(self.tensors[name].shape)

    def dtype(self, name):
        return self.tensors[name].dtype

    def tensor(self, name):
        return self.tensors[name]


def _model_of(folder, dtype, tensors=None):
    from trapetum_amd.engine.model import Model
    from trapetum_amd.engine.runtime import Runtime
    from trapetum_amd.registry import config_from_folder
    from trapetum_amd.weights import WeightFolder, load_folder, load_into
    arch, cfg = config_from_folder(folder)
    model = Model(arch.build_spec(cfg), Runtime(dtype=dtype, device="cuda:0"))
    if tensors is None:
        load_folder(model, folder)
    else:
        load_into(model, _Tensors(tensors))
    return model, cfg


def _whole(model, toks):
    cache = model.new_cache(max_tokens=128, page_size=16)
    s = cache.acquire()
    return model.step(cache, [s], toks, counts=[len(toks)], want=list(range(len(toks)))).double().cpu()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_0_is_local_and_layer_types_overrides(tmp_path, dtype):
    """A model of layer 0 alone (tiny B, window 16): a changed token 0 leaves the logits at positions >= 16 untouched,
    bit for bit, because an even layer is local; `layer_types` naming it full_attention flips that.  Fails when the
    engine takes odd layers for the local ones or ignores `layer_types`."""
    folder = make_folder(tmp_path, "B", name="one_layer", num_hidden_layers=1)
    model, cfg = _model_of(folder, dtype)
    toks = random_tokens(40, cfg.vocab_size, 5)
    other = [(toks[0] + 1) % cfg.vocab_size] + toks[1:]
    a, b = _whole(model, toks), _whole(model, other)
    assert torch.equal(a[16:], b[16:]) and not torch.equal(a[15], b[15])
    pcfg, pw = plain.read_folder(folder)
    assert rel_l2(a, plain.forward(pcfg, pw, toks)) < TOL[dtype]
    folder = make_folder(tmp_path, "B", name="one_full_layer", num_hidden_layers=1, layer_types=["full_attention"])
    model, cfg = _model_of(folder, dtype)
    a, b = _whole(model, toks), _whole(model, other)
    assert not torch.equal(a[39], b[39])
    pcfg, pw = plain.read_folder(folder)
    assert pcfg["layer_types"] == ["full_attention"] and rel_l2(a, plain.forward(pcfg, pw, toks)) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_no_layers_oracle_and_sandwich_identity(tmp_path, dtype):
    """Without layers the logits are norm(E[tok] * sqrt(D)) @ E^T (the lookup is scaled, the head is not), and with
    post-norm weights of -1 (a gain of 0) every layer adds nothing, so the same holds with layers.  Fails when a
    post-norm is applied after the residual sum instead of before it, or the head uses the scaled table.  (That the
    post-norm takes the sub-layer's output, not its input, is what test_post_norms_stand_on_the_sub_layers_outputs pins.)"""
    import math
    folder = make_folder(tmp_path, "B", name="no_layers", num_hidden_layers=0)
    model, cfg = _model_of(folder, dtype)
    pcfg, pw = plain.read_folder(folder)
    toks = random_tokens(7, cfg.vocab_size, 1)
    e = pw["model.embed_tokens.weight"]
    x = e[toks] * math.sqrt(cfg.hidden_size)
    n = x / torch.sqrt((x * x).mean(-1, keepdim=True) + cfg.rms_norm_eps) * (1 + pw["model.norm.weight"])
    oracle = n @ e.T
    assert rel_l2(_whole(model, toks), oracle) < TOL[dtype]
    from trapetum_amd.weights import WeightFolder
    folder = make_folder(tmp_path, "B")
    src = WeightFolder(folder)
    tensors = {name: src.tensor(name).clone() for name in src.names()}
    src.close()
    for name in tensors:
        if "post_attention_layernorm" in name or "post_feedforward_layernorm" in name:
            tensors[name] = -torch.ones_like(tensors[name])
    model, cfg = _model_of(folder, dtype, tensors)
    pcfg, pw = plain.read_folder(folder)                     # the same embedding and final norm: the same oracle
    e = pw["model.embed_tokens.weight"]
    x = e[toks] * math.sqrt(cfg.hidden_size)
    n = x / torch.sqrt((x * x).mean(-1, keepdim=True) + cfg.rms_norm_eps) * (1 + pw["model.norm.weight"])
    assert rel_l2(_whole(model, toks), n @ e.T) < TOL[dtype]
    model, cfg = _model_of(folder, dtype)
    assert rel_l2(_whole(model, toks), n @ e.T) > 10 * TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_post_norms_stand_on_the_sub_layers_outputs(tmp_path, dtype):
    """Output projections eight times as large leave the logits where they were, because the norm that follows a
    sub-layer normalises that sub-layer's output before the residual sum (runtime/src/lib.rs:4530-4533) and an RMS norm
    forgets its input's scale (up to eps).  With the post-norm on the sub-layer's input instead, the factor of eight
    would reach the stream (the plain implementation's test of the same name shows that mistake moving the logits by more
    than a tenth).  A factor of 8 is exact in bfloat16, so both engines see the same change."""
    from trapetum_amd.weights import WeightFolder
    folder = make_folder(tmp_path, "B")
    src = WeightFolder(folder)
    tensors = {name: src.tensor(name).clone() for name in src.names()}
    src.close()
    toks = random_tokens(19, 512, 2)
    model, cfg = _model_of(folder, dtype, tensors)
    ref = _whole(model, toks)
    for name in tensors:
        if name.endswith("self_attn.o_proj.weight") or name.endswith("mlp.down_proj.weight"):
            tensors[name] = tensors[name] * 8.0
    model, cfg = _model_of(folder, dtype, tensors)
    got = _whole(model, toks)
    assert rel_l2(got, ref) < (1e-3 if dtype == "float32" else 2e-2), rel_l2(got, ref)
    pcfg, pw = plain.read_folder(folder)
    assert rel_l2(got, plain.forward(pcfg, pw, toks)) < 2 * TOL[dtype] + 1e-3
