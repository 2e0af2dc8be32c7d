"""Each part alone on the GPU, built through the registry with sizes of its own, against the plain functions."""
import math

import pytest
import torch

from trapetum_amd.cache import ModelCache
from trapetum_amd.engine.batch import StepContext
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.registry import build_part, part_class

from .plain import gemma2_plain as plain
from .tiny import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 2e-6, "bfloat16": 1e-2}


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def rt(request):
    return Runtime(dtype=request.param, device=DEV)


def bound(part, rt, tensors):
    """Bind a part to bf16-stored tensors; returns them widened for the plain functions."""
    stored = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    part.bind({k: v.to(DEV) for k, v in stored.items()}, rt)
    return {k: v.double() for k, v in stored.items()}


class OnePartContext:
    """A step context for one part: a cache with one entry and the geometry of the given sequences."""

    def __init__(self, rt, spec, max_tokens=512, page=16):
        self.rt = rt
        self.cache = ModelCache([spec], max_tokens, max_tokens, 8, page, rt.dtype, rt.device)

    def step(self, slots, counts):
        starts = [self.cache.length(s) for s in slots]
        for s, c in zip(slots, counts):
            self.cache.grow(s, c)
        ctx = StepContext(self.rt, self.cache, slots, counts, starts, list(range(sum(counts))))
        ctx.entry = ctx.cache_owner = 0
        return ctx


def act(rt, t):
    return t.to(rt.dtype).to(DEV)


def test_norm(rt):
    norm = build_part("norm", ("rms_norm", {"size": 88, "eps": 1e-4, "weight_offset": 1.0}))
    w = bound(norm, rt, {"weight": rnd(88, seed=1, scale=0.3)})
    x = rnd(7, 88, seed=2, scale=2.0)
    got = norm.forward(type("C", (), {"ops": rt.ops, "dtype": rt.dtype})(), x.to(DEV))
    assert rel_l2(got, plain.rms_norm(x.double(), w["weight"], 1e-4)) < TOL[str(rt.dtype).split(".")[1]]
    plain_norm = build_part("norm", ("rms_norm", {"size": 88, "eps": 1e-4}))        # without the offset: gain = w
    w = bound(plain_norm, rt, {"weight": rnd(88, seed=1, scale=0.3)})
    assert torch.equal(plain_norm.gain.cpu(), w["weight"].float())


def test_position_tables():
    rope = build_part("position", ("rope", {"rotary_dim": 48, "theta": 37.0}))
    assert torch.allclose(rope.inv_freq(torch.device(DEV)).cpu().double(), plain.rope_inv_freq(48, 37.0, torch.float64), rtol=1e-6)
    assert build_part("position", ("none", {})).rotary_dim == 0
    with pytest.raises(ValueError):
        build_part("position", ("rope", {"rotary_dim": 7, "theta": 10.0}))


def test_gated_mlp(rt):
    ff = build_part("feed_forward", ("gated_mlp", {"hidden_size": 88, "intermediate_size": 200, "activation": "gelu_tanh"}))
    w = bound(ff, rt, {"gate_proj.weight": rnd(200, 88, seed=3, scale=0.2), "up_proj.weight": rnd(200, 88, seed=4, scale=0.2),
                       "down_proj.weight": rnd(88, 200, seed=5, scale=0.2)})
    x = rnd(9, 88, seed=6).to(torch.bfloat16)
    got = rt.ops.rows(ff.forward(type("C", (), {"ops": rt.ops, "dtype": rt.dtype})(), act(rt, x)), rt.dtype)
    ref = plain.geglu(x.double(), w["gate_proj.weight"], w["up_proj.weight"], w["down_proj.weight"], lambda t: t)
    assert rel_l2(got, ref) < TOL[str(rt.dtype).split(".")[1]]


def test_embedding_and_head(rt):
    emb = build_part("embedding", ("scaled_embedding", {"vocab_size": 331, "hidden_size": 88, "scale": math.sqrt(88)}))
    head = build_part("head", ("linear_head", {"vocab_size": 331, "hidden_size": 88, "softcap": 11.0}))
    table = rnd(331, 88, seed=7, scale=0.1)
    w = bound(emb, rt, {"weight": table})
    bound(head, rt, {"weight": table})
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    tok = torch.tensor([5, 330, 0, 17], dtype=torch.int32, device=DEV)
    x = emb.forward(ctx, tok)
    assert x.dtype == torch.float32 and rel_l2(x, plain.embed(tok.cpu().long(), w["weight"], 88)) < 1e-6
    rows = rnd(4, 88, seed=8).to(torch.bfloat16)
    z = head.forward(ctx, act(rt, rows))
    assert z.dtype == torch.float32
    assert rel_l2(z, plain.softcap(rows.double() @ w["weight"].T, 11.0)) < TOL[str(rt.dtype).split(".")[1]]


ATT = dict(hidden_size=88, num_heads=6, num_kv_heads=2, head_dim=32, query_scale=0.21, softcap=9.0, window=7,
           position=("rope", {"rotary_dim": 32, "theta": 300.0}))


def attention_reference(w, x, window):
    cfg = {"num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 32, "rope_theta": 300.0,
           "query_pre_attn_scalar": 1 / 0.21 ** 2, "attn_logit_softcapping": 9.0}
    W = {"L.self_attn." + k: v for k, v in w.items()}
    return plain.attention_block(x.double(), torch.arange(x.shape[0]), W, "L.", cfg, window, lambda t: t)


def test_attention_mixer_prefill_and_decode(rt):
    tol = 3e-6 if rt.dtype == torch.float32 else 1.5e-2
    mixer = build_part("mixer", ("attention", ATT))
    w = bound(mixer, rt, {"q_proj.weight": rnd(192, 88, seed=9, scale=0.3), "k_proj.weight": rnd(64, 88, seed=10, scale=0.3),
                          "v_proj.weight": rnd(64, 88, seed=11, scale=0.3), "o_proj.weight": rnd(88, 192, seed=12, scale=0.3)})
    seqs = [rnd(n, 88, seed=20 + n).to(torch.bfloat16) for n in (30, 9)]
    refs = [attention_reference(w, x, 7) for x in seqs]
    one = OnePartContext(rt, mixer.cache_spec())
    slots = [one.cache.acquire(), one.cache.acquire()]
    lens = [22, 5]
    ctx = one.step(slots, lens)
    got = rt.ops.rows(mixer.forward(ctx, act(rt, torch.cat([x[:n] for x, n in zip(seqs, lens)])), one.cache.site(0)), rt.dtype)
    assert rel_l2(got[:22], refs[0][:22]) < tol and rel_l2(got[22:], refs[1][:5]) < tol
    for step in range(8):                                   # the second sequence ends after 4 more tokens
        live = [i for i in range(2) if lens[i] + step < seqs[i].shape[0]]
        ctx = one.step([slots[i] for i in live], [1] * len(live))
        got = rt.ops.rows(mixer.forward(ctx, act(rt, torch.stack([seqs[i][lens[i] + step] for i in live])), one.cache.site(0)), rt.dtype)
        for j, i in enumerate(live):
            assert rel_l2(got[j], refs[i][lens[i] + step]) < 2 * tol, (step, i)


def test_window_edge_shows(rt):
    """The key that has just left the window is made to dominate: if the kernel still sees it, the output is its value."""
    tol = 3e-6 if rt.dtype == torch.float32 else 1.5e-2
    mixer = build_part("mixer", ("attention", dict(ATT, softcap=None, position=("none", {}), window=7, query_scale=1.0)))
    eye = torch.eye(192, 88)
    w = bound(mixer, rt, {"q_proj.weight": eye, "k_proj.weight": eye[:64], "v_proj.weight": rnd(64, 88, seed=13),
                          "o_proj.weight": torch.eye(88, 192)})
    x = rnd(20, 88, seed=14, scale=0.1).to(torch.bfloat16)
    x[12 - 7, :32] = 6.0                                     # key of position 5: outside the window of query 12 by one
    x[12, :32] = 6.0                                         # query 12 scores it 1152, everything else about 0
    cfg = {"num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 32, "rope_theta": 1.0, "query_pre_attn_scalar": 1.0}
    one = OnePartContext(rt, mixer.cache_spec())
    s = one.cache.acquire()
    got = rt.ops.rows(mixer.forward(one.step([s], [20]), act(rt, x), one.cache.site(0)), rt.dtype)
    q = (x.double() @ w["q_proj.weight"].T).reshape(20, 6, 32)
    k = (x.double() @ w["k_proj.weight"].T).reshape(20, 2, 32)
    v = (x.double() @ w["v_proj.weight"].T).reshape(20, 2, 32)
    ref = plain.attention(q, k, v, 1.0, None, 7).reshape(20, 192) @ w["o_proj.weight"].T
    leaked = plain.attention(q, k, v, 1.0, None, 8).reshape(20, 192) @ w["o_proj.weight"].T
    assert rel_l2(leaked[12], ref[12]) > 0.1                 # the test can tell the two apart
    assert rel_l2(got, ref) < tol
    # the same edge, decoded token by token through the ring
    one2 = OnePartContext(rt, mixer.cache_spec())
    s = one2.cache.acquire()
    rows = [rt.ops.rows(mixer.forward(one2.step([s], [1]), act(rt, x[i:i + 1]), one2.cache.site(0)), rt.dtype) for i in range(20)]
    assert rel_l2(torch.cat(rows), ref) < tol


def test_cap_comes_after_the_scale(rt):
    """Dots of +1e6 and -1e6 with a scale of 1/4 and a cap of 3: the probabilities are softmax([+3, -3]) if the cap is
    applied to the scaled score (runtime/cuda/codebook_gemv.cu:254-255) and softmax([+3/4, -3/4]) if the scale came
    after the cap; random weights cannot tell the two apart, because tanh is linear for their small scores.  Whole
    prompt and token by token; fails when a kernel multiplies by the scale after the cap."""
    tol = 3e-6 if rt.dtype == torch.float32 else 1.5e-2
    mixer = build_part("mixer", ("attention", dict(ATT, softcap=3.0, query_scale=0.25, window=None, position=("none", {}))))
    w = bound(mixer, rt, {"q_proj.weight": torch.eye(192, 88), "k_proj.weight": -torch.eye(64, 88),
                          "v_proj.weight": rnd(64, 88, seed=15), "o_proj.weight": torch.eye(88, 192)})
    x = torch.zeros(2, 88)
    x[0, 0], x[1, 0] = -1e3, 1e3                           # keys +1e3 and -1e3 on element 0, the query at position 1 +1e3
    x[:, 40:] = rnd(2, 48, seed=16)                         # what the values are made of
    x = x.to(torch.bfloat16)
    v = (x.double() @ w["v_proj.weight"].T)[:, :32]         # kv head 0, which query head 0 reads
    p = torch.softmax(torch.tensor([3.0, -3.0], dtype=torch.float64), 0)
    want = p[0] * v[0] + p[1] * v[1]
    wrong = torch.softmax(torch.tensor([0.75, -0.75], dtype=torch.float64), 0)
    assert rel_l2(wrong[0] * v[0] + wrong[1] * v[1], want) > 0.1
    one = OnePartContext(rt, mixer.cache_spec())
    s = one.cache.acquire()
    got = rt.ops.rows(mixer.forward(one.step([s], [2]), act(rt, x), one.cache.site(0)), rt.dtype)
    assert rel_l2(got[1, :32], want) < tol
    one = OnePartContext(rt, mixer.cache_spec())
    s = one.cache.acquire()
    rows = [rt.ops.rows(mixer.forward(one.step([s], [1]), act(rt, x[i:i + 1]), one.cache.site(0)), rt.dtype) for i in range(2)]
    assert rel_l2(rows[1][0, :32], want) < tol


@pytest.mark.parametrize("m", [1, 8, 200])
def test_the_gate_is_what_the_activation_is_applied_to(rt, m):
    """gate = -20 and up = +5 give gelu_tanh(-20) * 5 = 0; with the two swapped the result is gelu_tanh(5) * -20 = -100
    (runtime/cuda/codebook_gemv.cu:531-537, runtime/src/lib.rs:4511-4513).  One, a few and many rows run on different
    product kernels; fails when a gated epilogue activates the up half."""
    ff = build_part("feed_forward", ("gated_mlp", {"hidden_size": 16, "intermediate_size": 16, "activation": "gelu_tanh"}))
    gate, up = torch.zeros(16, 16), torch.zeros(16, 16)
    gate[:, 0], up[:, 0] = -20.0, 5.0
    bound(ff, rt, {"gate_proj.weight": gate, "up_proj.weight": up, "down_proj.weight": torch.eye(16)})
    x = torch.zeros(m, 16)
    x[:, 0] = 1.0
    got = rt.ops.rows(ff.forward(type("C", (), {"ops": rt.ops, "dtype": rt.dtype})(), act(rt, x)), rt.dtype)
    assert float(got.float().abs().max()) < 1e-3
    bound(ff, rt, {"gate_proj.weight": up, "up_proj.weight": gate, "down_proj.weight": torch.eye(16)})
    got = rt.ops.rows(ff.forward(type("C", (), {"ops": rt.ops, "dtype": rt.dtype})(), act(rt, x)), rt.dtype)
    assert float((got.float() + 100.0).abs().max()) < 0.5


def test_sandwich_block(rt):
    tol = 5e-6 if rt.dtype == torch.float32 else 1.5e-2
    make_norm = lambda site=None: build_part("norm", ("rms_norm", {"size": 88, "eps": 1e-5, "weight_offset": 1.0}))
    block = part_class("block", "sandwich")(build_part("mixer", ("attention", dict(ATT, window=None))),
                                            build_part("feed_forward", ("gated_mlp", {"hidden_size": 88, "intermediate_size": 200, "activation": "gelu_tanh"})),
                                            make_norm)
    W = {}
    W.update({"self_attn." + k: v for k, v in bound(block.mixer, rt, {
        "q_proj.weight": rnd(192, 88, seed=30, scale=0.2), "k_proj.weight": rnd(64, 88, seed=31, scale=0.2),
        "v_proj.weight": rnd(64, 88, seed=32, scale=0.2), "o_proj.weight": rnd(88, 192, seed=33, scale=0.2)}).items()})
    W.update({"mlp." + k: v for k, v in bound(block.feed_forward, rt, {
        "gate_proj.weight": rnd(200, 88, seed=34, scale=0.2), "up_proj.weight": rnd(200, 88, seed=35, scale=0.2),
        "down_proj.weight": rnd(88, 200, seed=36, scale=0.2)}).items()})
    names = {"pre_mixer_norm": "input_layernorm", "post_mixer_norm": "post_attention_layernorm",
             "pre_ff_norm": "pre_feedforward_layernorm", "post_ff_norm": "post_feedforward_layernorm"}
    for i, (site, name) in enumerate(names.items()):
        W[name + ".weight"] = bound(block.norms[site], rt, {"weight": rnd(88, seed=40 + i, scale=0.3)})["weight"]
    cfg = {"num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 32, "rope_theta": 300.0, "rms_norm_eps": 1e-5,
           "query_pre_attn_scalar": 1 / 0.21 ** 2, "attn_logit_softcapping": 9.0, "sliding_window": 10 ** 6}
    x = rnd(13, 88, seed=50)
    ref = plain.block(x.double(), torch.arange(13), {"model.layers.1." + k: v for k, v in W.items()}, 1, cfg, lambda t: t)
    one = OnePartContext(rt, block.mixer.cache_spec())
    s = one.cache.acquire()
    stream = x.to(DEV).clone()
    out, nxt = block.forward(one.step([s], [13]), stream, one.cache.site(0))
    assert nxt is None and out.dtype == torch.float32 and rel_l2(out, ref) < tol
    # the next block's first norm, fused into this block's last add
    follow = make_norm()
    wf = bound(follow, rt, {"weight": rnd(88, seed=60, scale=0.3)})["weight"]
    one = OnePartContext(rt, block.mixer.cache_spec())
    s = one.cache.acquire()
    out, nxt = block.forward(one.step([s], [13]), x.to(DEV).clone(), one.cache.site(0), next_norm=follow)
    assert rel_l2(nxt, plain.rms_norm(ref, wf, 1e-5)) < max(tol, 3e-6)
