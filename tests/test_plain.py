"""What pins the plain implementation beside the reference's text: special cases that reduce to a library
routine, invariants, and the vectors the reference's own checks hold.  Each is chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place, a scale applied twice) fails it."""
import math

import pytest
import torch

from .plain import gemma2_plain as plain
from .tiny import TINY_A, TINY_B, make_folder, random_tokens, rel_l2

D = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D)


# ---- RMSNorm ------------------------------------------------------------------------------------------
def test_rms_norm_cases():
    x = rnd(5, 12)
    zero = torch.zeros(12, dtype=D)
    y = plain.rms_norm(x, zero, 1e-6)
    assert torch.allclose(y, x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6))      # w = 0 still scales: (1 + w)
    assert torch.allclose((plain.rms_norm(x, zero, 0.0) ** 2).mean(-1), torch.ones(5, dtype=D))
    assert torch.allclose(plain.rms_norm(3.0 * x, zero, 0.0), plain.rms_norm(x, zero, 0.0))
    w = rnd(12, seed=1)
    assert torch.allclose(plain.rms_norm(x, w, 1e-6), y * (1 + w))
    big = plain.rms_norm(x * 1e-4, zero, 1.0)                                             # eps is added to the mean of squares
    assert torch.allclose(big, x * 1e-4 / torch.sqrt((x * x).mean(-1, keepdim=True) * 1e-8 + 1.0))


# ---- RoPE ---------------------------------------------------------------------------------------------------
def test_rope_cases():
    x = rnd(4, 3, 8)
    assert torch.equal(plain.rope(x, torch.zeros(4, dtype=torch.long), 10000.0), x)       # position 0: identity
    v = rnd(1, 1, 2, seed=2)
    r = plain.rope(v, torch.tensor([3]), 77.0)[0, 0]                                     # head size 2: a rotation by p radians
    c, s = math.cos(3.0), math.sin(3.0)
    assert torch.allclose(r, torch.tensor([v[0, 0, 0] * c - v[0, 0, 1] * s, v[0, 0, 1] * c + v[0, 0, 0] * s], dtype=D))
    y = plain.rope(x, torch.tensor([5, 9, 2, 40]), 500.0)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1))
    # pairs are (d, d + half), frequencies theta^(-2d/hd): element 1 pairs with element 5 at angle p * theta^(-2/8)
    one = torch.zeros(1, 1, 8, dtype=D)
    one[0, 0, 1] = 1.0
    z = plain.rope(one, torch.tensor([7]), 500.0)[0, 0]
    ang = 7 * 500.0 ** (-2 / 8)
    want = torch.zeros(8, dtype=D)
    want[1], want[5] = math.cos(ang), math.sin(ang)
    assert torch.allclose(z, want)
    assert torch.allclose(plain.rope_inv_freq(8, 500.0, D), torch.tensor([500.0 ** (-2 * d / 8) for d in range(4)], dtype=D))


def test_rope_scores_depend_on_distance_only():
    q, k = rnd(1, 1, 16, seed=3), rnd(1, 1, 16, seed=4)
    def score(p, t):
        return float((plain.rope(q, torch.tensor([p]), 100.0) * plain.rope(k, torch.tensor([t]), 100.0)).sum())
    assert abs(score(9, 4) - score(109, 104)) < 1e-9
    assert abs(score(9, 4) - score(4, 9)) > 1e-3                                           # the sign of the angle matters


# ---- attention ------------------------------------------------------------------------------------------------
def sdpa(q, k, v, scale):
    T = q.shape[0]
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    s = torch.einsum("thd,shd->hts", q, k) * scale
    s = s.masked_fill(~mask, float("-inf"))
    return torch.einsum("hts,shd->thd", torch.softmax(s, -1), v)


def test_attention_reduces_to_plain_softmax_attention():
    q, k, v = rnd(9, 4, 8, seed=5), rnd(9, 4, 8, seed=6), rnd(9, 4, 8, seed=7)
    got = plain.attention(q, k, v, 1 / math.sqrt(8), None, None)
    assert torch.allclose(got, sdpa(q, k, v, 1 / math.sqrt(8)))
    lib = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    assert torch.allclose(got, lib.transpose(0, 1))


def test_attention_grouping_scale_cap_window():
    q, k, v = rnd(11, 6, 8, seed=8), rnd(11, 2, 8, seed=9), rnd(11, 2, 8, seed=10)
    got = plain.attention(q, k, v, 0.3, None, None)
    rep = lambda t: t.repeat_interleave(3, dim=1)                                           # heads 0-2 read kv head 0
    assert torch.allclose(got, sdpa(q, rep(k), rep(v), 0.3))
    assert torch.allclose(plain.attention(q, k, v, 0.3 / 2, None, None), plain.attention(q / 2, k, v, 0.3, None, None))
    assert torch.allclose(plain.attention(q, k, v, 0.3, 1e30, None), got)                   # a huge cap is no cap
    capped = plain.attention(q * 50, k, v, 0.3, 2.0, None)
    assert not torch.allclose(capped, plain.attention(q * 50, k, v, 0.3, None, None), atol=1e-3)
    assert torch.allclose(plain.attention(q, k, v, 0.3, None, 11), got)                     # window >= length: global
    assert torch.allclose(plain.attention(q, k, v, 0.3, None, 1), rep(v))                   # window 1: the token's own v
    w4 = plain.attention(q, k, v, 0.3, 5.0, 4)
    k2, v2 = k.clone(), v.clone()
    k2[3] += 9.0
    v2[3] -= 9.0
    w4b = plain.attention(q, k2, v2, 0.3, 5.0, 4)
    assert torch.equal(w4[7:], w4b[7:]) and not torch.allclose(w4[6], w4b[6])              # position 3 leaves the window at 7
    assert torch.allclose(plain.softcap(torch.tensor([1e-3], dtype=D), 50.0), torch.tensor([1e-3], dtype=D), rtol=1e-6)
    assert float(plain.softcap(torch.tensor([1e9], dtype=D), 50.0)) == 50.0
    assert float(plain.softcap(torch.tensor([-3.0], dtype=D), 7.0)) == -float(plain.softcap(torch.tensor([3.0], dtype=D), 7.0))


def saturating_case():
    """Two keys whose dots with the query at position 1 are +1e6 and -1e6: the capped scores are +cap and -cap
    whatever the scale, if the cap comes after the scale."""
    q, k = torch.zeros(2, 1, 4, dtype=D), torch.zeros(2, 1, 4, dtype=D)
    q[1, 0, 0], k[0, 0, 0], k[1, 0, 0] = 1e3, 1e3, -1e3
    v = rnd(2, 1, 4, seed=30)
    return q, k, v


def test_cap_comes_after_the_scale():
    """score = dot * scale, then cap * tanh(score / cap) (runtime/cuda/codebook_gemv.cu:254-255).  With saturating dots and
    a scale of 1/4 the probabilities are softmax([+cap, -cap]); capping first and scaling after gives
    softmax([+cap/4, -cap/4]).  Fails when `softcap` in plain.attention moves before the multiplication by the scale."""
    q, k, v = saturating_case()
    got = plain.attention(q, k, v, 0.25, 3.0, None)[1, 0]
    p = torch.softmax(torch.tensor([3.0, -3.0], dtype=D), 0)
    assert torch.allclose(got, p[0] * v[0, 0] + p[1] * v[1, 0], atol=1e-12)
    wrong = torch.softmax(torch.tensor([0.75, -0.75], dtype=D), 0)
    assert not torch.allclose(got, wrong[0] * v[0, 0] + wrong[1] * v[1, 0], atol=1e-3)


def test_the_gate_is_what_the_activation_is_applied_to():
    """act = gelu_tanh(gate) * up (runtime/cuda/codebook_gemv.cu:531-537 with g = gate, u = up: runtime/src/lib.rs:4511-4513).
    A gate of -20 with an up of +5 gives 0; the swap, gelu_tanh(5) * -20, gives -100.  Fails when the activation moves
    to the up projection in plain.geglu."""
    one = torch.ones(1, 1, dtype=D)
    got = plain.geglu(one, -20.0 * one, 5.0 * one, one, lambda t: t)
    assert abs(float(got)) < 1e-9
    assert abs(float(plain.geglu(one, 5.0 * one, -20.0 * one, one, lambda t: t)) + 100.0) < 1e-3


# ---- feed-forward, embedding, head, sandwich ---------------------------------------------------------------------
def test_gelu_and_geglu():
    g = torch.linspace(-6, 6, 101, dtype=D)
    assert torch.allclose(plain.gelu_tanh(g), torch.nn.functional.gelu(g, approximate="tanh"), atol=1e-9)
    assert float(plain.gelu_tanh(torch.tensor(0.0, dtype=D))) == 0.0
    x, wg, wu, wd = rnd(3, 8, seed=11), rnd(16, 8, seed=12), rnd(16, 8, seed=13), rnd(8, 16, seed=14)
    want = (torch.nn.functional.gelu(x @ wg.T, approximate="tanh") * (x @ wu.T)) @ wd.T
    assert torch.allclose(plain.geglu(x, wg, wu, wd, lambda t: t), want)
    swapped = (torch.nn.functional.gelu(x @ wu.T, approximate="tanh") * (x @ wg.T)) @ wd.T
    assert not torch.allclose(want, swapped)


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory):
    return make_folder(tmp_path_factory.mktemp("m"), "B")


def test_no_layers_oracle_and_sandwich_identity(folder_b):
    cfg, w = plain.read_folder(folder_b)
    toks = random_tokens(7, cfg["vocab_size"], 1)
    e = w["model.embed_tokens.weight"]
    x = e[toks] * math.sqrt(cfg["hidden_size"])                                             # the lookup is scaled, the head is not
    n = x / torch.sqrt((x * x).mean(-1, keepdim=True) + cfg["rms_norm_eps"]) * (1 + w["model.norm.weight"])
    oracle = n @ e.T
    assert torch.allclose(plain.forward(dict(cfg, num_hidden_layers=0), w, toks), oracle)
    # post-norm weights of -1 give a gain of 0: every layer adds nothing and the logits are the oracle's
    w2 = dict(w)
    for l in range(cfg["num_hidden_layers"]):
        for name in ("post_attention_layernorm", "post_feedforward_layernorm"):
            w2[f"model.layers.{l}.{name}.weight"] = -torch.ones_like(w[f"model.layers.{l}.{name}.weight"])
    assert torch.allclose(plain.forward(cfg, w2, toks), oracle)
    assert not torch.allclose(plain.forward(cfg, w, toks), oracle, atol=1e-3)
    capped = plain.forward(dict(cfg, final_logit_softcapping=3.0), w, toks)
    assert float(capped.abs().max()) <= 3.0
    assert torch.equal(capped.argmax(-1), plain.forward(cfg, w, toks).argmax(-1))           # the cap is monotone


def test_post_norms_stand_on_the_sub_layers_outputs(folder_b):
    """The norm after the mixer (and after the feed-forward) normalises that sub-layer's OUTPUT before the residual sum
    (runtime/src/lib.rs:4530-4533): an RMS norm forgets its input's scale, so output projections eight times as large
    leave the logits where they were (up to the norm's eps).  A post-norm applied to the sub-layer's input instead, or
    none at all, lets the factor of eight through."""
    cfg, w = plain.read_folder(folder_b)
    toks = random_tokens(19, cfg["vocab_size"], 2)
    w8 = dict(w)
    for l in range(cfg["num_hidden_layers"]):
        for name in ("self_attn.o_proj", "mlp.down_proj"):
            w8[f"model.layers.{l}.{name}.weight"] = 8.0 * w[f"model.layers.{l}.{name}.weight"]
    ref, got = plain.forward(cfg, w, toks), plain.forward(cfg, w8, toks)
    assert rel_l2(got, ref) < 1e-3, rel_l2(got, ref)

    def post_norm_on_the_input(x, positions, W, layer, c, rnd, angle_dtype=None):     # the mistake: it passes the factor on
        p = f"model.layers.{layer}."
        n = plain.rms_norm(plain.rms_norm(x, W[p + "input_layernorm.weight"], c["rms_norm_eps"]), W[p + "post_attention_layernorm.weight"], c["rms_norm_eps"])
        x = x + plain.attention_block(n, positions, W, p, c, plain.layer_window(c, layer), rnd)
        n = plain.rms_norm(plain.rms_norm(x, W[p + "pre_feedforward_layernorm.weight"], c["rms_norm_eps"]), W[p + "post_feedforward_layernorm.weight"], c["rms_norm_eps"])
        return x + plain.geglu(n, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"], rnd)
    right = plain.block
    try:
        plain.block = post_norm_on_the_input
        assert rel_l2(plain.forward(cfg, w8, toks), plain.forward(cfg, w, toks)) > 0.1
    finally:
        plain.block = right


def test_shifting_all_positions_changes_nothing(folder_b):
    cfg, w = plain.read_folder(folder_b)
    toks = random_tokens(20, cfg["vocab_size"], 2)
    assert torch.allclose(plain.forward(cfg, w, toks), plain.forward(cfg, w, toks, first_position=1000), atol=1e-9)


def test_local_layers_forget_and_global_layers_do_not(folder_b):
    cfg, w = plain.read_folder(folder_b)                                                    # window 16, layers 0 and 2 local
    toks = random_tokens(60, cfg["vocab_size"], 3)
    other = list(toks)
    other[0] = (toks[0] + 1) % cfg["vocab_size"]
    a, b = plain.forward(cfg, w, toks), plain.forward(cfg, w, other)
    assert not torch.allclose(a[59], b[59], atol=1e-9)                                      # layer 1 still sees token 0
    only_local = dict(cfg, layer_types=None)
    plain_window = plain.layer_window
    try:
        plain.layer_window = lambda c, l: c["sliding_window"]                               # every layer local
        a, b = plain.forward(only_local, w, toks), plain.forward(only_local, w, other)
    finally:
        plain.layer_window = plain_window
    assert torch.equal(a[3 * 15 + 1:], b[3 * 15 + 1:]) and not torch.allclose(a[30], b[30], atol=1e-12)


def test_layer_0_is_local_and_layer_types_overrides(folder_b):
    """A model of layer 0 alone (window 16): a changed token 0 leaves the logits at positions >= 16 untouched, because an
    even layer is local; `layer_types` naming it full_attention flips that.  Fails when the parity in plain.layer_window
    is swapped (layer 0 global), or when `layer_types` is ignored."""
    cfg, w = plain.read_folder(folder_b)
    one = dict(cfg, num_hidden_layers=1)
    toks = random_tokens(40, cfg["vocab_size"], 5)
    other = [(toks[0] + 1) % cfg["vocab_size"]] + toks[1:]
    a, b = plain.forward(one, w, toks), plain.forward(one, w, other)
    assert torch.equal(a[16:], b[16:]) and not torch.allclose(a[15], b[15], atol=1e-9)
    full = dict(one, layer_types=["full_attention"])
    a, b = plain.forward(full, w, toks), plain.forward(full, w, other)
    assert not torch.allclose(a[39], b[39], atol=1e-9)
    two = dict(cfg, num_hidden_layers=2, layer_types=["full_attention", "sliding_attention"])
    assert not torch.allclose(plain.forward(two, w, toks)[39], plain.forward(dict(cfg, num_hidden_layers=2), w, toks)[39], atol=1e-9)


# ---- token choice --------------------------------------------------------------------------------------------------
def test_argmax_ties():
    z = [-1.0] * 7001
    z[100] = z[7000] = 5.0                                     # the reference's vector: runtime/src/bin/opt_check.rs:37-65
    assert plain.argmax(z) == 100
    assert plain.argmax([2.0, 2.0, 1.0]) == 0


def test_sampler():
    z = torch.tensor([0.1, 2.0, -1.0, 1.9, 0.5])
    assert plain.sample(z, 0.0, 1.0, 0, 0.3) == 1
    assert all(plain.sample(z, 1e-4, 1.0, 5, u) == 1 for u in (0.0, 0.5, 0.999))            # T -> 0: greedy
    assert plain.sample(z, 1.0, 1e-9, 5, 0.99) == 1                                           # a tiny nucleus keeps the top only
    assert {plain.sample(z, 1.0, 1.0, 2, u) for u in (0.0, 0.4, 0.6, 0.99)} == {1, 3}        # top_k = 2
    p = torch.softmax(z.double() / 0.7, 0)
    n, counts = 20000, [0] * 5
    state = 12345
    for _ in range(n):
        state = plain.xorshift64(state)
        counts[plain.sample(z, 0.7, 1.0, 5, plain.uniform_from_state(state))] += 1
    chi2 = sum((c - n * float(q)) ** 2 / (n * float(q)) for c, q in zip(counts, p))
    assert chi2 < 18.5                                                                        # 4 degrees of freedom, p = 0.001
    # sorted walk: u below the top's probability picks the top, just above it the second
    order = sorted(range(5), key=lambda i: -float(z[i]))
    assert plain.sample(z, 0.7, 1.0, 5, float(p[order[0]]) - 1e-6) == order[0]
    assert plain.sample(z, 0.7, 1.0, 5, float(p[order[0]]) + 1e-6) == order[1]


def test_repetition_penalty_and_generator():
    z = torch.tensor([2.0, -2.0, 1.0, 0.5])
    got = plain.repetition_penalty(z, [0, 1, 1, 0], 2.0)
    assert got.tolist() == [1.0, -4.0, 1.0, 0.5] and z[0] == 2.0                              # each token once, by sign
    assert plain.repetition_penalty(z, [0], 1.0) is z
    s = plain.xorshift64(1)
    assert s == ((1 ^ (1 << 13)) ^ ((1 ^ (1 << 13)) >> 7)) ^ ((((1 ^ (1 << 13)) ^ ((1 ^ (1 << 13)) >> 7)) << 17) & ((1 << 64) - 1))
    assert 0.0 <= plain.uniform_from_state(s) < 1.0


def test_greedy_loop_stops_before_the_stop_token(folder_b):
    cfg, w = plain.read_folder(folder_b)
    p = random_tokens(6, cfg["vocab_size"], 4)
    free = plain.greedy_generate(cfg, w, p, 5)
    assert len(free) == 5
    assert plain.greedy_generate(cfg, w, p, 5, stop_ids=(free[2],)) == free[:free.index(free[2])]
