"""Plain Gemma-2: whole sequences, no cache, one function for each part.

Written from the formulas of the reference runtime (paths relative to the
reference checkout); it shares no code with the engine.  Every function takes
its sizes and constants as arguments.  Arithmetic runs in `dtype` (float64 by
default); `rnd` is an optional rounding hook applied where a reduced-precision
engine stores an activation, so that a comparison measures summation order
rather than storage width (the reference's CPU twins do the same with fp16:
runtime/src/bin/attn.rs:27-29, model.rs:44-129).
"""
import json
import math
import os
import struct

import torch


# ----------------------------------------------------------------------------
# reading a model folder (own reader; format facts from model/export_safetensors.py:24-48)
# ----------------------------------------------------------------------------
_DT = {"F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
       "F64": torch.float64, "I32": torch.int32, "I64": torch.int64}


def read_folder(folder, dtype=torch.float64):
    """config dict and {name: tensor in `dtype`} of a folder with config.json + model.safetensors."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    out = {}
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        raw = f.read()
    n = struct.unpack("<Q", raw[:8])[0]
    hdr = json.loads(raw[8:8 + n])
    base = 8 + n
    for name, meta in hdr.items():
        if name == "__metadata__":
            continue
        s, e = meta["data_offsets"]
        t = torch.frombuffer(bytearray(raw[base + s:base + e]), dtype=_DT[meta["dtype"]])
        out[name] = t.reshape(meta["shape"]).to(dtype)
    return cfg, out


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------
def rms_norm(x, w, eps):
    """y = x * rsqrt(mean(x^2) + eps) * (1 + w).

    runtime/cuda/codebook_gemv.cu:192-202 (sum of squares / n + eps, rsqrt, times weight)
    with the weight being 1 + w: model/export_gemma.py:25-26.
    """
    ss = (x * x).sum(dim=-1, keepdim=True)
    scale = torch.rsqrt(ss / x.shape[-1] + eps)
    return (x * scale) * (1.0 + w)


def rope_inv_freq(head_dim, theta, dtype):
    """inv_freq[d] = 1 / theta^(2d / head_dim), d in [0, head_dim/2).  model/export_gemma.py:53."""
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=dtype) / head_dim))


def rope(x, positions, theta, angle_dtype=None):
    """Rotate-half RoPE on x [T, heads, head_dim] at integer `positions` [T].

    Pair (d, d + head_dim/2), angle = pos * inv_freq[d]:
    x[d]' = x[d] cos - x[d+half] sin ; x[d+half]' = x[d+half] cos + x[d] sin.
    runtime/cuda/codebook_gemv.cu:219-230.
    `angle_dtype`: the width the table and the angle are formed in.  The reference forms both in 32-bit
    (model/export_gemma.py:53 `.float()`, codebook_gemv.cu:225 `(float)pos * inv_freq[d]`), whose rounding of an
    angle of some thousand radians is about pos * 1e-7: nothing at the positions of a short test, a few 1e-5 of the
    logits at positions beyond 4,000.  None: exact angles in x's own width.
    """
    hd = x.shape[-1]
    half = hd // 2
    adt = angle_dtype or x.dtype
    inv = rope_inv_freq(hd, theta, adt)
    ang = (positions.to(adt)[:, None] * inv[None, :]).to(x.dtype)      # [T, half]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x0, x1 = x[..., :half], x[..., half:]
    return torch.cat([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1)


def softcap(s, cap):
    """cap * tanh(s / cap) when cap is set (> 0).  runtime/cuda/codebook_gemv.cu:255, runtime/src/lib.rs:4560."""
    if cap is None or cap <= 0:
        return s
    return cap * torch.tanh(s / cap)


def attention(q, k, v, scale, cap, window):
    """Causal grouped-query attention over one whole sequence.

    q [T, H, hd], k, v [T, KV, hd] -> [T, H, hd].  Query head h reads kv head
    h // (H // KV); score = (q . k) * scale, then the soft cap, then a softmax
    over the visible keys, then the weighted sum of v
    (runtime/cuda/codebook_gemv.cu:240-270; the reference's scale is
    rsqrt(head_dim), here an argument).  Visible keys of the query at p:
    t <= p, and with a window W also p - t < W (the reference models no window,
    runtime/src/lib.rs:4455; W keys including the query's own).
    """
    T, H, hd = q.shape
    KV = k.shape[1]
    group = H // KV
    out = torch.zeros_like(q)
    for h in range(H):
        g = h // group
        for p in range(T):
            lo = 0 if window is None else max(0, p - window + 1)
            s = (k[lo:p + 1, g, :] @ q[p, h, :]) * scale
            s = softcap(s, cap)
            e = torch.exp(s - s.max())
            prob = e / e.sum()
            out[p, h, :] = prob @ v[lo:p + 1, g, :]
    return out


def gelu_tanh(g):
    """0.5 g (1 + tanh(0.7978845608 (g + 0.044715 g^3))).  runtime/cuda/codebook_gemv.cu:531-537."""
    return 0.5 * g * (1.0 + torch.tanh(0.7978845608 * (g + 0.044715 * g * g * g)))


def geglu(x, w_gate, w_up, w_down, rnd):
    """down(gelu_tanh(gate x) * up x); gate and up stay unrounded.  runtime/src/lib.rs:4511-4516."""
    act = rnd(gelu_tanh(x @ w_gate.T) * (x @ w_up.T))
    return act @ w_down.T


def embed(tokens, table, hidden):
    """table[token] * sqrt(hidden).  model/export_gemma.py:59-61."""
    return table[tokens] * math.sqrt(hidden)


def attention_block(x, positions, W, p, cfg, window, rnd, angle_dtype=None):
    """q/k/v projections, RoPE on q and k, attention, output projection.  runtime/src/lib.rs:4483-4496."""
    T = x.shape[0]
    H, KV, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = rnd(x @ W[p + "self_attn.q_proj.weight"].T).reshape(T, H, hd)
    k = rnd(x @ W[p + "self_attn.k_proj.weight"].T).reshape(T, KV, hd)
    v = rnd(x @ W[p + "self_attn.v_proj.weight"].T).reshape(T, KV, hd)
    theta = float(cfg.get("rope_theta", 10000.0))
    q, k = rnd(rope(q, positions, theta, angle_dtype)), rnd(rope(k, positions, theta, angle_dtype))
    scale = 1.0 / math.sqrt(cfg["query_pre_attn_scalar"])
    a = rnd(attention(q, k, v, scale, cfg.get("attn_logit_softcapping"), window))
    return a.reshape(T, H * hd) @ W[p + "self_attn.o_proj.weight"].T


def layer_window(cfg, layer):
    """Even layers are local (window), odd layers global, unless config.json lists `layer_types`
    (the reference models no window: runtime/src/lib.rs:4455)."""
    kinds = cfg.get("layer_types")
    if kinds:
        return cfg["sliding_window"] if kinds[layer] == "sliding_attention" else None
    return cfg["sliding_window"] if layer % 2 == 0 else None


def block(x, positions, W, layer, cfg, rnd, angle_dtype=None):
    """x += post_attn_norm(attn(input_norm(x))); x += post_ff_norm(mlp(pre_ff_norm(x))).

    runtime/src/lib.rs:4527-4540.
    """
    p = f"model.layers.{layer}."
    eps = cfg["rms_norm_eps"]
    n = rnd(rms_norm(x, W[p + "input_layernorm.weight"], eps))
    a = rnd(attention_block(n, positions, W, p, cfg, layer_window(cfg, layer), rnd, angle_dtype))
    x = x + rms_norm(a, W[p + "post_attention_layernorm.weight"], eps)
    n = rnd(rms_norm(x, W[p + "pre_feedforward_layernorm.weight"], eps))
    m = rnd(geglu(n, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"],
                  W[p + "mlp.down_proj.weight"], rnd))
    x = x + rms_norm(m, W[p + "post_feedforward_layernorm.weight"], eps)
    return x


def head(x, W, cfg, rnd):
    """final norm, tied unscaled embedding as the head, final soft cap.  runtime/src/lib.rs:4557-4560."""
    n = rnd(rms_norm(x, W["model.norm.weight"], cfg["rms_norm_eps"]))
    z = n @ W["model.embed_tokens.weight"].T
    return softcap(z, cfg.get("final_logit_softcapping"))


def forward(cfg, W, tokens, rnd=None, first_position=0, angle_dtype=None):
    """Logits [T, vocab] at every position of one whole sequence.  runtime/src/lib.rs:4553-4562.
    `angle_dtype`: see rope()."""
    rnd = rnd or (lambda t: t)
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(first_position, first_position + len(tokens))
    x = embed(tokens, W["model.embed_tokens.weight"], cfg["hidden_size"])
    for layer in range(cfg["num_hidden_layers"]):
        x = block(x, positions, W, layer, cfg, rnd, angle_dtype)
    return head(x, W, cfg, rnd)


def round_bf16(t):
    """Round through bfloat16 (round to nearest even), keeping the dtype."""
    return t.to(torch.bfloat16).to(t.dtype)


# ----------------------------------------------------------------------------
# token choice and the plain loop
# ----------------------------------------------------------------------------
def argmax(logits):
    """Strict '>' scan: the smallest index wins a tie.  runtime/src/lib.rs:1376-1380."""
    best = 0
    for i in range(1, len(logits)):
        if logits[i] > logits[best]:
            best = i
    return best


def xorshift64(state):
    """One step of the reference's generator (<<13, >>7, <<17 on 64 bits).  runtime/src/bin/serve.rs:63."""
    m = (1 << 64) - 1
    state ^= (state << 13) & m
    state ^= state >> 7
    state ^= (state << 17) & m
    return state


def uniform_from_state(state):
    """(state >> 11) / 2^53.  runtime/src/bin/serve.rs:65."""
    return (state >> 11) / float(1 << 53)


def repetition_penalty(logits, recent, penalty):
    """Each distinct recent token: logit / penalty if > 0 else logit * penalty.  runtime/src/bin/serve.rs:285-294."""
    if penalty <= 1.0:
        return logits
    logits = logits.clone()
    for t in set(recent):
        logits[t] = logits[t] / penalty if logits[t] > 0 else logits[t] * penalty
    return logits


def sample(logits, temperature, top_p, top_k, u):
    """Greedy for temperature <= 0; else the top_k largest (ties: smaller id first),
    softmax((z - max) / T), the shortest prefix whose mass reaches top_p, and a walk
    with r = u * kept mass.  runtime/src/bin/serve.rs:41-72 (top_k is 256 there).
    top_k 0 (not in the reference): the whole vocabulary in id order, no nucleus."""
    z = [float(v) for v in logits]
    if temperature <= 0:
        return argmax(z)
    if top_k > 0:
        idx = sorted(range(len(z)), key=lambda i: (-z[i], i))[:top_k]
        mx = z[idx[0]]
    else:
        assert top_p >= 1
        idx = list(range(len(z)))
        mx = max(z)
    probs = [math.exp((z[i] - mx) / temperature) for i in idx]
    total = sum(probs)
    probs = [p / total for p in probs]
    keep, cum = len(probs), 0.0
    for k, p in enumerate(probs):
        cum += p
        if cum >= top_p:
            keep = k + 1
            break
    r = u * sum(probs[:keep])
    for k in range(keep):
        if r < probs[k]:
            return idx[k]
        r -= probs[k]
    return idx[0]


def greedy_generate(cfg, W, prompt, n_new, stop_ids=()):
    """Prefill, then push-token / forward / argmax; a stop token ends it and is not kept.

    runtime/src/lib.rs:1574-1588 (loop), runtime/src/bin/serve.rs:347-350 (stop before push).
    Every step recomputes the whole sequence: no cache.
    """
    seq = list(prompt)
    out = []
    while len(out) < n_new:
        tok = argmax(forward(cfg, W, seq)[-1])
        if tok in stop_ids:
            break
        out.append(tok)
        seq.append(tok)
    return out
