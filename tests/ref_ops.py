"""Plain torch references of the kernel library, one function per kernel, same signatures.

Two uses: the GPU tests compare each HIP kernel with its function here, and the
CPU tests run the engine's host logic (cache, step, batching, generation) on
these instead of the HIP library.  fp32 arithmetic, rounded once to the output
dtype, like the kernels.  None of this is on the product path.
"""
import math

import torch

GROUP = 16          # rows of gate, then rows of up, alternate in groups of this many


def pack_gate_up(w_gate, w_up):
    i, k = w_gate.shape
    ip = -(-i // GROUP) * GROUP
    g = torch.zeros((ip, k), dtype=w_gate.dtype, device=w_gate.device)
    u = torch.zeros_like(g)
    g[:i], u[:i] = w_gate, w_up
    return torch.stack([g.reshape(-1, GROUP, k), u.reshape(-1, GROUP, k)], dim=1).reshape(2 * ip, k).contiguous()


def embed_rows(tokens, table, scale):
    return table[tokens.long()].float() * scale


def _norm(x, gain, eps):
    x = x.float()
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gain


def rms_norm(x, gain, eps, out_dtype):
    return _norm(x, gain, eps).to(out_dtype)


def add_rms_norm(stream, rows, gain_post, eps_post, gain_next, eps_next, out_dtype):
    t = rows.float() if gain_post is None else _norm(rows, gain_post, eps_post)
    stream += t
    if gain_next is None:
        return None
    return _norm(stream, gain_next, eps_next).to(out_dtype)


def linear(x, w, out_dtype, softcap=None, defer=False, bias=None):
    y = x.float() @ w.float().T
    if bias is not None:
        y = y + bias.float()
    if softcap:
        y = softcap * torch.tanh(y / softcap)
    return y.to(out_dtype)


def _gelu_tanh(g):
    return 0.5 * g * (1.0 + torch.tanh(0.7978845608 * (g + 0.044715 * g * g * g)))


def gated_linear(x, w_packed, inter, activation, out_dtype):
    act = {"gelu_tanh": _gelu_tanh, "silu": lambda g: g * torch.sigmoid(g)}[activation]
    y = x.float() @ w_packed.float().T                     # [M, 2 * ip]
    y = y.reshape(x.shape[0], -1, 2, GROUP)
    g, u = y[:, :, 0, :].reshape(x.shape[0], -1), y[:, :, 1, :].reshape(x.shape[0], -1)
    return (act(g) * u)[:, :inter].to(out_dtype).contiguous()


def _rotate(x, pos, inv_freq, rotary_dim, pairing="halves"):
    """x [M, heads, hd] fp32, pos [M]."""
    if inv_freq is None or rotary_dim == 0:
        return x
    half = rotary_dim // 2
    ang = pos.float()[:, None] * inv_freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    if pairing == "neighbours":                          # pair d: elements 2d and 2d + 1
        x0, x1 = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        turned = torch.stack([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1).reshape(*x.shape[:-1], rotary_dim)
        return torch.cat([turned, x[..., rotary_dim:]], dim=-1)
    x0, x1 = x[..., :half], x[..., half:rotary_dim]
    return torch.cat([x0 * c - x1 * s, x1 * c + x0 * s, x[..., rotary_dim:]], dim=-1)


def _cache_rows(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap):
    KV, page, hd = k_pool.shape[1], k_pool.shape[2], k_pool.shape[3]
    for r in range(k.shape[0]):
        s, p = int(row_seq[r]), int(row_pos[r])
        row = p
        if rows_cap:
            if p + rows_cap < int(new_len[s]):
                continue                                  # a later row of this step lands on the same ring row
            row = p % rows_cap
        pg = int(table[s, row // page])
        assert pg >= 0
        k_pool[pg, :, row % page, :] = k[r].reshape(KV, hd)
        v_pool[pg, :, row % page, :] = v[r].reshape(KV, hd)


def rope_kv_write(q, k, v, H, KV, hd, inv_freq, rotary_dim, row_seq, row_pos, new_len, table,
                  k_pool, v_pool, rows_cap, pairing="halves", write=True):
    m = q.shape[0]
    q.copy_(_rotate(q.float().reshape(m, H, hd), row_pos, inv_freq, rotary_dim, pairing).reshape(m, H * hd).to(q.dtype))
    if k is None:
        return
    k.copy_(_rotate(k.float().reshape(m, KV, hd), row_pos, inv_freq, rotary_dim, pairing).reshape(m, KV * hd).to(k.dtype))
    if write:
        _cache_rows(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap)


def kv_write(k, v, KV, hd, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap):
    _cache_rows(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap)


def _attend(qrow, keys, vals, scale, softcap):
    """qrow [hd], keys/vals [n, hd], fp32."""
    s = (keys @ qrow) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    p = torch.softmax(s, dim=0)
    return p @ vals


def attention_prefill(q, k, v, H, KV, hd, cu_rows, max_count, scale, softcap, window, out_dtype, row_seq=None, row_pos=None,
                      cached=None, shape=0):
    """k, v: the step's own rows.  cached None: every sequence starts at position 0.  Else cached = (new_len, table,
    k_pool, v_pool, rows_cap): sequence i's first row stands at new_len[i] - its count, and the positions before it are
    read from the cache as it is."""
    m = q.shape[0]
    out = torch.zeros((m, H * hd), dtype=torch.float32, device=q.device)
    qf, kf, vf = q.float().reshape(m, H, hd), k.float().reshape(-1, KV, hd), v.float().reshape(-1, KV, hd)
    g = H // KV
    for i in range(len(cu_rows) - 1):
        a, b = int(cu_rows[i]), int(cu_rows[i + 1])
        start, keys, vals = 0, kf[a:b], vf[a:b]
        if cached is not None:
            new_len, table, k_pool, v_pool, rows_cap = cached
            page = k_pool.shape[2]
            start = int(new_len[i]) - (b - a)
            first = max(0, start - (window - 1)) if window else 0       # the earliest position any query of the step sees
            pos = torch.arange(first, start)
            rows = pos % rows_cap if rows_cap else pos
            pages = table[i].long()[rows // page]
            assert (pages >= 0).all()
            keys = torch.cat([torch.zeros(first, KV, hd), k_pool[pages, :, rows % page, :].float().cpu(), kf[a:b].cpu()]).to(q.device)
            vals = torch.cat([torch.zeros(first, KV, hd), v_pool[pages, :, rows % page, :].float().cpu(), vf[a:b].cpu()]).to(q.device)
        for r in range(a, b):
            p = start + r - a
            lo = 0 if not window else max(0, p - window + 1)
            for h in range(H):
                out[r, h * hd:(h + 1) * hd] = _attend(qf[r, h], keys[lo:p + 1, h // g], vals[lo:p + 1, h // g], scale, softcap)
    return out.to(out_dtype)


def attention_decode(q, H, KV, hd, new_len, table, k_pool, v_pool, rows_cap, scale, softcap, window, out_dtype, max_keys=None):
    n = q.shape[0]
    page = k_pool.shape[2]
    out = torch.zeros((n, H * hd), dtype=torch.float32, device=q.device)
    qf = q.float().reshape(n, H, hd)
    g = H // KV
    for i in range(n):
        p = int(new_len[i]) - 1
        lo = 0 if not window else max(0, p - window + 1)
        pos = torch.arange(lo, p + 1)
        rows = pos % rows_cap if rows_cap else pos
        pages = table[i].long()[rows // page]
        assert (pages >= 0).all()
        keys = k_pool[pages, :, rows % page, :].float()          # [n_keys, KV, hd]
        vals = v_pool[pages, :, rows % page, :].float()
        for h in range(H):
            out[i, h * hd:(h + 1) * hd] = _attend(qf[i, h], keys[:, h // g], vals[:, h // g], scale, softcap)
    return out.to(out_dtype)


def fuses_decode_step(dtype, H, KV, hd, k_pool):
    return False


def attention_decode_step(qkv, H, KV, hd, inv_freq, rotary_dim, new_len, table, k_pool, v_pool, rows_cap, scale, softcap,
                          window, out_dtype, max_keys=None, write_kv=True, splits=None):
    """The fused decode step as its three parts: qkv float32 [n, (H + 2 KV) hd] (already summed over K slices),
    rotated in float32 and rounded once to the cache's dtype."""
    n = qkv.shape[0]
    pos = new_len.to(torch.int32) - 1
    q = _rotate(qkv[:, :H * hd].float().reshape(n, H, hd), pos, inv_freq, rotary_dim).reshape(n, H * hd).to(k_pool.dtype)
    if write_kv:
        k = _rotate(qkv[:, H * hd:(H + KV) * hd].float().reshape(n, KV, hd), pos, inv_freq, rotary_dim).to(k_pool.dtype)
        v = qkv[:, (H + KV) * hd:].reshape(n, KV, hd).to(k_pool.dtype)
        page = k_pool.shape[2]
        for i in range(n):
            row = int(pos[i]) % rows_cap if rows_cap else int(pos[i])
            pg = int(table[i, row // page])
            assert pg >= 0
            k_pool[pg, :, row % page, :] = k[i]
            v_pool[pg, :, row % page, :] = v[i]
    return attention_decode(q, H, KV, hd, new_len, table, k_pool, v_pool, rows_cap, scale, softcap, window, out_dtype)


def rows(r, dtype):
    return r


def gather_rows(x, rows):
    return x[rows.long()].contiguous()


def argmax(logits):
    """Smallest index among the largest values."""
    mx = logits.max(dim=-1, keepdim=True).values
    idx = torch.arange(logits.shape[-1], device=logits.device).expand_as(logits)
    big = torch.full_like(idx, logits.shape[-1])
    return torch.where(logits == mx, idx, big).min(dim=-1).values.to(torch.int32)


def apply_repetition_penalty(logits, recent, penalty):
    """recent int32 [B, R], -1 = empty; each distinct token once: z / penalty if z > 0 else z * penalty."""
    if penalty <= 1.0:
        return
    for b in range(logits.shape[0]):
        for t in set(int(x) for x in recent[b] if int(x) >= 0):
            z = logits[b, t]
            logits[b, t] = z / penalty if z > 0 else z * penalty


def sample(logits, temperature, top_k, top_p, uniforms):
    """Per row: the top_k largest (ties: smaller id first), p = softmax((z - max) / T) over them, the
    shortest prefix with mass >= top_p, walk with r = u * kept mass.  Returns int32 [B]."""
    out = []
    for b in range(logits.shape[0]):
        z = logits[b].double()
        k = min(top_k, z.numel()) if top_k > 0 else z.numel()
        if top_k > 0:
            order = sorted(range(z.numel()), key=lambda i: (-float(z[i]), i))[:k]
        else:
            order = list(range(z.numel()))            # the whole vocabulary, in id order, no nucleus
        zs = torch.tensor([float(z[i]) for i in order], dtype=torch.float64)
        p = torch.exp((zs - zs.max()) / temperature)
        p = p / p.sum()
        cum = torch.cumsum(p, 0)
        keep = k
        for j in range(k):
            if float(cum[j]) >= top_p:
                keep = j + 1
                break
        r = float(uniforms[b]) * float(p[:keep].sum())
        tok = order[0]
        for j in range(keep):
            if r < float(p[j]):
                tok = order[j]
                break
            r -= float(p[j])
        out.append(tok)
    return torch.tensor(out, dtype=torch.int32, device=logits.device)
