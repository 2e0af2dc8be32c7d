"""Grouped-query attention over the cache, with optional score cap and window.

In the reference's order (runtime/src/lib.rs:4483-4496): q, k, v projections,
RoPE on q and k, append k (rotated) and v to the cache, attention, output
projection.  Scores: (q . k) * query_scale, then cap * tanh(s / cap) when a cap is
set, softmax in fp32 over the visible keys, weighted sum of v; query head h reads
kv head h // (heads / kv_heads) (runtime/cuda/codebook_gemv.cu:240-270).  The
reference fixes the scale to rsqrt(head_dim) (cu:249) and has no window
(lib.rs:4455); both are parameters here: the query at position p sees keys
t <= p, and with a window W only those with p - t < W.

The three projections are one product over the concatenated weight.  A run that
reads another run's cache projects and rotates its queries only.  In a decode step
rotation, cache write and attention are one kernel launch where the kernel library
has one for the geometry (`ops.fuses_decode_step`); the order of the arithmetic is
the same.  A step that continues sequences by several tokens, or mixes starting and running sequences, attends
over the cached positions its queries still see, read in place through the page table, plus its own rows (the
reference's multi-token step walks its cache from any position: runtime/src/lib.rs:676-720,
runtime/cuda/codebook_gemv.cu:410-440), and caches its own rows after the attention.
"""
from ..cache.store import TokenSpec
from ..models.spec import TensorSpec
from ..registry import build_part, register_part
from .base import Mixer


class Attention(Mixer):
    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, query_scale,
                 softcap=None, window=None, position=("none", {})):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are no multiple of {num_kv_heads} kv heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.query_scale = float(query_scale)
        self.softcap = float(softcap) if softcap else 0.0
        self.window = int(window) if window else 0
        self.position = build_part("position", position)
        if self.position.rotary_dim > head_dim:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head_dim {head_dim}")

    def tensor_specs(self):
        d, q, kv = self.hidden_size, self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        return {"q_proj.weight": TensorSpec((q, d)), "k_proj.weight": TensorSpec((kv, d)),
                "v_proj.weight": TensorSpec((kv, d)), "o_proj.weight": TensorSpec((d, q))}

    def cache_spec(self):
        per_token = (self.num_kv_heads, self.head_dim)
        return TokenSpec.of(self.window or None, k=per_token, v=per_token)

    def bind(self, tensors, rt):
        import torch
        self.rt = rt
        self.w_qkv = rt.matrix(torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"],
                                          tensors["v_proj.weight"]], dim=0)).contiguous()
        self.w_o = rt.matrix(tensors["o_proj.weight"])
        self.inv_freq = self.position.inv_freq(rt.device)

    def forward(self, ctx, x, site):
        ops = ctx.ops
        H, KV, hd = self.num_heads, self.num_kv_heads, self.head_dim
        Q, KVD = H * hd, KV * hd
        owns_cache = ctx.cache_owner == ctx.entry
        if site.spec.window is not None and not 0 < self.window <= site.spec.window:
            raise ValueError(f"this attention sees {self.window or 'all'} keys back, the cache it reads keeps {site.spec.window}")
        table = ctx.page_table(site.group_index)
        k_pool, v_pool = site.tensor("k"), site.tensor("v")         # [pages, kv_heads, page, head_dim]
        rows_cap = site.rows_cap or 0
        pairing = self.position.pairing
        if ctx.mode == "decode" and pairing == "halves" and ops.fuses_decode_step(ctx.dtype, H, KV, hd, k_pool):
            # one launch rotates, writes the cache and attends; the projections may stay in K slices until then
            qkv = ops.linear(x, self.w_qkv if owns_cache else self.w_qkv[:Q], ctx.dtype, defer=True)
            out = ops.attention_decode_step(qkv, H, KV, hd, self.inv_freq, self.position.rotary_dim, ctx.new_len,
                                            table, k_pool, v_pool, rows_cap, self.query_scale, self.softcap,
                                            self.window, ctx.dtype, max_keys=ctx.max_rows_visible(site), write_kv=owns_cache)
            return ops.linear(out, self.w_o, ctx.dtype, defer=True)
        if owns_cache:
            qkv = ops.linear(x, self.w_qkv, ctx.dtype)
            q, k, v = qkv[:, :Q], qkv[:, Q:Q + KVD], qkv[:, Q + KVD:]
        else:
            q, k, v = ops.linear(x, self.w_qkv[:Q], ctx.dtype), None, None
        if ctx.mode == "decode":
            ops.rope_kv_write(q, k, v, H, KV, hd, self.inv_freq, self.position.rotary_dim,
                              ctx.row_seq, ctx.row_pos, ctx.new_len, table, k_pool, v_pool, rows_cap, pairing=pairing)
            out = ops.attention_decode(q, H, KV, hd, ctx.new_len, table, k_pool, v_pool, rows_cap,
                                       self.query_scale, self.softcap, self.window, ctx.dtype,
                                       max_keys=ctx.max_rows_visible(site))
            return ops.linear(out, self.w_o, ctx.dtype, defer=True)
        # Sequences that go on by several tokens (or some start while others go on) see cached positions and the
        # step's own rows.  The attention reads the cached ones where they lie, as earlier steps left them, and the
        # step's rows from the step; only then are the step's rows cached: in a window's ring without a row to spare
        # they take the places of positions that the step's earlier queries still see.
        extend = ctx.mode == "extend"
        ops.rope_kv_write(q, k, v, H, KV, hd, self.inv_freq, self.position.rotary_dim,
                          ctx.row_seq, ctx.row_pos, ctx.new_len, table, k_pool, v_pool, rows_cap, pairing=pairing,
                          write=not extend)
        if owns_cache:
            ctx.offer_step_rows(k=k, v=v)
        else:
            theirs = ctx.step_rows_of(ctx.cache_owner)
            k, v = theirs["k"], theirs["v"]
        out = ops.attention_prefill(q, k, v, H, KV, hd, ctx.cu_rows, ctx.max_count,
                                    self.query_scale, self.softcap, self.window, ctx.dtype,
                                    row_seq=ctx.row_seq, row_pos=ctx.row_pos,
                                    cached=(ctx.new_len, table, k_pool, v_pool, rows_cap) if extend else None)
        if extend and owns_cache:
            row_seq, row_pos, new_len = ctx.row_seq, ctx.row_pos, ctx.new_len
            ctx.after_readers(lambda: ops.kv_write(k, v, KV, hd, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap))
        return ops.linear(out, self.w_o, ctx.dtype, defer=True)


register_part("mixer", "attention", Attention)
