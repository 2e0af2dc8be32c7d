"""The HIP kernel library behind the parts: thin, checking wrappers over its C entry points.

Every function takes torch tensors on the GPU, checks shape, dtype and layout on the host (a kernel is never
launched on operands it does not fit), and enqueues on torch's current stream.  There is no CPU path: without
a GPU or a compiled library, loading fails with an error.
"""
import ctypes

import torch

from . import build as _build

_c = ctypes
_P, _I, _L, _F = _c.c_void_p, _c.c_int, _c.c_long, _c.c_float

_CORE_SIGS = {
    "tp_embed_rows": [_P, _P, _I, _F, _P, _I, _I, _I, _P],
    "tp_rms_norm": [_P, _I, _P, _F, _P, _I, _I, _I, _P],
    "tp_add_rms_norm": [_P, _P, _I, _I, _L, _P, _F, _P, _F, _P, _I, _I, _I, _P],
    "tp_gather_rows": [_P, _P, _P, _I, _I, _I, _P],
    "tp_sum_slices": [_P, _I, _L, _P, _I, _L, _P],
    "tp_rope_kv_write": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _P],
    "tp_kv_write": [_P, _L, _P, _L, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _P],
    "tp_gated_act": [_P, _P, _I, _I, _I, _I, _P],
    "tp_linear": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P, _L, _I, _I, _P],
    "tp_linear_workspace_bytes": [_I, _I, _I, _I, _I, _I, _I, _I, _I],
    "tp_attn_simple_prefill": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _P, _P],
    "tp_attn_simple_decode": [_P, _L, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _P, _P],
    "tp_argmax": [_P, _I, _I, _P, _P, _P],
    "tp_argmax_workspace_bytes": [_I, _I],
    "tp_repetition_penalty": [_P, _I, _I, _P, _I, _F, _P],
    "tp_recent_push": [_P, _P, _P, _I, _I, _P],
    "tp_add_bias": [_P, _I, _P, _I, _I, _P],
    "tp_sample": [_P, _I, _I, _F, _I, _F, _P, _P, _P, _P],
    "tp_sample_workspace_bytes": [_I, _I],
    "tp_probe_stream": [_P, _L, _P, _I, _P],
    "tp_probe_mfma": [_I, _I, _I, _P, _P, _P],
}
_ATTN_SIGS = {
    "tp_attn_prefill": [_P, _L, _P, _L, _P, _L, _I, _I, _I, _P, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _P, _I, _P],
    "tp_attn_decode": [_P, _L, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _P, _P, _I, _P],
    "tp_attn_decode_workspace_floats": [_I, _I, _I],
    "tp_attn_decode_fused": [_P, _I, _I, _L, _L, _P, _I, _I, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _F, _I, _P, _P, _I, _P],
}

EPI_NONE, EPI_SOFTCAP, EPI_GATED = 0, 1, 2
ROPE_PAIRINGS = {"halves": 0, "neighbours": 1}          # the kernel library's TP_ROPE_* enumerators
GATE_ACTIVATIONS = {"gelu_tanh": 0, "silu": 1}       # what a gated product's epilogue can apply to the gate
GATE_GROUP = 16


class KernelError(RuntimeError):
    """A kernel refused its operands, or the library could not be loaded."""


class SplitRows:
    """Rows of a product still in K slices: fp32 [slices, M, N], to be added in slice order by the kernel that
    consumes them (`add_rms_norm`), which saves a launch and a rounding.  `HipOps.rows()` adds them otherwise."""

    def __init__(self, slices):
        self.slices = slices
        self.shape = tuple(slices.shape[1:])
        self.dtype = torch.float32


def _code(dtype):
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise KernelError(f"dtype {dtype} is not supported by the kernels (float32 or bfloat16)")


def _bind(lib, sigs):
    lib.tp_last_error.restype = _c.c_char_p
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = _c.c_long if name.endswith(("_bytes", "_floats", "_elems")) else _I


class HipOps:
    def __init__(self, device):
        if device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError(
                "the HIP kernels need an AMD GPU: no CPU path exists (device %s, torch.cuda.is_available() = %s)"
                % (device, torch.cuda.is_available()))
        self.device = device
        try:
            path = _build.build_core()
            self.lib = _c.CDLL(path)
        except (OSError, _build.BuildError) as e:
            raise KernelError(f"the HIP kernel library could not be built or loaded: {e}") from None
        _bind(self.lib, _CORE_SIGS)
        self._attn = {}
        self._sample_ws = {}
        from .. import flags
        plain = flags.force_plain()
        self.force_linear = 1 if plain else 0   # 1 plain, 2 skinny, 3 tiled (6: its wide tile, 7: its 128 x 96 tile, 8, 9: loads into LDS, 128 x 128 and 128 x 96; 10, 11: 64 x 32 and 64 x 64 tiles, two k steps ahead), 4 multiply-adds (1-2 rows), 5 blocks of 8 rows of W
        self.force_plain_attention = plain
        self._timed = None                      # with TRAPETUM_AMD_PROFILE=1: [(entry point, start event, end event)] not yet summed
        self._profile_totals = {}               # entry point -> (milliseconds, calls)
        if flags.profile():
            import atexit
            self._timed = []
            atexit.register(self.profile_report)

    # ---- helpers -----------------------------------------------------------------------------------
    def _stream(self):
        return torch.cuda.current_stream(self.device).cuda_stream

    def _call(self, lib, name, *args):
        if self._timed is not None:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            rc = getattr(lib, name)(*args)
            b.record()
            self._timed.append((name, a, b))
            if len(self._timed) >= self.PROFILE_FOLD:
                self._fold_profile()            # so that a long run holds a bounded number of events
        else:
            rc = getattr(lib, name)(*args)
        if rc != 0:
            raise KernelError(lib.tp_last_error().decode())

    PROFILE_FOLD = 4096                         # timed calls kept as events before they are summed

    def _fold_profile(self):
        """Sum the timed calls so far into the totals per entry point and let go of their events."""
        if not self._timed:
            return
        self._timed[-1][2].synchronize()
        for name, a, b in self._timed:
            ms, n = self._profile_totals.get(name, (0.0, 0))
            self._profile_totals[name] = (ms + a.elapsed_time(b), n + 1)
        self._timed = []

    def profile_report(self, file=None):
        """The time of the calls so far per entry point, most expensive first (TRAPETUM_AMD_PROFILE=1); forgets them."""
        import sys
        if self._timed is None:
            return
        self._fold_profile()
        total, self._profile_totals = self._profile_totals, {}
        if not total:
            return
        out = file or sys.stderr
        for name, (ms, n) in sorted(total.items(), key=lambda kv: -kv[1][0]):
            print(f"[profile] op={name} calls={n} total_ms={ms:.3f} mean_us={1e3 * ms / n:.2f}", file=out, flush=True)

    def _dev(self, *tensors):
        for t in tensors:
            if t is not None and t.device != self.device and not (t.device.type == "cuda" and t.device.index == (self.device.index or 0)):
                raise KernelError(f"tensor on {t.device}, the kernels run on {self.device}")

    @staticmethod
    def _rows(t, what):
        """2-D, unit stride along the row; returns the row stride in elements."""
        if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
            raise KernelError(f"{what}: expected rows with contiguous elements, found shape {tuple(t.shape)} strides {t.stride()}")
        return t.stride(0)

    def attn_lib(self, head_dim):
        if head_dim not in self._attn:
            try:
                lib = _c.CDLL(_build.build_attention(head_dim))
            except (OSError, _build.BuildError) as e:
                raise KernelError(f"the attention kernels for head_dim {head_dim} could not be built or loaded: {e}") from None
            _bind(lib, _ATTN_SIGS)
            self._attn[head_dim] = lib
        return self._attn[head_dim]

    # ---- weights layout ----------------------------------------------------------------------------
    def pack_gate_up(self, w_gate, w_up):
        """[2 * ceil16(I), K]: 16 rows of gate, the 16 rows of up of the same units, and so on; zero rows pad."""
        i, k = w_gate.shape
        ip = -(-i // GATE_GROUP) * GATE_GROUP
        out = torch.zeros((2, ip, k), dtype=w_gate.dtype, device=w_gate.device)
        out[0, :i] = w_gate
        out[1, :i] = w_up
        return out.reshape(2, ip // GATE_GROUP, GATE_GROUP, k).transpose(0, 1).reshape(2 * ip, k).contiguous()

    # ---- row-wise kernels ----------------------------------------------------------------------------
    def embed_rows(self, tokens, table, scale):
        self._dev(tokens, table)
        if tokens.dtype != torch.int32 or tokens.dim() != 1 or not tokens.is_contiguous():
            raise KernelError("embed_rows: tokens must be a contiguous int32 vector")
        if not table.is_contiguous() or table.dim() != 2:
            raise KernelError("embed_rows: the table must be a contiguous matrix")
        m, (v, d) = tokens.numel(), table.shape
        out = torch.empty((m, d), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_embed_rows", tokens.data_ptr(), table.data_ptr(), _code(table.dtype), float(scale),
                   out.data_ptr(), m, d, v, self._stream())
        return out

    def rms_norm(self, x, gain, eps, out_dtype):
        self._dev(x, gain)
        if not x.is_contiguous() or x.dim() != 2:
            raise KernelError("rms_norm: rows must be a contiguous matrix")
        m, d = x.shape
        if gain.dtype != torch.float32 or gain.numel() != d or not gain.is_contiguous():
            raise KernelError(f"rms_norm: gain must be float32 [{d}]")
        out = torch.empty((m, d), dtype=out_dtype, device=self.device)
        self._call(self.lib, "tp_rms_norm", x.data_ptr(), _code(x.dtype), gain.data_ptr(), float(eps), out.data_ptr(),
                   _code(out_dtype), m, d, self._stream())
        return out

    def add_rms_norm(self, stream, rows, gain_post, eps_post, gain_next, eps_next, out_dtype):
        """stream += post-norm(rows) (or rows); returns next-norm(stream) or None.  rows: a tensor or SplitRows."""
        m, d = stream.shape
        n_slices, stride = 1, 0
        if isinstance(rows, SplitRows) and d > self.MAX_SLICED_WIDTH:
            rows = self.rows(rows, out_dtype)            # the fused kernel keeps a row in registers: wider rows are added first
        if isinstance(rows, SplitRows):
            n_slices, stride = rows.slices.shape[0], rows.slices.stride(0)
            rows = rows.slices[0]
        self._dev(stream, rows, gain_post, gain_next)
        if stream.dtype != torch.float32 or not stream.is_contiguous():
            raise KernelError("add_rms_norm: the stream must be contiguous float32")
        if tuple(rows.shape) != (m, d) or not rows.is_contiguous():
            raise KernelError(f"add_rms_norm: rows {tuple(rows.shape)} do not match the stream {(m, d)}")
        for g in (gain_post, gain_next):
            if g is not None and (g.dtype != torch.float32 or g.numel() != d or not g.is_contiguous()):
                raise KernelError(f"add_rms_norm: gains must be float32 [{d}]")
        out = torch.empty((m, d), dtype=out_dtype, device=self.device) if gain_next is not None else None
        self._call(self.lib, "tp_add_rms_norm", stream.data_ptr(), rows.data_ptr(), _code(rows.dtype), n_slices, stride,
                   gain_post.data_ptr() if gain_post is not None else None, float(eps_post),
                   gain_next.data_ptr() if gain_next is not None else None, float(eps_next),
                   out.data_ptr() if out is not None else None, _code(out_dtype), m, d, self._stream())
        return out

    MAX_SLICED_WIDTH = 8192        # widest row `add_rms_norm` takes in K slices

    def rows(self, rows, dtype):
        """A tensor of `dtype` from what `linear` returned: K slices are added in slice order."""
        if not isinstance(rows, SplitRows):
            return rows
        sl = rows.slices
        self._dev(sl)
        if sl.dtype != torch.float32 or sl.dim() != 3 or not sl.is_contiguous():
            raise KernelError("rows: K slices must be contiguous float32 [slices, rows, columns]")
        out = torch.empty(sl.shape[1:], dtype=dtype, device=self.device)
        self._call(self.lib, "tp_sum_slices", sl.data_ptr(), sl.shape[0], sl.stride(0), out.data_ptr(), _code(dtype),
                   out.numel(), self._stream())
        return out

    def gather_rows(self, x, rows):
        self._dev(x, rows)
        if x.dtype != torch.float32 or not x.is_contiguous() or x.dim() != 2:
            raise KernelError("gather_rows: expected a contiguous float32 matrix")
        if rows.dtype != torch.int32 or not rows.is_contiguous():
            raise KernelError("gather_rows: row indices must be contiguous int32")
        out = torch.empty((rows.numel(), x.shape[1]), dtype=torch.float32, device=self.device)
        self._call(self.lib, "tp_gather_rows", x.data_ptr(), rows.data_ptr(), out.data_ptr(), rows.numel(),
                   x.shape[1], x.shape[0], self._stream())
        return out

    def rope_kv_write(self, q, k, v, H, KV, hd, inv_freq, rotary_dim, row_seq, row_pos, new_len, table,
                      k_pool, v_pool, rows_cap, pairing="halves", write=True):
        """Rotate q and k in place and write k, v into the cache.  write=False: rotate only (a step whose attention
        reads the cache as earlier steps left it caches its rows afterwards, with `kv_write`).
        pairing: one of ROPE_PAIRINGS, which elements of a head turn together."""
        if pairing not in ROPE_PAIRINGS:
            raise KernelError(f"rope_kv_write: pairing '{pairing}' has no kernel ({', '.join(ROPE_PAIRINGS)})")
        self._dev(q, k, v, inv_freq, row_seq, row_pos, new_len, table, k_pool, v_pool)
        m = q.shape[0]
        qs = self._rows(q, "rope_kv_write q")
        if q.shape[1] != H * hd:
            raise KernelError(f"rope_kv_write: q has {q.shape[1]} columns, {H} heads of {hd} need {H * hd}")
        if rotary_dim:
            if inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2:
                raise KernelError(f"rope_kv_write: a rotation over {rotary_dim} needs float32 inv_freq [{rotary_dim // 2}]")
        for t, n in ((row_seq, m), (row_pos, m)):
            if t.dtype != torch.int32 or t.numel() != n:
                raise KernelError("rope_kv_write: row_seq and row_pos must be int32, one entry per row")
        kp = vp = ks = vs = 0
        page = table_w = 1
        write = write and k is not None
        if k is not None:
            ks, vs = self._rows(k, "rope_kv_write k"), self._rows(v, "rope_kv_write v")
            if k.shape != (m, KV * hd) or v.shape != (m, KV * hd) or k.dtype != q.dtype or v.dtype != q.dtype:
                raise KernelError("rope_kv_write: k and v must be [rows, kv_heads * head_dim] of q's dtype")
            kp, vp = k.data_ptr(), v.data_ptr()
        if write:
            self._check_pools("rope_kv_write", q.dtype, new_len.numel(), KV, hd, new_len, table, k_pool, v_pool)
            page, table_w = k_pool.shape[2], table.shape[1]
        self._call(self.lib, "tp_rope_kv_write", q.data_ptr(), qs, kp or None, ks, vp or None, vs, _code(q.dtype), m, H, KV, hd,
                   inv_freq.data_ptr() if rotary_dim else None, rotary_dim, row_seq.data_ptr(), row_pos.data_ptr(),
                   new_len.data_ptr(), table.data_ptr() if write else None, table_w,
                   k_pool.data_ptr() if write else None, v_pool.data_ptr() if write else None,
                   page, rows_cap if write else 0, ROPE_PAIRINGS[pairing], self._stream())

    def kv_write(self, k, v, KV, hd, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap):
        """The step's keys (rotated already) and values into the cache: what `rope_kv_write(write=False)` left undone."""
        self._dev(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool)
        m = k.shape[0]
        ks, vs = self._rows(k, "kv_write k"), self._rows(v, "kv_write v")
        if k.shape != (m, KV * hd) or v.shape != (m, KV * hd) or k.dtype != v.dtype:
            raise KernelError("kv_write: k and v must be [rows, kv_heads * head_dim] of one dtype")
        for t in (row_seq, row_pos):
            if t.dtype != torch.int32 or t.numel() != m:
                raise KernelError("kv_write: row_seq and row_pos must be int32, one entry per row")
        self._check_pools("kv_write", k.dtype, new_len.numel(), KV, hd, new_len, table, k_pool, v_pool)
        self._call(self.lib, "tp_kv_write", k.data_ptr(), ks, v.data_ptr(), vs, _code(k.dtype), m, KV, hd, row_seq.data_ptr(),
                   row_pos.data_ptr(), new_len.data_ptr(), table.data_ptr(), table.shape[1], k_pool.data_ptr(),
                   v_pool.data_ptr(), k_pool.shape[2], rows_cap, self._stream())

    # ---- matrix products -----------------------------------------------------------------------------
    def _linear(self, x, w, out_dtype, epilogue, cap, units, defer=False, act=0):
        self._dev(x, w)
        if x.dim() != 2 or w.dim() != 2 or not x.is_contiguous() or not w.is_contiguous():
            raise KernelError("linear: rows and matrix must be contiguous 2-D tensors")
        if x.dtype != w.dtype:
            raise KernelError(f"linear: rows are {x.dtype}, the matrix is {w.dtype}")
        m, k = x.shape
        n = w.shape[0]
        if w.shape[1] != k:
            raise KernelError(f"linear: rows have {k} columns, the matrix {w.shape[1]}")
        cols = units if epilogue == EPI_GATED else n
        algo = self.force_linear
        nbytes = self.lib.tp_linear_workspace_bytes(_code(x.dtype), _code(out_dtype), m, n, k, epilogue, units,
                                                    1 if defer else 0, algo)
        if defer and epilogue == EPI_NONE and nbytes and nbytes % (m * n * 4) == 0 and nbytes // (m * n * 4) > 1:
            slices = torch.empty((nbytes // (m * n * 4), m, n), dtype=torch.float32, device=self.device)
            self._call(self.lib, "tp_linear", x.data_ptr(), w.data_ptr(), None, _code(x.dtype), _code(out_dtype),
                       m, n, k, epilogue, float(cap), units, act, slices.data_ptr(), nbytes, 1, algo, self._stream())
            return SplitRows(slices)
        out = torch.empty((m, cols), dtype=out_dtype, device=self.device)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device) if nbytes else None
        self._call(self.lib, "tp_linear", x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(x.dtype), _code(out_dtype),
                   m, n, k, epilogue, float(cap), units, act, ws.data_ptr() if ws is not None else None, nbytes, 0, algo,
                   self._stream())
        return out

    def linear(self, x, w, out_dtype, softcap=None, defer=False, bias=None):
        """x @ w^T (+ bias).  defer: the caller hands the result to `add_rms_norm` (or through `rows()`), so a product
        computed in K slices may come back as SplitRows.  bias: float32 [rows of w], added by a kernel of its own
        (the products have no bias operand), so a product with a bias is never left in slices."""
        if bias is not None:
            if softcap:
                raise KernelError("linear: a bias and a cap together have no kernel")
            y = self._linear(x, w, out_dtype, EPI_NONE, 0.0, 0)
            self._dev(bias)
            if bias.dtype != torch.float32 or bias.numel() != y.shape[1] or not bias.is_contiguous():
                raise KernelError(f"linear: the bias must be contiguous float32 [{y.shape[1]}]")
            self._call(self.lib, "tp_add_bias", y.data_ptr(), _code(y.dtype), bias.data_ptr(), y.shape[0], y.shape[1], self._stream())
            return y
        if softcap:
            return self._linear(x, w, out_dtype, EPI_SOFTCAP, softcap, 0)
        return self._linear(x, w, out_dtype, EPI_NONE, 0.0, 0, defer=defer)

    def gated_linear(self, x, w_packed, inter, activation, out_dtype):
        """act(x @ gate^T) * (x @ up^T) over the packed matrix of `pack_gate_up`; activation: one of GATE_ACTIVATIONS."""
        if activation not in GATE_ACTIVATIONS:
            raise KernelError(f"gated_linear: activation '{activation}' has no kernel ({', '.join(GATE_ACTIVATIONS)})")
        return self._linear(x, w_packed, out_dtype, EPI_GATED, 0.0, inter, act=GATE_ACTIVATIONS[activation])

    # ---- attention -------------------------------------------------------------------------------------
    def _fast_attention(self, dtype, H, KV, hd):
        return not self.force_plain_attention and dtype == torch.bfloat16 and hd % 16 == 0 and hd <= 256 and H // KV <= 16

    def attention_prefill(self, q, k, v, H, KV, hd, cu_rows, max_count, scale, softcap, window, out_dtype,
                          row_seq=None, row_pos=None, cached=None, shape=0):
        """Causal attention of the step's queries over the step's own rows of keys and values and, with
        `cached` = (new_len, table, k_pool, v_pool, rows_cap), over the positions before them, read in place from the
        cache as earlier steps left it (the step's own rows are not looked for there).  Without `cached` every sequence
        starts at position 0; with it row_pos holds absolute positions, sequence s's first row standing at
        new_len[s] - its count.  shape: the matrix-core kernel's block shape (0: chosen by the size of the step)."""
        self._dev(q, k, v, cu_rows)
        m = q.shape[0]
        qs, ks, vs = self._rows(q, "attention q"), self._rows(k, "attention k"), self._rows(v, "attention v")
        if q.shape[1] != H * hd or k.shape != (m, KV * hd) or v.shape != (m, KV * hd):
            raise KernelError("attention_prefill: q must be [rows, heads * head_dim], k and v [rows, kv_heads * head_dim]")
        if not (q.dtype == k.dtype == v.dtype == out_dtype):
            raise KernelError("attention_prefill: q, k, v and the output share one dtype")
        n_seq = cu_rows.numel() - 1
        new_len = table = k_pool = v_pool = None
        page, rows_cap, table_w = 1, 0, 1
        if cached is not None:
            new_len, table, k_pool, v_pool, rows_cap = cached
            self._dev(new_len, table, k_pool, v_pool)
            self._check_pools("attention_prefill", q.dtype, n_seq, KV, hd, new_len, table, k_pool, v_pool)
            page, table_w, rows_cap = k_pool.shape[2], table.shape[1], rows_cap or 0
        ptr = lambda t: t.data_ptr() if t is not None else None
        out = torch.empty((m, H * hd), dtype=out_dtype, device=self.device)
        if self._fast_attention(q.dtype, H, KV, hd) and (cached is None or (page >= 16 and page & (page - 1) == 0)):
            lib = self.attn_lib(hd)
            self._call(lib, "tp_attn_prefill", q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs,
                       m, H, KV, cu_rows.data_ptr(), n_seq, int(max_count), ptr(new_len), ptr(table), table_w,
                       ptr(k_pool), ptr(v_pool), page, rows_cap,
                       float(scale), float(softcap), int(window), out.data_ptr(), int(shape), self._stream())
            return out
        if cached is not None and (row_seq is None or row_pos is None):
            raise KernelError("attention_prefill: cached positions need every row's sequence and position")
        if row_seq is None:
            counts = (cu_rows[1:] - cu_rows[:-1]).long()
            row_seq = torch.repeat_interleave(torch.arange(n_seq, device=self.device, dtype=torch.int32), counts)
            row_pos = (torch.arange(m, device=self.device, dtype=torch.int32) - cu_rows[:-1][row_seq.long()]).to(torch.int32)
        self._call(self.lib, "tp_attn_simple_prefill", q.data_ptr(), qs, k.data_ptr(), ks, v.data_ptr(), vs, _code(q.dtype),
                   m, H, KV, hd, cu_rows.data_ptr(), row_seq.data_ptr(), row_pos.data_ptr(), ptr(new_len), ptr(table), table_w,
                   ptr(k_pool), ptr(v_pool), page, rows_cap, float(scale), float(softcap),
                   int(window), out.data_ptr(), self._stream())
        return out

    @staticmethod
    def decode_splits(n, KV, hd, keys):
        """Slices of the keys per (sequence, kv head) in a decode step: enough blocks to keep every CU streaming
        (about 1536; 768 when the pairs alone are many), each with at least one round of 64 keys.  Measured on
        MI355X from 1 to 64 sequences and 500 to 8000 keys this is within 7 % of the best count everywhere; more
        slices cost little (a second launch adds them), fewer cost up to half."""
        pairs = n * KV
        want = -(-(1536 if pairs < 192 else 768) // pairs)
        return max(1, min(want, -(-keys // 64), 128))

    def _check_pools(self, what, dtype, n, KV, hd, new_len, table, k_pool, v_pool):
        if new_len.numel() != n or new_len.dtype != torch.int32:
            raise KernelError(f"{what}: one int32 length per sequence")
        if k_pool.dtype != dtype or k_pool.dim() != 4 or tuple(k_pool.shape[1:]) != (KV, k_pool.shape[2], hd) \
                or v_pool.shape != k_pool.shape or not k_pool.is_contiguous() or not v_pool.is_contiguous():
            raise KernelError(f"{what}: cache pools must be contiguous [pages, kv_heads, page, head_dim] of {dtype}")
        if table.dtype != torch.int32 or table.dim() != 2 or table.shape[0] != n or not table.is_contiguous():
            raise KernelError(f"{what}: the page table must be contiguous int32 [sequences, pages]")

    def attention_decode(self, q, H, KV, hd, new_len, table, k_pool, v_pool, rows_cap, scale, softcap, window,
                         out_dtype, max_keys=None, splits=None):
        self._dev(q, new_len, table, k_pool, v_pool)
        n = q.shape[0]
        qs = self._rows(q, "attention q")
        if q.shape[1] != H * hd:
            raise KernelError("attention_decode: q must be [sequences, heads * head_dim]")
        self._check_pools("attention_decode", q.dtype, n, KV, hd, new_len, table, k_pool, v_pool)
        out = torch.empty((n, H * hd), dtype=out_dtype, device=self.device)
        page = k_pool.shape[2]
        if self._fast_attention(q.dtype, H, KV, hd) and page >= 16 and page & (page - 1) == 0:
            lib = self.attn_lib(hd)
            keys = int(max_keys) if max_keys else k_pool.shape[0] * k_pool.shape[2]
            nsplit = int(splits) if splits else self.decode_splits(n, KV, hd, keys)
            floats = lib.tp_attn_decode_workspace_floats(n, H, nsplit)
            ws = torch.empty(floats, dtype=torch.float32, device=self.device) if floats else None
            self._call(lib, "tp_attn_decode", q.data_ptr(), qs, n, H, KV, new_len.data_ptr(), table.data_ptr(),
                       table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[2], rows_cap, float(scale),
                       float(softcap), int(window), out.data_ptr(), ws.data_ptr() if ws is not None else None, nsplit,
                       self._stream())
            return out
        self._call(self.lib, "tp_attn_simple_decode", q.data_ptr(), qs, _code(q.dtype), n, H, KV, hd, new_len.data_ptr(),
                   table.data_ptr(), table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(), k_pool.shape[2], rows_cap,
                   float(scale), float(softcap), int(window), out.data_ptr(), self._stream())
        return out

    def fuses_decode_step(self, dtype, H, KV, hd, k_pool):
        """Whether `attention_decode_step` exists for this geometry: the caller then skips `rope_kv_write`."""
        page = k_pool.shape[2]
        return self._fast_attention(dtype, H, KV, hd) and page >= 16 and page & (page - 1) == 0

    def attention_decode_step(self, qkv, H, KV, hd, inv_freq, rotary_dim, new_len, table, k_pool, v_pool, rows_cap,
                              scale, softcap, window, out_dtype, max_keys=None, write_kv=True, splits=None):
        """A decode step's rotation, cache write and attention in one launch.  qkv: each sequence's projections
        [queries | keys | values] (queries only when write_kv is false), a bf16 tensor or what
        `linear(..., defer=True)` returned; sequence i's token has position new_len[i] - 1."""
        split = isinstance(qkv, SplitRows)
        rows = qkv.slices if split else qkv
        self._dev(rows, inv_freq, new_len, table, k_pool, v_pool)
        n, width = rows.shape[-2], rows.shape[-1]
        if width != (H + (2 * KV if write_kv else 0)) * hd:
            raise KernelError(f"attention_decode_step: rows of {width} columns, {H} heads and {KV} kv heads of {hd} need "
                              f"{(H + (2 * KV if write_kv else 0)) * hd}")
        if out_dtype != torch.bfloat16 or not self.fuses_decode_step(out_dtype, H, KV, hd, k_pool):
            raise KernelError("attention_decode_step: no fused kernel for this geometry (see fuses_decode_step)")
        if split:
            if rows.dtype != torch.float32 or not rows.is_contiguous():
                raise KernelError("attention_decode_step: K slices must be contiguous float32")
            n_slices, slice_stride, row_stride = rows.shape[0], rows.shape[1] * rows.shape[2], rows.shape[2]
        else:
            if rows.dim() != 2 or rows.dtype not in (torch.bfloat16, torch.float32):
                raise KernelError("attention_decode_step: projections must be 2-D, bfloat16 or float32")
            n_slices, slice_stride, row_stride = 1, 0, self._rows(rows, "attention_decode_step qkv")
        if rotary_dim and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rotary_dim // 2):
            raise KernelError(f"attention_decode_step: a rotation over {rotary_dim} needs float32 inv_freq [{rotary_dim // 2}]")
        self._check_pools("attention_decode_step", torch.bfloat16, n, KV, hd, new_len, table, k_pool, v_pool)
        lib = self.attn_lib(hd)
        keys = int(max_keys) if max_keys else k_pool.shape[0] * k_pool.shape[2]
        nsplit = int(splits) if splits else self.decode_splits(n, KV, hd, keys)
        floats = lib.tp_attn_decode_workspace_floats(n, H, nsplit)
        ws = torch.empty(floats, dtype=torch.float32, device=self.device) if floats else None
        out = torch.empty((n, H * hd), dtype=out_dtype, device=self.device)
        self._call(lib, "tp_attn_decode_fused", rows.data_ptr(), _code(rows.dtype), n_slices, slice_stride, row_stride,
                   inv_freq.data_ptr() if rotary_dim else None, int(rotary_dim), 1 if write_kv else 0,
                   n, H, KV, new_len.data_ptr(), table.data_ptr(), table.shape[1], k_pool.data_ptr(), v_pool.data_ptr(),
                   k_pool.shape[2], rows_cap, float(scale), float(softcap), int(window), out.data_ptr(),
                   ws.data_ptr() if ws is not None else None, nsplit, self._stream())
        return out

    # ---- token choice -------------------------------------------------------------------------------------
    def argmax(self, logits, out=None):
        """Smallest index of the largest value per row, int32; into `out` if given."""
        self._dev(logits)
        if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
            raise KernelError("argmax: logits must be contiguous float32 [rows, vocab]")
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        else:
            self._dev(out)
            if out.dtype != torch.int32 or out.shape != (logits.shape[0],) or not out.is_contiguous():
                raise KernelError("argmax: the output must be contiguous int32 [rows]")
        nbytes = self.lib.tp_argmax_workspace_bytes(logits.shape[0], logits.shape[1])
        ws = torch.empty(nbytes, dtype=torch.uint8, device=self.device) if nbytes else None
        self._call(self.lib, "tp_argmax", logits.data_ptr(), logits.shape[0], logits.shape[1], out.data_ptr(),
                   ws.data_ptr() if ws is not None else None, self._stream())
        return out

    def apply_repetition_penalty(self, logits, recent, penalty):
        """In place.  recent: int32 [rows, R], -1 where empty."""
        self._dev(logits, recent)
        if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
            raise KernelError("repetition_penalty: logits must be contiguous float32 [rows, vocab]")
        if recent.dtype != torch.int32 or recent.dim() != 2 or recent.shape[0] != logits.shape[0] or not recent.is_contiguous():
            raise KernelError("repetition_penalty: recent tokens must be contiguous int32 [rows, R]")
        self._call(self.lib, "tp_repetition_penalty", logits.data_ptr(), logits.shape[0], logits.shape[1],
                   recent.data_ptr(), recent.shape[1], float(penalty), self._stream())

    def recent_push(self, tokens, recent, cursor):
        """Row i's token goes into row i of the ring `recent` (int32 [rows, R]) at cursor[i], which moves on by one."""
        self._dev(tokens, recent, cursor)
        n = tokens.numel()
        if tokens.dtype != torch.int32 or not tokens.is_contiguous() or cursor.dtype != torch.int32 or cursor.numel() != n \
                or not cursor.is_contiguous():
            raise KernelError("recent_push: tokens and cursors must be contiguous int32 of one length")
        if recent.dtype != torch.int32 or recent.dim() != 2 or recent.shape[0] != n or not recent.is_contiguous():
            raise KernelError("recent_push: the ring must be contiguous int32 [rows, R]")
        self._call(self.lib, "tp_recent_push", tokens.data_ptr(), recent.data_ptr(), cursor.data_ptr(), n, recent.shape[1],
                   self._stream())

    def sample(self, logits, temperature, top_k, top_p, uniforms, out=None):
        self._dev(logits, uniforms)
        if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
            raise KernelError("sample: logits must be contiguous float32 [rows, vocab]")
        if uniforms.dtype != torch.float32 or uniforms.numel() != logits.shape[0] or not uniforms.is_contiguous():
            raise KernelError("sample: one float32 uniform number per row")
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=self.device)
        else:
            self._dev(out)
            if out.dtype != torch.int32 or out.shape != (logits.shape[0],) or not out.is_contiguous():
                raise KernelError("sample: the output must be contiguous int32 [rows]")
        # the candidate filter's workspace starts zeroed and every call leaves it zeroed again: kept between calls
        shape = tuple(logits.shape)
        if shape not in self._sample_ws:
            nbytes = self.lib.tp_sample_workspace_bytes(shape[0], shape[1])
            self._sample_ws[shape] = torch.zeros(nbytes, dtype=torch.uint8, device=self.device) if nbytes else None
        ws = self._sample_ws[shape]
        self._call(self.lib, "tp_sample", logits.data_ptr(), shape[0], shape[1], float(temperature),
                   int(top_k), float(top_p), uniforms.data_ptr(), out.data_ptr(), ws.data_ptr() if ws is not None else None,
                   self._stream())
        return out

    # ---- probes: what the GPU gives a kernel at best -----------------------------------------------------------
    def _best_ms(self, launch, repeats):
        launch()
        torch.cuda.synchronize(self.device)
        best = float("inf")
        for _ in range(repeats):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            launch()
            b.record()
            b.synchronize()
            best = min(best, a.elapsed_time(b))
        return best

    def measured_ceilings(self, stream_bytes=4 << 30, repeats=5):
        """(GB/s of a streaming read of device memory, flop/s of a loop of bf16 matrix instructions), each the best
        of a few runs of a probe kernel."""
        cus = torch.cuda.get_device_properties(self.device).multi_processor_count
        sink = torch.zeros(4, dtype=torch.float32, device=self.device)
        buf = torch.empty(stream_bytes, dtype=torch.uint8, device=self.device).fill_(1)
        ms = self._best_ms(lambda: self._call(self.lib, "tp_probe_stream", buf.data_ptr(), stream_bytes, sink.data_ptr(),
                                              cus * 32, self._stream()), repeats)
        gbs = stream_bytes / (ms * 1e-3) / 1e9
        del buf
        best, mhz = 0.0, 0.0
        clocks = torch.zeros(2, dtype=torch.int64, device=self.device)
        for kind in (0, 1):                            # the 16x16x32 and the 32x32x16 form of the instruction
            iters, blocks = 20000, cus * 8
            ms = self._best_ms(lambda: self._call(self.lib, "tp_probe_mfma", kind, iters, blocks, sink.data_ptr(),
                                                  clocks.data_ptr(), self._stream()), repeats)
            flops = blocks * 4 * iters * 131072.0 / (ms * 1e-3)
            if flops > best:
                c = clocks.tolist()
                best, mhz = flops, (100.0 * c[0] / c[1] if c[1] else 0.0)
        self.matrix_clock_mhz = mhz                    # the shader clock while the matrix loop ran
        return gbs, best
