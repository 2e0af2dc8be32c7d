"""The geometry of one step: which rows belong to which sequence at which position.

A step runs M rows packed without padding: sequence i brings counts[i] tokens at
positions start[i] .. start[i] + counts[i] - 1, start[i] being what the cache holds
of it.  Any mix is a step: sequences that start, sequences that go on by one token,
sequences that go on by several.  The engine names three shapes so that parts can
pick their kernels: "decode" (every sequence brings one token), "prefill" (every
sequence starts at its first token) and "extend" (anything else: a mixer then sees
the cached positions before `start` as well as the step's own rows).  The
reference's step is one token of one sequence (runtime/src/lib.rs:4553); its
multi-token step takes M consecutive positions of one sequence from any position
(runtime/src/lib.rs:845-869).
"""
import numpy as np


class StepError(ValueError):
    """The step's shape is not one the engine runs."""


def classify(counts, starts):
    if not counts:
        raise StepError("a step needs at least one sequence")
    if any(c <= 0 for c in counts):
        raise StepError(f"every sequence of a step brings at least one token, found counts {list(counts)}")
    if all(c == 1 for c in counts):
        return "decode"
    if all(s == 0 for s in starts):
        return "prefill"
    return "extend"


def step_arrays(cache, slots, counts, starts, want_rows, table_widths=None):
    """The step's geometry as int32 arrays, in the order StepContext slices them."""
    n, m = len(slots), int(sum(counts))
    cu = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(counts, out=cu[1:])
    row_seq = np.repeat(np.arange(n), counts)
    row_pos = np.concatenate([np.arange(s, s + c) for s, c in zip(starts, counts)])
    new_len = np.asarray(starts) + np.asarray(counts)
    want = np.asarray(want_rows, dtype=np.int64)
    if want.size and (want.min() < 0 or want.max() >= m):
        raise StepError(f"wanted rows {list(want_rows)} reach outside the step's {m} rows")
    parts = [np.asarray(slots), cu, row_seq, row_pos, new_len, want]
    shapes = []
    for gi in range(len(cache.token_groups)):
        t = cache.page_table(gi, slots, None if table_widths is None else table_widths[gi])
        shapes.append(t.shape)
        parts.append(t.reshape(-1))
    flat = np.concatenate([np.asarray(p, dtype=np.int32).reshape(-1) for p in parts])
    return flat, shapes


class StaticStep:
    """Fixed device memory for the geometry of decode steps of one batch size, so that a captured HIP graph
    finds every step's numbers at the same addresses.  Page tables have the cache's widest width.  `extra` more
    int32 follow the geometry for what else changes with the step (a sampler's uniform numbers, as bit patterns)."""

    RING = 8

    def __init__(self, rt, cache, n_seq, extra=0):
        import torch
        self.rt = rt
        self.n_seq = n_seq
        self.table_widths = [g.max_pages_per_seq for g in cache.token_groups]
        self.geometry = 6 * n_seq + 1 + sum(n_seq * w for w in self.table_widths)
        self.size = self.geometry + extra
        self.device_buffer = torch.zeros(self.size, dtype=torch.int32, device=rt.device)
        self.pinned = [torch.zeros(self.size, dtype=torch.int32, pin_memory=True) for _ in range(self.RING)]
        self.events = [None] * self.RING
        self.turn = 0

    def extra_view(self):
        return self.device_buffer[self.geometry:]

    def fill(self, flat, extra=None):
        """Queue the copy of this step's numbers into the fixed buffer (on the current stream)."""
        import torch
        assert flat.size == self.geometry, (flat.size, self.geometry)
        i = self.turn
        self.turn = (i + 1) % self.RING
        if self.events[i] is not None:
            self.events[i].synchronize()
        self.pinned[i][:self.geometry].copy_(torch.from_numpy(flat))
        if extra is not None:
            assert extra.size == self.size - self.geometry
            self.pinned[i][self.geometry:].copy_(torch.from_numpy(extra))
        self.device_buffer.copy_(self.pinned[i], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.events[i] = ev


class StepContext:
    """Everything parts need during a step.  Device tensors are int32."""

    def __init__(self, rt, cache, slots, counts, starts, want_rows, static=None, length_bound=None):
        """static: a StaticStep that the caller has filled with this step's numbers (a step captured in a graph reads
        them there); length_bound: the longest sequence the captured launches must serve."""
        self.rt = rt
        self.ops = rt.ops
        self.dtype = rt.dtype
        self.cache = cache
        self.slots = list(slots)
        self.counts = list(counts)
        self.starts = list(starts)
        self.mode = classify(self.counts, self.starts)
        self.n_seq = len(self.slots)
        self.n_rows = int(sum(self.counts))
        self.max_count = max(self.counts)
        self.entry = None               # schedule entry now running
        self.cache_owner = None         # entry whose cache it uses
        self.static = static
        self.length_bound = length_bound
        self._shared = set()            # entries whose cache a later entry reads
        self._step_rows = {}
        n, m = self.n_seq, self.n_rows
        self._after_step = []           # work put off until every entry of the step has run
        flat, shapes = step_arrays(cache, self.slots, self.counts, self.starts, want_rows,
                                   static.table_widths if static is not None else None)
        if static is not None:
            dev = static.device_buffer
        else:
            dev = rt.upload_i32(flat)
        o = 0

        def take(k):
            nonlocal o
            t = dev[o:o + k]
            o += k
            return t
        self.slot_ids = take(n)
        self.cu_rows = take(n + 1)
        self.row_seq = take(m)
        self.row_pos = take(m)
        self.new_len = take(n)
        self.n_want = len(want_rows)
        self.identity_want = list(want_rows) == list(range(m))
        self.want_rows = take(self.n_want)
        self._tables = [take(int(np.prod(sh))).reshape(sh) for sh in shapes]

    def page_table(self, group_index):
        return self._tables[group_index]

    def dump(self, stage, x):
        """With TRAPETUM_AMD_DEBUG_DUMP=1: one line of statistics of `x` (rows of the step at this stage of the running
        schedule entry) on stderr; nothing otherwise."""
        from .. import flags
        if not flags.debug_dump() or x is None:
            return
        import sys
        t = self.ops.rows(x, x.dtype).double()
        print(f"[ldump] L={-1 if self.entry is None else self.entry} stage={stage} l2={float(t.norm()):.6e} "
              f"absmax={float(t.abs().max()):.6e} mean={float(t.mean()):.6e}", file=sys.stderr, flush=True)

    def max_rows_visible(self, site):
        """Most cached rows any sequence of this step can see at this cache site (a host number, for launch geometry).
        With fixed step memory (a captured graph) it is the graph's bound on the lengths."""
        longest = max(s + c for s, c in zip(self.starts, self.counts))
        if self.length_bound is not None:
            longest = max(longest, self.length_bound)
        return min(longest, site.rows_cap) if site.rows_cap else longest

    # what the running entry is about to cache of this step's rows, for the entries that read its cache in this step
    def mark_shared(self, entries):
        self._shared = set(entries)

    def offer_step_rows(self, **tensors):
        """tensors: this step's own rows of the running entry's per-token tensors, by name."""
        if self.entry in self._shared:
            self._step_rows[self.entry] = tensors

    def step_rows_of(self, entry):
        return self._step_rows[entry]

    def after_readers(self, work):
        """Run `work()` once nobody in this step reads the running entry's cache as earlier steps left it any more:
        at once, or at the end of the step when later entries read this entry's cache."""
        if self.entry in self._shared:
            self._after_step.append(work)
        else:
            work()

    def finish(self):
        """What was put off until the end of the step."""
        for work in self._after_step:
            work()
        self._after_step = []
