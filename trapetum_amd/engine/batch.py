"""The geometry of one step: which rows belong to which sequence at which position.

A step runs M rows packed without padding: sequence i brings counts[i] tokens at
positions start[i] .. start[i] + counts[i] - 1.  Either every sequence starts
(start 0, whole prompts: "prefill") or every sequence goes on by one token
("decode").  The reference's step is one token of one sequence
(runtime/src/lib.rs:4553); its only multi-token step takes consecutive positions
of one sequence (runtime/src/lib.rs:845-869).
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
    raise StepError(
        "a step either starts every sequence at its first token or continues every sequence by one token; "
        f"found counts {list(counts)} at lengths {list(starts)}")


class StepContext:
    """Everything parts need during a step.  Device tensors are int32."""

    def __init__(self, rt, cache, slots, counts, starts, want_rows):
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
        self._shared = set()            # entries whose step keys/values a later entry reads
        self._step_kv = {}
        n, m = self.n_seq, self.n_rows
        cu = np.zeros(n + 1, dtype=np.int64)
        np.cumsum(self.counts, out=cu[1:])
        row_seq = np.repeat(np.arange(n), self.counts)
        row_pos = np.concatenate([np.arange(s, s + c) for s, c in zip(self.starts, self.counts)])
        new_len = np.asarray(self.starts) + np.asarray(self.counts)
        want = np.asarray(want_rows, dtype=np.int64)
        if want.size and (want.min() < 0 or want.max() >= m):
            raise StepError(f"wanted rows {want_rows} reach outside the step's {m} rows")
        parts = [np.asarray(self.slots), cu, row_seq, row_pos, new_len, want]
        tables = []
        for gi, g in enumerate(cache.kv_groups):
            tables.append(cache.page_table(gi, self.slots))
            parts.append(tables[-1].reshape(-1))
        flat = np.concatenate([np.asarray(p, dtype=np.int32).reshape(-1) for p in parts])
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
        self.want_rows = take(want.size)
        self.n_want = int(want.size)
        self._tables = [take(t.size).reshape(t.shape) for t in tables]

    def page_table(self, group_index):
        return self._tables[group_index]

    def max_keys(self, site):
        """Most keys any sequence of this step can see at this cache site (a host number, for launch geometry)."""
        longest = max(s + c for s, c in zip(self.starts, self.counts))
        return min(longest, site.rows_cap) if site.rows_cap else longest

    # keys and values of this step, for entries that read another entry's cache during a prefill
    def mark_shared(self, entries):
        self._shared = set(entries)

    def offer_step_kv(self, k, v):
        if self.entry in self._shared:
            self._step_kv[self.entry] = (k, v)

    def step_kv_of(self, entry):
        return self._step_kv[entry]
