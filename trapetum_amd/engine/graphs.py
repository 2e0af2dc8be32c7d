"""Decode steps replayed from captured HIP graphs.

A decode step is some three hundred small launches; replaying them from a graph removes the host's share of
the step (the reference reports the same lever for its own loop: runtime/README.md:49-58, and wraps capture
and replay in `Graph`, runtime/src/lib.rs:1211-1236).  A graph is captured for a batch size out of a few (powers
of two), for a bound on the lengths of its sequences (1024, 2048, ...: launch geometry that depends on lengths,
the slices of the decode attention, is sized for the bound) and for one way of choosing the next tokens (none,
argmax, or sampling with given constants), which is part of the graph: it leaves the chosen ids where its next
replay reads its tokens, so a generation loop needs neither a launch nor a copy between replays.  A batch of
fewer sequences than the graph has rows fills the rest with rows that stand for no sequence: they read and write
the cache's spare page and spare slot.  What changes from step to step (slots, positions, lengths, page tables,
the sampler's uniform numbers) lives at fixed device addresses, shared by the graphs of one batch size, that are
refilled by one copy before each replay; page tables have the cache's widest width.  The recent tokens that a
repetition penalty looks at are a ring per row on the device, which the graph itself extends by the id it chose.  No memset node is
recorded: buffers are filled by copies and kernels.  The least recently used graphs are dropped beyond
`max_graphs`.
"""
import collections

import numpy as np
import torch

from ..sampling.sampler import RECENT_WINDOW
from .batch import StaticStep, StepContext, step_arrays


def graph_rows(n):
    """Rows of the graph that serves a batch of n sequences: the next power of two."""
    nb = 1
    while nb < n:
        nb *= 2
    return nb


def length_bound(longest, max_context):
    bound = 1024
    while bound < longest:
        bound *= 2
    return min(bound, max_context)


class _Rows:
    """Fixed memory of one batch size: the step's geometry and uniform numbers, and the tokens."""

    def __init__(self, rt, cache, nb):
        self.nb = nb
        self.static = StaticStep(rt, cache, nb, extra=nb)
        self.tokens = torch.zeros(nb, dtype=torch.int32, device=rt.device)
        self.uniforms = self.static.extra_view().view(torch.float32)
        self.recent = torch.full((nb, RECENT_WINDOW), -1, dtype=torch.int32, device=rt.device)     # rings of chosen and prompt ids
        self.cursor = torch.zeros(nb, dtype=torch.int32, device=rt.device)                      # where a row's next id goes


class _Captured:
    def __init__(self, graph, ctx, logits):
        self.graph, self.ctx, self.logits = graph, ctx, logits


class GraphedDecode:
    def __init__(self, model, cache, max_graphs=16):
        if model.rt.device.type != "cuda":
            raise RuntimeError("HIP graphs need the GPU")
        self.model = model
        self.cache = cache
        self.max_graphs = max_graphs
        self.rows_of = {}                                   # batch size of a graph -> _Rows
        self.graphs = collections.OrderedDict()             # (rows, length bound, choice) -> _Captured
        self.captures = 0

    def rows(self, nb):
        if nb not in self.rows_of:
            self.rows_of[nb] = _Rows(self.model.rt, self.cache, nb)
        return self.rows_of[nb]

    def _choose(self, choice, logits, rows):
        """choice: None, ("greedy",) or ("sample", temperature, top_k, top_p), either followed by ("penalty", value):
        then the logits of the rows' recent tokens are changed first.  The ids go where the tokens lie, and into the
        rows' rings."""
        if choice is None:
            return
        ops = self.model.rt.ops
        penalty = choice[-1][1] if isinstance(choice[-1], tuple) else None
        if penalty is not None:
            ops.apply_repetition_penalty(logits, rows.recent, penalty)
        if choice[0] == "greedy":
            ops.argmax(logits, out=rows.tokens)
        else:
            ops.sample(logits, choice[1], choice[2], choice[3], rows.uniforms, out=rows.tokens)
        if penalty is not None:
            ops.recent_push(rows.tokens, rows.recent, rows.cursor)

    def run(self, nb, slots, starts, choice=None, uniforms=None):
        """One decode step of `nb` rows (nb a size `graph_rows` gives): row i continues the sequence in slots[i], which
        holds starts[i] tokens and has room for one more (the caller has grown it), or stands for no sequence
        (the cache's spare slot, start 0).  The rows' tokens are `self.rows(nb).tokens`; afterwards that tensor
        holds the chosen ids if a choice is asked for.  Returns the logits fp32 [nb, vocab] in memory that the next
        step of this graph overwrites."""
        model, cache = self.model, self.cache
        rows = self.rows(nb)
        if len(slots) != nb:
            raise ValueError(f"a graph of {nb} rows was given {len(slots)} slots")
        counts, want = [1] * nb, list(range(nb))
        flat, _ = step_arrays(cache, slots, counts, starts, want, rows.static.table_widths)
        extra = None
        if uniforms is not None:
            extra = np.asarray(uniforms, dtype=np.float32).view(np.int32)
        rows.static.fill(flat, extra)
        key = (nb, length_bound(max(starts) + 1, cache.max_context), choice)
        cap = self.graphs.get(key)
        if cap is not None:
            self.graphs.move_to_end(key)
            cap.graph.replay()
            return cap.logits
        ctx = StepContext(model.rt, cache, slots, counts, starts, want, static=rows.static, length_bound=key[1])
        logits = model.run(ctx, rows.tokens)                # this step, eagerly; also loads what capture must not
        self._choose(choice, logits, rows)
        torch.cuda.synchronize(model.rt.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):                       # records the launches and runs none of them
            captured_logits = model.run(ctx, rows.tokens)
            self._choose(choice, captured_logits, rows)
        self.graphs[key] = _Captured(graph, ctx, captured_logits)
        self.captures += 1
        while len(self.graphs) > self.max_graphs:
            self.graphs.popitem(last=False)
        return logits

    def step(self, slots, tokens):
        """One decode step of the sequences in `slots` (a token each) without a choice of tokens; returns fp32 logits
        [len(slots), vocab] in memory that the next step overwrites.  The batch is padded to a graph's rows."""
        model, cache = self.model, self.cache
        counts, starts, want, tok = model.prepare(cache, slots, tokens)
        if any(c != 1 for c in counts):
            raise ValueError("graphed steps take one token per sequence")
        n, nb = len(slots), graph_rows(len(slots))
        rows = self.rows(nb)
        rows.tokens[:n].copy_(tok)
        pad = nb - n
        logits = self.run(nb, list(slots) + [cache.spare_slot] * pad, list(starts) + [0] * pad)
        return logits[:n]
