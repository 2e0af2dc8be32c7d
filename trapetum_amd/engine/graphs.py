"""Decode steps replayed from captured HIP graphs, one graph per batch size and bound on the lengths.

A decode step is some three hundred small launches; replaying them from a graph removes the host's share of
the step (the reference reports the same lever for its own loop: runtime/README.md:49-58, and wraps capture
and replay in `Graph`, runtime/src/lib.rs:1211-1236).  What changes from step to step (slots, positions,
lengths, page tables, tokens) lives at fixed device addresses that are refilled before each replay; page
tables have the cache's widest width, and launch geometry that depends on lengths (the slices of the decode
attention) is sized for the graph's bound on the lengths.  No memset node is recorded: buffers are filled by
copies and kernels.
"""
import torch

from .batch import StaticStep, StepContext, step_arrays


class _Captured:
    def __init__(self, static, tokens, ctx, graph, logits):
        self.static, self.tokens, self.ctx, self.graph, self.logits = static, tokens, ctx, graph, logits


class GraphedDecode:
    def __init__(self, model, cache, greedy=False):
        """greedy: the graph also picks every sequence's next token (argmax) and leaves it where the next replay
        reads its tokens, so that a greedy loop needs neither a launch nor a copy between replays; `chosen` is that
        tensor after a step."""
        if model.rt.device.type != "cuda":
            raise RuntimeError("HIP graphs need the GPU")
        self.model = model
        self.cache = cache
        self.greedy = greedy
        self.chosen = None
        self.by_batch = {}

    def step(self, slots, tokens):
        """One decode step of the sequences in `slots` (a token each); returns fp32 logits [len(slots), vocab]
        in memory that the next step of this batch size overwrites."""
        model, cache = self.model, self.cache
        counts, starts, want, tok = model.prepare(cache, slots, tokens)
        if any(c != 1 for c in counts):
            raise ValueError("graphed steps take one token per sequence")
        # launch geometry that depends on lengths (how many blocks share a sequence's keys) is fixed in a
        # graph, so a graph serves lengths up to a bound: the next power of two, at least 1024
        longest = max(s + 1 for s in starts)
        bound = 1024
        while bound < longest:
            bound *= 2
        bound = min(bound, cache.max_context)
        b = (len(slots), bound)
        cap = self.by_batch.get(b)
        if cap is None:
            static = StaticStep(model.rt, cache, len(slots), bound)
            tokens_static = torch.zeros(len(slots), dtype=torch.int32, device=model.rt.device)
            tokens_static.copy_(tok)
            ctx = StepContext(model.rt, cache, slots, counts, starts, want, static=static)
            logits = model.run(ctx, tokens_static)          # this step, eagerly; also loads what capture must not
            if self.greedy:
                model.rt.ops.argmax(logits, out=tokens_static)
            torch.cuda.synchronize(model.rt.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                captured_logits = model.run(ctx, tokens_static)
                if self.greedy:
                    model.rt.ops.argmax(captured_logits, out=tokens_static)
            self.by_batch[b] = _Captured(static, tokens_static, ctx, graph, captured_logits)
            self.chosen = tokens_static
            return logits
        flat, _ = step_arrays(cache, slots, counts, starts, want, cap.static.table_widths)
        cap.static.fill(flat)
        if tok.data_ptr() != cap.tokens.data_ptr():
            cap.tokens.copy_(tok)
        cap.graph.replay()
        self.chosen = cap.tokens
        return cap.logits
