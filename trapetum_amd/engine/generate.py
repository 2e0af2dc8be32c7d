"""The generation loop above the step function.

Requests are taken in order into batches; a batch's prompts run in one step, then every live sequence one
token per step; a sequence that ends (stop token, token limit, context limit) leaves the batch and gives its
slot back at once; when a batch is done the next one takes the freed slots.  The plain loop is the
reference's (runtime/src/bin/gemma_run.rs:12-15, runtime/src/lib.rs:1574-1588): push the chosen token, run
it, choose the next; a stop token ends the sequence before it is emitted (runtime/src/bin/serve.rs:347-350),
and the last emitted token is not run through the model.  The reference runs one sequence and truncates long
prompts silently (serve.rs:323-326); here a prompt that cannot fit is an error.

The chosen tokens stay on the device: a step reads the ids the step before chose, and the host reads them one
step behind, after it has enqueued the next step, so the GPU does not wait for the host.  A sequence that turns
out to have stopped has then run one step for nothing.  With captured graphs (`GraphedDecode`) the choice is
part of the graph and a step is one copy of its numbers and one replay; without them the same loop runs eager
steps.  There is one loop: `BatchRun` is what `generate` runs, and what the benchmark times.
"""
import collections
import dataclasses
from typing import List

import numpy as np
import torch

from ..cache.slots import CacheError
from ..sampling.sampler import RequestSampling, Sampler, SamplingParams
from .graphs import graph_rows


@dataclasses.dataclass
class Finished:
    tokens: List[int]
    reason: str                 # "stop", "length" (max_tokens reached) or "context" (the cache's context is full)


def plan_batch(queue, prompts, max_tokens, max_batch, free_tokens, page_size, max_context):
    """How many requests from the head of the queue run together: as many as have room for their prompt and
    everything they may generate, each rounded up to whole pages.  Returns the number taken (at least one,
    or an error if even the first does not fit)."""
    taken = 0
    budget = free_tokens
    for i in queue:
        if taken >= max_batch:
            break
        n = len(prompts[i])
        if n == 0:
            raise ValueError(f"request {i} has an empty prompt")
        if n > max_context:
            raise CacheError(f"request {i}: a prompt of {n} tokens exceeds the context of {max_context}")
        need = min(n + max_tokens, max_context)
        need = -(-need // page_size) * page_size
        if need > budget:
            break
        budget -= need
        taken += 1
    if taken == 0:
        i = queue[0]
        raise CacheError(
            f"request {i} needs room for {min(len(prompts[i]) + max_tokens, max_context)} tokens, "
            f"the cache has {free_tokens} free")
    return taken


class EagerRows:
    """A batch's rows while it decodes, by eager steps: row r is the r-th sequence of the batch; `tokens[r]` is the
    id it chose last."""

    def __init__(self, model, cache, slots, sampler, requests):
        self.model, self.cache, self.slots, self.sampler, self.requests = model, cache, slots, sampler, requests
        self.tokens = None

    def start(self, ids):
        self.tokens = ids

    def step(self, rows):
        """Run the rows' last tokens through the model and choose their next ones."""
        everyone = len(rows) == self.tokens.numel()
        index = None if everyone else torch.tensor(rows, dtype=torch.long, device=self.tokens.device)
        tok = self.tokens if everyone else self.tokens[index]
        logits = self.model.step(self.cache, [self.slots[r] for r in rows], tok)
        ids = self.sampler.choose_on_device(logits, [self.requests[r] for r in rows])
        if everyone:
            self.tokens = ids
        else:
            self.tokens = self.tokens.clone()
            self.tokens[index] = ids

    def fetch(self):
        """Start the download of the rows' last ids; returns a function that waits for it and gives {row: id}."""
        wait = self.model.rt.download_i32(self.tokens)
        return lambda: dict(enumerate(wait()))


class GraphRows:
    """The same by graph replays.  A row keeps its place in the graph while its sequence lives; the places of
    sequences that ended, and those beyond the batch, stand for no sequence (the cache's spare slot).  When half
    of a graph's rows or fewer are left alive, the live ones move to the front of a graph of half the size."""

    def __init__(self, graphs, model, cache, slots, sampler, requests):
        self.graphs, self.model, self.cache, self.slots = graphs, model, cache, slots
        self.requests = requests
        self.choice = sampler.graph_choice()
        self.penalty = isinstance(self.choice[-1], tuple)
        self.nb = graph_rows(len(slots))
        self.place = list(range(len(slots)))          # row -> place in the graph's rows

    def start(self, ids):
        rows, n = self.graphs.rows(self.nb), len(self.slots)
        rows.tokens[:n].copy_(ids)
        if self.penalty:
            # the rings start as the host knows them (the prompts' last tokens) and take the first ids on the device
            rings = [Sampler.ring_of(r) for r in self.requests]
            rt = self.model.rt
            rows.recent[:n].copy_(rt.upload_i32(np.asarray([ring for ring, _ in rings], dtype=np.int32).reshape(-1)).view(n, -1))
            rows.cursor[:n].copy_(rt.upload_i32(np.asarray([at for _, at in rings], dtype=np.int32)))
            rt.ops.recent_push(rows.tokens, rows.recent, rows.cursor)

    def step(self, rows):
        cache = self.cache
        nb = graph_rows(len(rows))
        if nb < self.nb:                              # the live rows move into a smaller graph
            old, new = self.graphs.rows(self.nb), self.graphs.rows(nb)
            index = torch.tensor([self.place[r] for r in rows], dtype=torch.long, device=old.tokens.device)
            new.tokens[:len(rows)].copy_(old.tokens[index])
            if self.penalty:
                new.recent[:len(rows)].copy_(old.recent[index])
                new.cursor[:len(rows)].copy_(old.cursor[index])
            self.place = [None] * len(self.place)
            for at, r in enumerate(rows):
                self.place[r] = at
            self.nb = nb
        slots, starts = [cache.spare_slot] * self.nb, [0] * self.nb
        uniforms = [0.5] * self.nb if self.choice[0] == "sample" else None
        live = [self.slots[r] for r in rows]
        cache.check_grow(live, [1] * len(live))
        for r in rows:
            at = self.place[r]
            slots[at] = self.slots[r]
            starts[at] = cache.grow(self.slots[r], 1)
            if uniforms is not None:
                uniforms[at] = self.requests[r].next_uniform()
        self.graphs.run(self.nb, slots, starts, self.choice, uniforms)

    def fetch(self):
        wait = self.model.rt.download_i32(self.graphs.rows(self.nb).tokens)
        place = list(self.place)
        return lambda: (lambda ids: {r: ids[at] for r, at in enumerate(place) if at is not None})(wait())


class BatchRun:
    """One batch of requests from its prompts to its last token.

    items: [(request index, prompt tokens, request id for the sampler)].  `prefill()` runs the prompts and chooses
    every sequence's first token; each `advance()` enqueues one more decode step for the sequences that may go on
    and then settles the tokens of the step before (stops, limits, slots given back); `done` when no sequence is left.
    """

    def __init__(self, model, cache, items, max_tokens, sampler, seed, stop, graphs=None):
        self.model, self.cache, self.sampler = model, cache, sampler
        self.items = items
        self.max_tokens = max_tokens
        self.stop = stop
        self.requests = [RequestSampling(seed, rid, list(prompt)) for _, prompt, rid in items]
        self.out = [[] for _ in items]
        self.finished = {}                            # row -> Finished
        self.slots = []
        self.pending = None                           # (rows, wait): ids chosen on the device that the host has not read
        self.rows = None
        self.graphs = graphs
        # the host reads a step's ids before it enqueues the next only where it makes the choice itself from them
        self.in_turn = graphs is None and sampler.needs_the_last_token
        self.steps = 0

    @property
    def done(self):
        return self.pending is None

    def prefill(self):
        model, cache = self.model, self.cache
        self.slots = [cache.acquire() for _ in self.items]
        flat = [t for _, prompt, _ in self.items for t in prompt]
        logits = model.step(cache, self.slots, flat, counts=[len(prompt) for _, prompt, _ in self.items])
        ids = self.sampler.choose_on_device(logits, self.requests)
        if self.graphs is not None:
            self.rows = GraphRows(self.graphs, model, cache, self.slots, self.sampler, self.requests)
        else:
            self.rows = EagerRows(model, cache, self.slots, self.sampler, self.requests)
        self.rows.start(ids)
        self.pending = (list(range(len(self.items))), self.rows.fetch())

    def _may_go_on(self, r, emitted):
        """Whether row r, having emitted `emitted` tokens, runs its last token through the model for another one."""
        return emitted < self.max_tokens and len(self.items[r][1]) + emitted <= self.cache.max_context

    def _settle(self, rows, ids):
        """The ids the rows chose: a stop token ends a row, any other is emitted; returns (emitted, rows that go on)."""
        emitted, still = [], []
        for r in rows:
            tok, out = ids[r], self.out[r]
            if tok in self.stop:
                self.finished[r] = Finished(out, "stop")
            else:
                out.append(tok)
                emitted.append((self.items[r][0], tok))
                if len(out) >= self.max_tokens:
                    self.finished[r] = Finished(out, "length")
                elif len(self.items[r][1]) + len(out) > self.cache.max_context:
                    self.finished[r] = Finished(out, "context")
                else:
                    still.append(r)
            if r in self.finished:
                self.cache.release(self.slots[r])
                self.slots[r] = None
        return emitted, still

    def advance(self):
        """Returns what the settled step emitted: [(request index, token)]."""
        rows, wait = self.pending
        if self.in_turn:
            # the next choice looks at the tokens chosen so far: the host reads them before it goes on
            ids = wait()
            self.sampler.record([self.requests[r] for r in rows], [ids[r] for r in rows])
            emitted, still = self._settle(rows, ids)
            ahead = still
            if ahead:
                self.rows.step(ahead)
        else:
            # every row that its length allows to go on runs before the host knows what it chose last
            ahead = [r for r in rows if self._may_go_on(r, len(self.out[r]) + 1)]
            if ahead:
                self.rows.step(ahead)
            emitted, still = self._settle(rows, wait())
            ahead = [r for r in ahead if r in still]
        self.steps += 1
        self.pending = (ahead, self.rows.fetch()) if ahead else None
        return emitted

    def close(self):
        for i, s in enumerate(self.slots):
            if s is not None:
                self.cache.release(s)
                self.slots[i] = None
        self.pending = None


def generate(model, cache, prompts, max_tokens=256, params=None, seed=0, stop_ids=(), max_batch=64,
             on_tokens=None, with_reasons=False, graphs=None, request_ids=None):
    """Generate for every prompt (lists of token ids); returns the new tokens of each, in the prompts' order.

    on_tokens(step, [(request index, token), ...]) is called after every step with what it emitted.
    graphs: a GraphedDecode for the one-token steps.  request_ids: what the sampler's random numbers are keyed by
    beside the seed (default: a request's place in `prompts`).
    """
    params = params or SamplingParams()
    sampler = Sampler(model.rt, params)
    stop = set(int(s) for s in stop_ids)
    if request_ids is None:
        request_ids = list(range(len(prompts)))
    if len(request_ids) != len(prompts):
        raise ValueError(f"{len(prompts)} prompts but {len(request_ids)} request ids")
    results = [None] * len(prompts)
    if max_tokens <= 0:
        for i in range(len(prompts)):
            results[i] = Finished([], "length")
        return results if with_reasons else [r.tokens for r in results]
    queue = collections.deque(range(len(prompts)))
    step_no = 0
    while queue:
        free = cache.max_tokens - cache.tokens_held()
        n = plan_batch(queue, prompts, max_tokens, max_batch, free, cache.page_size, cache.max_context)
        batch = [queue.popleft() for _ in range(n)]
        run = BatchRun(model, cache, [(i, prompts[i], int(request_ids[i])) for i in batch], max_tokens, sampler, seed,
                       stop, graphs=graphs)
        try:
            run.prefill()
            while not run.done:
                emitted = run.advance()
                if on_tokens is not None and emitted:
                    on_tokens(step_no, emitted)
                step_no += 1
        finally:
            run.close()
        for r, i in enumerate(batch):
            results[i] = run.finished[r]
    return results if with_reasons else [r.tokens for r in results]
