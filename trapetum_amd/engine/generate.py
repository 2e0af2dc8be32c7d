"""The generation loop above the step function.

Requests are taken in order into batches; a batch's prompts run in one step, then every live sequence one
token per step; a sequence that ends (stop token, token limit, context limit) leaves the batch and gives its
slot back at once; when a batch is done the next one takes the freed slots.  The plain loop is the
reference's (runtime/src/bin/gemma_run.rs:12-15, runtime/src/lib.rs:1574-1588): push the chosen token, run
it, choose the next; a stop token ends the sequence before it is emitted (runtime/src/bin/serve.rs:347-350),
and the last emitted token is not run through the model.  The reference runs one sequence and truncates long
prompts silently (serve.rs:323-326); here a prompt that cannot fit is an error.
"""
import collections
import dataclasses
from typing import List

from ..cache.slots import CacheError
from ..sampling.sampler import RequestSampling, Sampler, SamplingParams


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


def _index(like, rows):
    import torch
    return torch.tensor(rows, dtype=torch.long, device=like.device)


def generate(model, cache, prompts, max_tokens=256, params=None, seed=0, stop_ids=(), max_batch=64,
             on_tokens=None, with_reasons=False, decode_step=None):
    """Generate for every prompt (lists of token ids); returns the new tokens of each, in the prompts' order.

    on_tokens(step, [(request index, token), ...]) is called after every step with what it emitted.
    decode_step(slots, tokens) -> logits replaces the model's step for the one-token steps (graph replay).
    """
    params = params or SamplingParams()
    sampler = Sampler(model.rt, params)
    stop = set(int(s) for s in stop_ids)
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
        slots = {i: cache.acquire() for i in batch}
        state = {i: RequestSampling(seed, i, list(prompts[i])) for i in batch}
        out = {i: [] for i in batch}
        try:
            flat = [t for i in batch for t in prompts[i]]
            logits = model.step(cache, [slots[i] for i in batch], flat, counts=[len(prompts[i]) for i in batch])
            live = list(batch)
            step = decode_step or (lambda sl, tk: model.step(cache, sl, tk))
            while live:
                requests = [state[i] for i in live]
                ids = sampler.choose_on_device(logits, requests)
                fetch = model.rt.download_i32(ids)
                # The next step is enqueued before the host knows the tokens (they stay on the device), so the GPU
                # does not wait for the host: every sequence that its length allows to go on takes part.  One that
                # turns out to have stopped has run one step for nothing; its row is dropped below.
                ahead = [i for i in live if len(out[i]) + 1 < max_tokens
                         and len(prompts[i]) + len(out[i]) + 1 <= cache.max_context]
                next_logits = None
                if ahead:
                    tokens = ids if len(ahead) == len(live) else ids[_index(ids, [live.index(i) for i in ahead])]
                    next_logits = step([slots[i] for i in ahead], tokens)
                chosen = fetch()
                sampler.record(requests, chosen)
                emitted, still = [], []
                for i, tok in zip(live, chosen):
                    if tok in stop:
                        results[i] = Finished(out[i], "stop")
                    else:
                        out[i].append(tok)
                        emitted.append((i, tok))
                        if len(out[i]) >= max_tokens:
                            results[i] = Finished(out[i], "length")
                        elif len(prompts[i]) + len(out[i]) > cache.max_context:
                            results[i] = Finished(out[i], "context")
                        else:
                            still.append(i)
                    if results[i] is not None:
                        cache.release(slots.pop(i))
                if on_tokens is not None and emitted:
                    on_tokens(step_no, emitted)
                step_no += 1
                if still and len(still) != len(ahead):
                    next_logits = next_logits[_index(next_logits, [ahead.index(i) for i in still])]
                live, logits = still, next_logits
        finally:
            for s in slots.values():
                cache.release(s)
    return results if with_reasons else [r.tokens for r in results]
