"""Choosing the next token: greedy, or the reference's temperature / top-p sampling.

As the reference's next_tok (runtime/src/bin/serve.rs:41-72): temperature <= 0 is argmax with the smallest
index winning ties (runtime/src/lib.rs:1376-1380); otherwise the top_k largest logits (256 there), softmax of
(z - max) / T, the shortest prefix whose mass reaches top_p, and a draw r = u * kept mass walked down the
sorted candidates.  A repetition penalty over the last 128 tokens, prompt included, comes first
(serve.rs:285-294, :327-333).  The reference seeds one xorshift64 state from the clock (serve.rs:309-311);
here every request owns a state derived from (seed, request id), the id being the caller's or else the
request's place in the call, and draws one number per token of its own, so a request's draws do not depend on
which other requests share its batch: the same request under the same id and seed gets the same tokens alone
and in a batch.  The logits never leave the device: only the chosen ids do.
"""
import collections
import dataclasses

import numpy as np
import torch

MASK64 = (1 << 64) - 1
RECENT_WINDOW = 128          # tokens the repetition penalty looks back over (serve.rs:327)
MAX_TOP_K = 1024


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 0.0            # 0 (or less): greedy
    top_p: float = 0.95                 # the reference's default (serve.rs:1292)
    top_k: int = 256                    # the reference keeps the 256 largest (serve.rs:52); 0: the whole vocabulary, in id order
    repetition_penalty: float = 1.0     # 1 (or less): off

    def validate(self):
        if not 0 <= self.top_k <= MAX_TOP_K:
            raise ValueError(f"top_k {self.top_k} must lie in 0..{MAX_TOP_K} (0: the whole vocabulary)")
        if not self.top_p > 0:
            raise ValueError(f"top_p {self.top_p} must be positive")
        if self.top_k == 0 and self.top_p < 1:
            raise ValueError(f"a nucleus (top_p {self.top_p}) needs top_k between 1 and {MAX_TOP_K}")


def xorshift64(state):
    """One step of the reference's generator (serve.rs:63)."""
    state ^= (state << 13) & MASK64
    state ^= state >> 7
    state ^= (state << 17) & MASK64
    return state


def initial_state(seed, index):
    """A non-zero 64-bit state from (seed, request id): splitmix64 over their mix."""
    z = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
    z ^= z >> 31
    return z | 1


class RequestSampling:
    """What sampling remembers of one request."""

    def __init__(self, seed, request_id, prompt):
        self.state = initial_state(seed, request_id)
        self.recent = collections.deque(prompt[-RECENT_WINDOW:], maxlen=RECENT_WINDOW)

    def next_uniform(self):
        self.state = xorshift64(self.state)
        return float(np.float32((self.state >> 11) / float(1 << 53)))     # the reference draws in f32 (serve.rs:65)

    def saw(self, token):
        self.recent.append(token)


class Sampler:
    def __init__(self, rt, params):
        params.validate()
        self.rt = rt
        self.params = params

    @property
    def needs_the_last_token(self):
        """Whether a choice made on the host's side (`choose_on_device`) depends on the tokens chosen before it: then
        the host must know them first.  (A captured graph keeps the recent tokens on the device instead.)"""
        return self.params.repetition_penalty > 1.0

    def graph_choice(self):
        """The choice as a captured decode graph makes it by itself (see GraphedDecode.run): ("greedy",) or
        ("sample", temperature, top_k, top_p), followed by ("penalty", value) when the recent tokens count."""
        p = self.params
        choice = ("greedy",) if p.temperature <= 0 else ("sample", float(p.temperature), int(p.top_k), float(p.top_p))
        if p.repetition_penalty > 1.0:
            choice += (("penalty", float(p.repetition_penalty)),)
        return choice

    @staticmethod
    def ring_of(request):
        """A request's recent tokens as a ring of RECENT_WINDOW places (-1: empty) and the place the next one takes."""
        recent = list(request.recent)
        return recent + [-1] * (RECENT_WINDOW - len(recent)), len(recent) % RECENT_WINDOW

    def choose(self, logits, requests):
        """logits fp32 [n, vocab] on the device (changed in place by a penalty); one RequestSampling per row.
        Returns the chosen ids as a list, after which each request has seen its token."""
        out = self.rt.download_i32(self.choose_on_device(logits, requests))()
        self.record(requests, out)
        return out

    def choose_on_device(self, logits, requests):
        """The choice as an int32 tensor on the device, nothing waited for; `record` the ids once they are known."""
        p = self.params
        ops = self.rt.ops
        if p.repetition_penalty > 1.0:
            recent = np.full((len(requests), RECENT_WINDOW), -1, dtype=np.int32)
            for i, r in enumerate(requests):
                recent[i, :len(r.recent)] = list(r.recent)
            ops.apply_repetition_penalty(logits, self.rt.upload_i32(recent), p.repetition_penalty)
        if p.temperature <= 0:
            return ops.argmax(logits)
        u = np.asarray([r.next_uniform() for r in requests], dtype=np.float32)
        uniforms = self.rt.upload_i32(u.view(np.int32)).view(torch.float32)
        return ops.sample(logits, p.temperature, p.top_k, p.top_p, uniforms)

    @staticmethod
    def record(requests, ids):
        for r, t in zip(requests, ids):
            r.saw(int(t))
