"""A batch decoded greedily with the chosen ids staying on the device (what the benchmark times).

Prompts run in one step; after that every step feeds the ids the previous step chose, so the host neither
reads logits nor waits for the device between steps (the reference downloads the whole logits vector and
picks on the host every token: runtime/src/lib.rs:4559-4560, runtime/src/bin/gemma_run.rs:15).
"""
from .graphs import GraphedDecode


class DecodeLoop:
    def __init__(self, model, cache, use_graph=True):
        self.model = model
        self.cache = cache
        self.graphed = GraphedDecode(model, cache, greedy=True) if use_graph else None
        self.slots = []
        self.tokens = None

    def start(self, prompts):
        self.slots = [self.cache.acquire() for _ in prompts]
        flat = [t for p in prompts for t in p]
        logits = self.model.step(self.cache, self.slots, flat, counts=[len(p) for p in prompts])
        self.tokens = self.model.rt.ops.argmax(logits)
        return self.tokens

    def step(self):
        if self.graphed is not None:               # the graph picks the tokens and leaves them where its next replay reads them
            self.graphed.step(self.slots, self.tokens)
            self.tokens = self.graphed.chosen
        else:
            logits = self.model.step(self.cache, self.slots, self.tokens)
            self.tokens = self.model.rt.ops.argmax(logits)
        return self.tokens

    def finish(self):
        for s in self.slots:
            self.cache.release(s)
        self.slots = []
