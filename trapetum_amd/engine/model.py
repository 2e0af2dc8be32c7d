"""A model assembled from a ModelSpec, and its one step function.

The step runs only the rows it is given, as one packed batch, from the cache
that earlier steps left, and returns fp32 logits at the wanted rows.  Order of
operations as in the reference's forward (runtime/src/lib.rs:4553-4562): embed,
each scheduled layer, final norm, head, final cap; the reference does this for one
token of one sequence and always returns the whole logits vector.
"""
import numpy as np
import torch

from ..cache.store import ModelCache
from ..models.spec import ModelSpec
from ..registry import build_part, part_class
from .batch import StepContext, StepError, classify


class AssembledLayer:
    def __init__(self, lspec):
        mixer = build_part("mixer", lspec.mixer)
        ff = build_part("feed_forward", lspec.feed_forward)
        block_cls = part_class("block", lspec.block[0])
        unknown = set(lspec.norms or {}) - set(block_cls.norm_sites())
        if unknown:
            raise ValueError(f"the layer's spec names norms for {sorted(unknown)}, block '{lspec.block[0]}' has {list(block_cls.norm_sites())}")
        self.block = block_cls(mixer, ff, lambda site: build_part("norm", lspec.norm_of(site)), **lspec.block[1])
        self.prefixes = lspec.prefixes
        self.places = [(mixer, self._prefix("mixer")), (ff, self._prefix("feed_forward"))]
        for site, norm in self.block.norms.items():
            self.places.append((norm, self._prefix(site)))
        if self.block.tensor_specs():
            self.places.append((self.block, self._prefix("block")))

    def _prefix(self, site):
        if site not in self.prefixes:
            raise ValueError(f"the layer's spec gives no tensor-name prefix for '{site}'")
        return self.prefixes[site]


class Model:
    def __init__(self, spec: ModelSpec, rt):
        spec.validate()
        self.spec = spec
        self.rt = rt
        self.embedding = build_part("embedding", spec.embedding)
        self.layers = [AssembledLayer(ls) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.places = [(self.embedding, spec.embedding_prefix)]
        for layer in self.layers:
            self.places.extend(layer.places)
        self.places.append((self.final_norm, spec.final_norm_prefix))
        self.places.append((self.head, spec.head_prefix))
        self.schedule = spec.schedule
        self._shared = sorted({e.cache_of for e in self.schedule if e.cache_of is not None})
        self.bound = False

    # --- tensors ------------------------------------------------------------------------
    def tensor_layout(self):
        """{checkpoint name: TensorSpec} of every tensor the model needs; two parts may name the
        same tensor (a tied head) if they agree on its shape."""
        out = {}
        for part, prefix in self.places:
            for local, ts in part.tensor_specs().items():
                name = prefix + local
                if name in out and tuple(out[name].shape) != tuple(ts.shape):
                    raise ValueError(f"tensor '{name}' is declared with shapes {out[name].shape} and {ts.shape}")
                out.setdefault(name, ts)
        return out

    def bind(self, fetch):
        """`fetch(name)` -> device tensor, called once per checkpoint name."""
        got = {}
        for part, prefix in self.places:
            local = {}
            for name in part.tensor_specs():
                full = prefix + name
                if full not in got:
                    got[full] = fetch(full)
                local[name] = got[full]
            part.bind(local, self.rt)
        self.bound = True

    # --- cache --------------------------------------------------------------------------
    def entry_cache_specs(self):
        specs = []
        for e in self.schedule:
            specs.append(None if e.cache_of is not None else self.layers[e.layer].block.mixer.cache_spec())
        return specs

    def new_cache(self, max_tokens, max_context=None, max_slots=None, page_size=64):
        max_context = max_context or max_tokens
        max_slots = max_slots or max(1, -(-max_tokens // page_size))
        return ModelCache(self.entry_cache_specs(), max_tokens, max_context, max_slots, page_size,
                          self.rt.dtype, self.rt.device)

    # --- the step -----------------------------------------------------------------------
    def step(self, cache, slots, tokens, counts=None, want=None):
        """Run one step.

        slots:  cache slots of the step's sequences.
        tokens: flat token ids, sequence after sequence (list, or an int32 device tensor);
        counts: tokens per sequence (default: one each).
        want:   flat row indices whose logits are returned, in this order (default: each sequence's
                last row).  Returns fp32 [len(want), vocab] on the device, or None when want is empty.
        """
        counts, starts, want, tok = self.prepare(cache, slots, tokens, counts, want)
        ctx = StepContext(self.rt, cache, slots, counts, starts, want)
        return self.run(ctx, tok)

    def prepare(self, cache, slots, tokens, counts=None, want=None):
        """Check the step, reserve its cache rows, and bring the tokens to the device.  A refused step leaves
        the cache as it was."""
        if not self.bound:
            raise RuntimeError("the model has no weights yet: load a folder or random weights first")
        n = len(slots)
        counts = [1] * n if counts is None else list(counts)
        if len(counts) != n:
            raise StepError(f"{n} slots but {len(counts)} counts")
        m = sum(counts)
        host_tokens = None
        if isinstance(tokens, torch.Tensor):
            if tokens.dtype != torch.int32 or tokens.numel() != m:
                raise StepError(f"token tensor must be int32 with {m} entries")
            tok = tokens.to(self.rt.device).reshape(-1)
        else:
            host_tokens = [int(t) for t in tokens]
            if len(host_tokens) != m:
                raise StepError(f"counts add up to {m} tokens, {len(host_tokens)} were given")
            bad = [t for t in host_tokens if not 0 <= t < self.spec.vocab_size]
            if bad:
                raise StepError(f"token id {bad[0]} is outside the vocabulary of {self.spec.vocab_size}")
        if want is None:
            want, o = [], 0
            for c in counts:
                o += c
                want.append(o - 1)
        want = [int(w) for w in want]
        if any(not 0 <= w < m for w in want):
            raise StepError(f"wanted rows {want} reach outside the step's {m} rows")
        for s in slots:
            if s not in cache.book.length:
                raise StepError(f"cache slot {s} is not in use")
        starts = [cache.length(s) for s in slots]
        classify(counts, starts)                 # refuses an empty step, before the cache changes
        cache.check_grow(slots, counts)
        for s, c in zip(slots, counts):
            cache.grow(s, c)
        if host_tokens is not None:
            tok = self.rt.upload_i32(np.asarray(host_tokens, dtype=np.int32))
        return counts, starts, want, tok

    def run(self, ctx, tok):
        """The device work of a step (what a HIP graph captures): embed, layers, final norm, head."""
        ctx.mark_shared(self._shared)
        cache = ctx.cache
        stream = self.embedding.forward(ctx, tok)
        ctx.dump("embed", stream)
        whole = ctx.n_want == ctx.n_rows and ctx.identity_want
        normed = None
        last = len(self.schedule) - 1
        for i, e in enumerate(self.schedule):
            ctx.entry = i
            ctx.cache_owner = i if e.cache_of is None else e.cache_of
            # the norm that meets the stream next, for this block to fuse into its last add
            if i < last:
                next_norm = self.layers[self.schedule[i + 1].layer].block.entry_norm()
            else:
                next_norm = self.final_norm if whole else None
            if next_norm is not None and next_norm.gain is None:
                next_norm = None
            stream, normed = self.layers[e.layer].block.forward(ctx, stream, cache.site(ctx.cache_owner),
                                                                 normed=normed, next_norm=next_norm)
        ctx.finish()
        if ctx.n_want == 0:
            return None
        if whole and normed is not None:
            rows = normed
        else:
            rows = stream if whole else ctx.ops.gather_rows(stream, ctx.want_rows)
            rows = self.final_norm.forward(ctx, rows)
        ctx.entry = None
        ctx.dump("final_norm", rows)
        logits = self.head.forward(ctx, rows)
        ctx.dump("logits", logits)
        from .. import flags
        if flags.debug_dump():                  # the five largest logits of the last wanted row, smaller ids first on ties
            import sys
            z = logits[-1].double().cpu()
            order = sorted(range(z.numel()), key=lambda i: (-float(z[i]), i))[:5]
            print("[ldump] top5= " + ",".join(f"{i}:{float(z[i]):.4f}" for i in order), file=sys.stderr, flush=True)
        return logits
