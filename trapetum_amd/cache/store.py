"""The cache's device storage.

Every run of a layer (a schedule entry) that keeps something between steps
declares what: tensors per token (of all tokens, or of a window of them), or a
state of fixed size.  Entries with the same needs form a group with storage of
its own:

  per token    one pool per named tensor; a tensor of shape (*lead, d) per token
               lives in a pool [entries, pages, *lead, page_size, d] (a page's rows
               stand before the last dimension, so that a row of d elements is
               contiguous); a sequence's rows are found through its page list.  A
               window group keeps a ring: position p lives in ring row p % rows_cap.
               (Attention declares keys and values, each (kv_heads, head_dim); a
               mixer that keeps one tensor per token declares one.)
  state        [entries, slots, *shape], zeroed when a slot is taken.

Beyond what sequences can take, every pool has one spare page and every state one
spare slot (`ModelCache.spare_slot`): a row of a step that stands for no sequence
(padding of a captured decode graph to its batch size) writes and reads there.

The reference allocates cache_k / cache_v [max_seq, kv_heads * head_dim] per
layer for its one sequence, K stored after RoPE (runtime/src/lib.rs:4475,
:4488-4490), and models no window (:4455).
"""
import dataclasses
from typing import Optional

import numpy as np
import torch

from .slots import CacheError, GroupPages, SlotBook


@dataclasses.dataclass(frozen=True)
class TokenSpec:
    """What a mixer keeps of every token: named tensors, each of a fixed shape, in the engine's activation dtype."""
    tensors: tuple                      # ((name, shape), ...): hashable, in the mixer's order
    window: Optional[int] = None        # None: every token is kept

    @staticmethod
    def of(window=None, **tensors):
        """TokenSpec.of(window, k=(kv_heads, head_dim), v=(kv_heads, head_dim))"""
        for name, shape in tensors.items():
            if not shape or any(int(n) <= 0 for n in shape):
                raise CacheError(f"per-token tensor '{name}' needs a shape of positive sizes, found {shape!r}")
        return TokenSpec(tuple((name, tuple(int(n) for n in shape)) for name, shape in tensors.items()), window)

    def shape_of(self, name):
        for n, shape in self.tensors:
            if n == name:
                return shape
        raise CacheError(f"the cache keeps no per-token tensor '{name}' here (it keeps {[n for n, _ in self.tensors]})")


@dataclasses.dataclass(frozen=True)
class StateSpec:
    shape: tuple
    dtype: str = "float32"              # "float32" or "activation" (the engine's activation dtype)


class CacheSite:
    """What one schedule entry sees of the cache."""

    def __init__(self, spec, group_index, index_in_group, group):
        self.spec = spec
        self.group_index = group_index
        self.index_in_group = index_in_group
        self._group = group

    @property
    def per_token(self):
        return isinstance(self.spec, TokenSpec)

    def tensor(self, name):
        """The pool of one of the per-token tensors the entry declared: [pages, *lead, page_size, d]."""
        self.spec.shape_of(name)
        return self._group.pools[name][self.index_in_group]

    @property
    def rows_cap(self):
        return self._group.pages.rows_cap

    @property
    def state(self):
        return self._group.tensor[self.index_in_group]


class _TokenGroup:
    def __init__(self, spec, entries, n_pages, max_slots, page_size, max_context, dtype, device, name):
        self.spec = spec
        self.entries = entries
        rows_cap = None
        if spec.window is not None and spec.window < max_context:
            rows_cap = -(-spec.window // page_size) * page_size
            n_pages = min(n_pages, max_slots * (rows_cap // page_size))      # a ring never grows beyond its rows
        self.pages = GroupPages(n_pages, page_size, rows_cap, name)
        self.spare_page = n_pages                                          # the pool's last page, never handed out
        self.pools = {}
        for tname, shape in spec.tensors:
            self.pools[tname] = torch.zeros((len(entries), n_pages + 1) + shape[:-1] + (page_size, shape[-1]), dtype=dtype, device=device)
        self.max_pages_per_seq = self.pages.max_pages(max_context)


class _StateGroup:
    def __init__(self, spec, entries, max_slots, dtype, device):
        self.spec = spec
        self.entries = entries
        dt = torch.float32 if spec.dtype == "float32" else dtype
        self.tensor = torch.zeros((len(entries), max_slots + 1) + tuple(spec.shape), dtype=dt, device=device)


class ModelCache:
    """Slots, pages and storage for one model instance.

    entry_specs: for every schedule entry a TokenSpec, a StateSpec or None.
    max_tokens:  tokens that live sequences may hold together, each rounded up to a page.
    max_context: longest single sequence.
    """

    def __init__(self, entry_specs, max_tokens, max_context, max_slots, page_size, dtype, device):
        if page_size <= 0 or page_size % 16:
            raise CacheError(f"page size {page_size} must be a positive multiple of 16")
        self.page_size = page_size
        self.max_context = max_context
        self.max_tokens = max_tokens
        self.max_slots = max_slots
        self.spare_slot = max_slots           # a slot no sequence takes: see the module's text
        n_pages = max(1, -(-max_tokens // page_size))
        self.token_groups, self.state_groups = [], []
        self._site_of = {}
        keyed = {}
        for entry, spec in enumerate(entry_specs):
            if spec is not None:
                keyed.setdefault(spec, []).append(entry)
        for spec, entries in keyed.items():
            if isinstance(spec, TokenSpec):
                name = f"tokens{len(self.token_groups)}:" + ("all" if spec.window is None else f"window{spec.window}")
                g = _TokenGroup(spec, entries, n_pages, max_slots, page_size, max_context, dtype, device, name)
                gi = len(self.token_groups)
                self.token_groups.append(g)
            elif isinstance(spec, StateSpec):
                g = _StateGroup(spec, entries, max_slots, dtype, device)
                gi = len(self.state_groups)
                self.state_groups.append(g)
            else:
                raise CacheError(f"schedule entry declares an unknown cache need: {spec!r}")
            for i, entry in enumerate(entries):
                self._site_of[entry] = CacheSite(spec, gi, i, g)
        self.book = SlotBook(max_slots, [g.pages for g in self.token_groups], max_context)

    # --- what parts use -------------------------------------------------------------
    def site(self, entry):
        return self._site_of.get(entry)

    # --- what the engine uses ---------------------------------------------------------
    def acquire(self):
        slot = self.book.acquire()
        for g in self.state_groups:
            g.tensor[:, slot].zero_()
        return slot

    def release(self, slot):
        self.book.release(slot)

    def grow(self, slot, count):
        return self.book.grow(slot, count)

    def check_grow(self, slots, counts):
        self.book.check_grow(slots, counts)

    def length(self, slot):
        return self.book.length[slot]

    def live_slots(self):
        return self.book.live()

    def tokens_held(self):
        return self.book.tokens_held(self.page_size)

    def page_table(self, group_index, slots, width=None):
        """int32 [len(slots), width]: page ids of each slot in a group, -1 where it has none; the spare slot's row
        names the spare page."""
        g = self.token_groups[group_index]
        width = width or max(1, max(len(g.pages.lists.get(s, ())) for s in slots))
        t = np.full((len(slots), width), -1, dtype=np.int32)
        for i, s in enumerate(slots):
            if s == self.spare_slot:
                t[i, 0] = g.spare_page
                continue
            p = g.pages.lists.get(s, ())
            t[i, :len(p)] = p
        return t

    def bytes(self):
        n = 0
        for g in self.token_groups:
            n += sum(p.numel() * p.element_size() for p in g.pools.values())
        for g in self.state_groups:
            n += g.tensor.numel() * g.tensor.element_size()
        return n
