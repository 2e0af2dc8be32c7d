"""Book-keeping of the cache on the host: slots, pages, lengths.

A slot stands for one live sequence.  What is kept per token lives in pages of
`page_size` rows drawn from one pool per group of layers; a slot's page list in
a group grows as its sequence grows and goes back to the pool when the slot is
released.  The reference keeps one dense buffer of max_seq rows per layer for
its single sequence and never checks the bound (runtime/src/lib.rs:4475,
:4489-4490); here every overflow is an error and nothing is lost or held twice.
"""


class CacheError(RuntimeError):
    """The cache cannot do what was asked (full, unknown slot, double release, context overflow)."""


class FreeList:
    """Integers 0..n-1, handed out lowest first, each held by at most one owner."""

    def __init__(self, n, what):
        self.n = n
        self.what = what
        self._free = list(range(n - 1, -1, -1))     # pop() yields the lowest
        self._held = [False] * n

    def available(self):
        return len(self._free)

    def take(self):
        if not self._free:
            raise CacheError(f"no free {self.what}: all {self.n} are in use")
        i = self._free.pop()
        self._held[i] = True
        return i

    def give_back(self, i):
        if not 0 <= i < self.n:
            raise CacheError(f"{self.what} {i} does not exist (there are {self.n})")
        if not self._held[i]:
            raise CacheError(f"{self.what} {i} is released twice or was never taken")
        self._held[i] = False
        self._free.append(i)
        self._free.sort(reverse=True)

    def held(self):
        return [i for i, h in enumerate(self._held) if h]


class GroupPages:
    """Pages of one group of layers: a pool and each slot's page list.

    `rows_cap`: None if a sequence keeps every row, else the number of rows of its
    ring (position p lives in ring row p % rows_cap)."""

    def __init__(self, n_pages, page_size, rows_cap, name):
        self.page_size = page_size
        self.rows_cap = rows_cap
        self.name = name
        self.pool = FreeList(n_pages, f"page of cache group '{name}'")
        self.lists = {}                               # slot -> [page ids]

    def rows_needed(self, length):
        return length if self.rows_cap is None else min(length, self.rows_cap)

    def pages_needed(self, length):
        return -(-self.rows_needed(length) // self.page_size)

    def max_pages(self, max_context):
        return self.pages_needed(max_context)

    def ensure(self, slot, length):
        pages = self.lists.setdefault(slot, [])
        need = self.pages_needed(length)
        if need - len(pages) > self.pool.available():
            raise CacheError(
                f"cache group '{self.name}' is full: slot {slot} needs {need - len(pages)} more pages of "
                f"{self.page_size} rows for length {length}, {self.pool.available()} of {self.pool.n} are free")
        while len(pages) < need:
            pages.append(self.pool.take())

    def release(self, slot):
        for p in self.lists.pop(slot, []):
            self.pool.give_back(p)


class SlotBook:
    """Slots, their lengths, and their pages in every group."""

    def __init__(self, max_slots, groups, max_context):
        self.slots = FreeList(max_slots, "cache slot")
        self.groups = groups                          # list of GroupPages
        self.max_context = max_context
        self.length = {}                              # slot -> tokens held

    def acquire(self):
        s = self.slots.take()
        self.length[s] = 0
        return s

    def release(self, slot):
        if slot not in self.length:
            raise CacheError(f"cache slot {slot} is released twice or was never taken")
        for g in self.groups:
            g.release(slot)
        del self.length[slot]
        self.slots.give_back(slot)

    def live(self):
        return sorted(self.length)

    def grow(self, slot, count):
        """Reserve room for `count` more tokens; returns the length before them."""
        if slot not in self.length:
            raise CacheError(f"cache slot {slot} is not in use")
        old = self.length[slot]
        new = old + count
        if new > self.max_context:
            raise CacheError(
                f"context overflow: slot {slot} holds {old} tokens, {count} more exceed the context of {self.max_context}")
        for g in self.groups:
            g.ensure(slot, new)
        self.length[slot] = new
        return old

    def check_grow(self, slots, counts):
        """Raise CacheError, changing nothing, if the sequences cannot all grow by their counts."""
        if len(set(slots)) != len(slots):
            raise CacheError(f"a step names a cache slot twice: {list(slots)}")
        for g in self.groups:
            need = 0
            for s, c in zip(slots, counts):
                if s not in self.length:
                    raise CacheError(f"cache slot {s} is not in use")
                new = self.length[s] + c
                if new > self.max_context:
                    raise CacheError(
                        f"context overflow: slot {s} holds {self.length[s]} tokens, {c} more exceed "
                        f"the context of {self.max_context}")
                need += g.pages_needed(new) - len(g.lists.get(s, ()))
            if need > g.pool.available():
                raise CacheError(
                    f"cache group '{g.name}' is full: the step needs {need} more pages of {g.page_size} rows, "
                    f"{g.pool.available()} of {g.pool.n} are free")

    def tokens_held(self, page_size):
        """Tokens that live sequences hold, each rounded up to a whole page."""
        return sum(-(-n // page_size) * page_size for n in self.length.values())
