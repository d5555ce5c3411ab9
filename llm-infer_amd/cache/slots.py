"""Host-side bookkeeping: which sequence slots and which pages are in use.
Pure Python, so that it is tested without a GPU."""
from __future__ import annotations


class CacheError(RuntimeError):
    pass


class SlotAllocator:
    """Slots 0..n-1.  A slot is held once; it is given back once; the lowest free slot is
    handed out first, so a batch that follows another uses the same slots again."""

    def __init__(self, n: int):
        if n <= 0:
            raise CacheError("a cache needs at least one slot")
        self.n = n
        self._free = list(range(n - 1, -1, -1))
        self._held = set()

    def alloc(self) -> int:
        if not self._free:
            raise CacheError(f"all {self.n} sequence slots are in use")
        s = self._free.pop()
        self._held.add(s)
        return s

    def free(self, slot: int) -> None:
        if slot not in self._held:
            raise CacheError(f"slot {slot} is not held (freed twice or never allocated)")
        self._held.remove(slot)
        self._free.append(slot)
        self._free.sort(reverse=True)

    def held(self) -> set:
        return set(self._held)

    @property
    def n_free(self) -> int:
        return len(self._free)


class PagePool:
    """Pages first..n-1 of a group's pool (pages below ``first`` are never handed out)."""

    def __init__(self, n: int, first: int = 1):
        self.n = n
        self.first = first
        self._free = list(range(n - 1, first - 1, -1))
        self._held = set()

    def alloc(self, count: int) -> list:
        if count > len(self._free):
            raise CacheError(f"the cache is full: {count} pages wanted, {len(self._free)} of "
                             f"{self.n - self.first} free")
        out = [self._free.pop() for _ in range(count)]
        self._held.update(out)
        return out

    def free(self, pages) -> None:
        for p in pages:
            if p not in self._held:
                raise CacheError(f"page {p} is not held (freed twice or never allocated)")
            self._held.remove(p)
            self._free.append(p)
        self._free.sort(reverse=True)

    @property
    def n_free(self) -> int:
        return len(self._free)

    def held(self) -> set:
        return set(self._held)
