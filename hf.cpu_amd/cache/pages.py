"""A pool of fixed-size pages: ids on a free stack, with the books kept so that a page
can be neither lost, handed out twice, nor given back more often than it is held. A page
may have several holders (a prefix shared by the forks of a request, src/model.c:271-301);
it returns to the stack when the last one lets go."""
from ..status import EINVAL, ENOMEM, EngineError, fail


class OutOfPages(EngineError):
    """The pool cannot give as many pages as were asked for."""

    def __init__(self, msg):
        super().__init__(ENOMEM, msg)


class PagePool:
    def __init__(self, n_pages):
        if n_pages <= 0:
            fail(EINVAL, f"a page pool needs at least one page, got {n_pages}")
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))      # stack: lowest id on top
        self._held = [0] * n_pages                          # holders per page
        self._used_before = bytearray(n_pages)
        self.high_water = 0
        self.reused = 0          # hand-outs of a page that had been held before

    @property
    def n_free(self):
        return len(self._free)

    @property
    def n_held(self):
        return self.n_pages - len(self._free)

    def take(self, count):
        """``count`` page ids, all or none."""
        if count > len(self._free):
            raise OutOfPages(f"{count} pages wanted, {len(self._free)} of {self.n_pages} free")
        out = []
        for _ in range(count):
            p = self._free.pop()
            assert not self._held[p], f"page {p} was on the free stack while held"
            self._held[p] = 1
            if self._used_before[p]:
                self.reused += 1
            self._used_before[p] = 1
            out.append(p)
        self.high_water = max(self.high_water, self.n_held)
        return out

    def share(self, pages):
        """One more holder for each of ``pages``."""
        for p in pages:
            if not 0 <= p < self.n_pages or not self._held[p]:
                fail(EINVAL, f"page {p} is shared but is not held")
        for p in pages:
            self._held[p] += 1

    def holders(self, page):
        return self._held[page]

    def give_back(self, pages):
        for p in pages:
            if not 0 <= p < self.n_pages or not self._held[p]:
                fail(EINVAL, f"page {p} is given back but is not held")
            self._held[p] -= 1
            if not self._held[p]:
                self._free.append(p)

    def check(self):
        """Raises AssertionError if the books do not balance."""
        assert len(set(self._free)) == len(self._free), "a page is on the free stack twice"
        assert all(not self._held[p] for p in self._free), "a free page is marked held"
        assert sum(1 for h in self._held if h) + len(self._free) == self.n_pages, "a page is lost"
