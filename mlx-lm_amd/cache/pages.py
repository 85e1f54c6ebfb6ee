"""A pool of page numbers with a LIFO free list."""


class PagePool:
    """Hands out page numbers ``0 .. n_pages-1`` and takes them back.

    The free list is last-in first-out, so a page that was just given back is
    the next one handed out: with few pages, pages really are used again.
    Giving back a page that is not held, or twice, is an error.
    """

    def __init__(self, n_pages):
        if n_pages <= 0:
            raise ValueError(f"a pool needs at least one page, got {n_pages}")
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))  # page 0 comes out first
        self._held = [False] * n_pages
        self.high_water = 0

    @property
    def n_free(self):
        return len(self._free)

    @property
    def n_held(self):
        return self.n_pages - len(self._free)

    def take(self, n):
        """``n`` pages, or ``None`` (and nothing taken) if fewer are free."""
        if n < 0:
            raise ValueError("cannot take a negative number of pages")
        if n > len(self._free):
            return None
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._held[p] = True
        self.high_water = max(self.high_water, self.n_held)
        return pages

    def give_back(self, pages):
        for p in pages:
            if not (0 <= p < self.n_pages):
                raise ValueError(f"page {p} is not of this pool")
            if not self._held[p]:
                raise ValueError(f"page {p} given back but not held")
            self._held[p] = False
            self._free.append(p)

    def check(self):
        """Every page is either free or held, exactly once."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise AssertionError("a page is on the free list twice")
        for p in range(self.n_pages):
            if self._held[p] == (p in free):
                raise AssertionError(f"page {p} is {'both held and free' if self._held[p] else 'lost'}")
