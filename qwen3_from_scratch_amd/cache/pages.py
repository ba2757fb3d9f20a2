"""Page accounting on the host: a pool of page numbers, and what each request holds."""


class OutOfPages(RuntimeError):
    """A request cannot grow because its group's pool is empty."""


class PagePool:
    """A fixed set of page numbers. Pages are handed out from a stack, so the
    page freed last is used again first."""

    def __init__(self, num_pages):
        if num_pages < 0:
            raise ValueError("a pool cannot have %d pages" % num_pages)
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages

    @property
    def num_free(self):
        return len(self._free)

    def take(self):
        if not self._free:
            raise OutOfPages("the page pool is empty")
        page = self._free.pop()
        self._held[page] = True
        return page

    def give(self, page):
        if not (0 <= page < self.num_pages) or not self._held[page]:
            raise RuntimeError("page %r is given back but is not held" % (page,))
        self._held[page] = False
        self._free.append(page)

    def is_held(self, page):
        return self._held[page]
