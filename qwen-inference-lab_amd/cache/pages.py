"""Host-side bookkeeping of one pool of pages: free list, block tables, credits.

A pool serves one *group* of schedule entries with the same need.  A page id is
valid in every entry of the group (one table indexes all its layers, as the
reference's single table does for all layers, qil/cache.py:47,79-82).

Admission reserves credits for a request's whole life, so partial prefills can
never exhaust the pool and deadlock (qil/cache.py:1-5,54-68); physical pages are
taken only as tokens are computed (qil/cache.py:70-77) and go back FIFO
(qil/cache.py:43,77,184).  A windowed pool also gives pages back as soon as the
window has passed them.
"""
from collections import deque


class CacheFull(RuntimeError):
    """No free page although one was needed."""


class PagePool:
    def __init__(self, *, num_pages, page_size, window=None, max_step_tokens=None):
        if type(num_pages) is not int or num_pages < 1 or type(page_size) is not int or page_size < 1:
            raise ValueError('num_pages and page_size must be positive integers')
        if window is not None and (type(window) is not int or window < 1):
            raise ValueError('window must be a positive integer or None')
        self.capacity, self.page_size, self.window = num_pages, page_size, window
        self.max_step_tokens = max_step_tokens
        self.free = deque(range(num_pages))
        self.tables = {}        # request -> list of page ids by logical block (-1: given back)
        self.first_live = {}    # request -> first logical block still held
        self.credits = {}       # request -> reserved pages (0 for unreserved admission)

    def pages_for(self, tokens):
        return (tokens + self.page_size - 1) // self.page_size

    def reservation_for(self, tokens):
        """Pages a request of ``tokens`` cached tokens can hold at any one time."""
        whole = self.pages_for(tokens)
        if self.window is None or self.max_step_tokens is None:
            return whole
        # live span of a step: window - 1 old keys + the step's tokens, not block aligned
        return min(whole, self.pages_for(self.window - 1 + self.max_step_tokens) + 1)

    @property
    def unreserved(self):
        return self.capacity - sum(self.credits.values())

    def can_admit(self, tokens):
        return tokens is None or self.reservation_for(tokens) <= self.unreserved

    def admit(self, request, tokens):
        if request in self.tables:
            raise ValueError('duplicate cache owner')
        self.tables[request] = []
        self.first_live[request] = 0
        self.credits[request] = 0 if tokens is None else self.reservation_for(tokens)

    def ensure(self, request, end):
        """Hold pages for positions [.., end).  All-or-nothing."""
        table = self.tables[request]
        needed = self.pages_for(end) - len(table)
        if needed > len(self.free):
            raise CacheFull(f'{needed} pages needed, {len(self.free)} free')
        for _ in range(max(0, needed)):
            table.append(self.free.popleft())

    def pass_window(self, request, computed):
        """Give back blocks no later query can see: all their keys j satisfy
        j <= p - window for every position p >= computed."""
        if self.window is None:
            return
        table = self.tables[request]
        horizon = computed - self.window + 1          # smallest key index still visible
        block = self.first_live[request]
        while block < len(table) and (block + 1) * self.page_size <= horizon:
            self.free.append(table[block])
            table[block] = -1
            block += 1
        self.first_live[request] = block

    def release(self, request):
        if request not in self.tables:
            raise ValueError('unknown cache owner')
        self.free.extend(page for page in self.tables.pop(request) if page >= 0)
        del self.first_live[request], self.credits[request]

    def held(self, request):
        return [page for page in self.tables[request] if page >= 0]

    def check(self):
        """Every page is free or held by exactly one request, none twice."""
        held = [page for request in self.tables for page in self.held(request)]
        everything = sorted(list(self.free) + held)
        if everything != list(range(self.capacity)):
            raise AssertionError(f'page accounting broken: free {sorted(self.free)}, held {sorted(held)}')
        for request, credit in self.credits.items():
            if credit and len(self.held(request)) > credit:
                raise AssertionError(f'request {request!r} holds more pages than it reserved')
