"""Paged cache with sequence slots.

One page id space serves every layer: page p is rows [p * page, (p + 1) * page) of each layer's pool, and a pool's rows are as
wide as that layer's cached state per token (layers may differ).  A live sequence owns a slot (a row of the block table) and
the pages its tokens fill; both go back to the free lists when it ends and are handed out again, most recently freed first.
"""
import torch


class CacheFull(RuntimeError):
    pass


class PagedCache:
    def __init__(self, row_widths, num_pages, max_seqs, dtype, device, page=64):
        if num_pages <= 0 or max_seqs <= 0:
            raise ValueError("the cache needs at least one page and one slot")
        self.page, self.num_pages, self.max_seqs = page, int(num_pages), int(max_seqs)
        self.pools = [torch.zeros((self.num_pages * page, w), dtype=dtype, device=device) for w in row_widths]
        self.free_pages = list(range(self.num_pages - 1, -1, -1))      # pop() -> lowest id first; freed pages are reused first
        self.free_slots = list(range(self.max_seqs - 1, -1, -1))
        self.pages = {}                                                # slot -> [page ids]
        self.length = {}                                               # slot -> tokens held
        self.table_host = torch.zeros((self.max_seqs, self.num_pages), dtype=torch.int32)
        self.table = self.table_host.to(device)
        self._dirty = False

    def pages_for(self, tokens):
        return (tokens + self.page - 1) // self.page

    def admit(self):
        if not self.free_slots:
            raise CacheFull(f"all {self.max_seqs} sequence slots are in use")
        s = self.free_slots.pop()
        self.pages[s], self.length[s] = [], 0
        return s

    def extend(self, slot, n):
        """Make room for n more tokens of `slot`; returns their flat row indices (position order)."""
        have, start = self.pages[slot], self.length[slot]
        need = self.pages_for(start + n) - len(have)
        if need > len(self.free_pages):
            raise CacheFull(f"{need} more pages needed, {len(self.free_pages)} free of {self.num_pages}")
        for _ in range(need):
            p = self.free_pages.pop()
            self.table_host[slot, len(have)] = p
            have.append(p)
            self._dirty = True
        self.length[slot] = start + n
        return [have[j // self.page] * self.page + j % self.page for j in range(start, start + n)]

    def release(self, slot):
        self.free_pages.extend(reversed(self.pages.pop(slot)))
        del self.length[slot]
        self.free_slots.append(slot)

    def block_table(self):
        """The device copy of the block table, uploaded if pages were handed out since the last call."""
        if self._dirty:
            self.table.copy_(self.table_host)
            self._dirty = False
        return self.table
