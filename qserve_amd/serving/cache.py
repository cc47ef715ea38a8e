"""Paged cache with sequence slots, and the fixed-size state of a sequence.

One page id space serves every layer: page p is rows [p * page, (p + 1) * page) of each layer's pool, and a pool's rows are as
wide as that layer's cached state per token (layers may differ; a width (n, w) makes n pools of one allocation, [n, rows, w]:
the key / value heads of one attention layer; (n, w, r) gives a page r rows instead of `page`: state kept per block of B
positions with r = ceil(page / B), the block that starts in page p at offset o owning row p r + o // B).  A live sequence owns a slot (a row of the block table) and the pages its
tokens fill; both go back to the free lists when it ends and are handed out again, most recently freed first.

State that does not grow with the sequence (a recurrent matrix, the last inputs of a short convolution, the previous token of
a token shift) lives in per-slot tensors, one per `StateSpec`:
* copies = 1: row `slot`.  One workgroup reads it, runs the sequence's tokens of the step, and writes it back.
* copies = 2: rows 2 slot + {0, 1}, read from one and written to the other, swapped every step the sequence takes part in
  (`step_rows`).  For state that the step's FIRST token reads and its LAST token writes from different workgroups.
A sequence's state is never cleared: kernels take a run that starts at position 0 as starting from zeros.
"""
import torch


class CacheFull(RuntimeError):
    pass


class StateSpec:
    """Per-sequence state of fixed size: `shape` per sequence, float unless `dtype` says otherwise; copies: see the module."""

    def __init__(self, shape, dtype=torch.float32, copies=1):
        if copies not in (1, 2):
            raise ValueError("a state has one copy or two")
        self.shape, self.dtype, self.copies = tuple(int(n) for n in shape), dtype, copies


class PagedCache:
    def __init__(self, row_widths, num_pages, max_seqs, dtype, device, page=64, states=()):
        if num_pages <= 0 or max_seqs <= 0:
            raise ValueError("the cache needs at least one page and one slot")
        self.page, self.num_pages, self.max_seqs = page, int(num_pages), int(max_seqs)
        rows = self.num_pages * page
        self.pools = []
        for w in row_widths:
            if isinstance(w, int):
                shape = (rows, w)
            else:
                if len(w) > 2 and not 0 < int(w[2]) <= page:
                    raise ValueError(f"a page of {page} positions cannot hold {w[2]} block rows")
                shape = (int(w[0]), self.num_pages * int(w[2]) if len(w) > 2 else rows, int(w[1]))
            self.pools.append(torch.zeros(shape, dtype=dtype, device=device))
        self.states = [torch.zeros((self.max_seqs * s.copies,) + s.shape, dtype=s.dtype, device=device) for s in states]
        self.parity = [0] * self.max_seqs
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

    def step_rows(self, slot):
        """-> (row to read, row to write) of the two-copy states for this step of `slot`; the next step reads what this one
        writes.  Call once per step and sequence."""
        p = self.parity[slot]
        self.parity[slot] = 1 - p
        return 2 * slot + p, 2 * slot + 1 - p

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
