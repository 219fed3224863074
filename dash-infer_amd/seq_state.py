"""Cache and state manager of the sequence engine: state slots, paged span caches, recurrent state.

A live request holds ONE slot.  Per slot the manager keeps
  * its length and its last token (host side: the embedding of the next token may depend on it),
  * for every paged cache (one per layer that writes one): a row of span pointers -- pages of `span_len` positions taken
    from a shared free list as the request grows and given back when it ends (the span pools are ops.SpanPool, the
    pointer tables have the layout dihip_kv_append / the attention kernels read: [slots][max_spans] device int64),
  * for every recurrent layer: named f32 state tensors [slots, ...] that start at zero when the slot is taken.
Pages and slots are reused in FIFO order, so a request rarely gets back what it just freed.
"""
from collections import deque

import torch

from . import ops


class SpanTable:
    """Span pointers of one paged cache: rows of `row_elems` elements of `dtype`, span_len positions per span."""

    def __init__(self, num_spans, slots, max_spans, span_len, row_elems, dtype, device):
        esz = torch.empty(0, dtype=dtype).element_size()
        self.pool = ops.SpanPool(num_spans, 1, span_len, row_elems, "none", dtype, device, nbytes=span_len * row_elems * esz)
        self.span_len, self.row_elems, self.dtype, self.max_spans = span_len, row_elems, dtype, max_spans
        self.host = torch.zeros(slots, max_spans, dtype=torch.int64, pin_memory=torch.cuda.is_available())
        self.ptrs = torch.zeros(slots, max_spans, dtype=torch.int64, device=device)

    def bind(self, slot, k, page):
        self.host[slot, k] = self.pool.span_ptr(page)

    def upload(self):
        self.ptrs.copy_(self.host, non_blocking=True)

    def rows(self, slot, pages, n):
        """the first n cached rows of a slot as a [n, row_elems] tensor (tests, diagnostics)"""
        out = []
        for k, p in enumerate(pages):
            v = self.pool.span_view(p).view(self.dtype).view(self.span_len, self.row_elems)
            out.append(v[: max(0, min(self.span_len, n - k * self.span_len))])
        return torch.cat(out) if out else torch.empty(0, self.row_elems, dtype=self.dtype)


class Slot:
    __slots__ = ("index", "length", "last_token", "pages")

    def __init__(self, index):
        self.index, self.length, self.last_token, self.pages = index, 0, None, []


class SequenceStateManager:
    def __init__(self, max_tokens, max_slots, span_len=64, device="cuda"):
        self.span_len, self.device = int(span_len), device
        self.num_pages = (int(max_tokens) + self.span_len - 1) // self.span_len
        self.max_slots = int(max_slots)
        self.free_pages = deque(range(self.num_pages))
        self.free_slots = deque(range(self.max_slots))
        self.live = {}
        self.tables = {}    # key -> SpanTable
        self.states = {}    # key -> f32 tensor [slots, ...]
        self._dirty = False

    # -- what the layers register at load ---------------------------------------------------------------------------
    def add_span_cache(self, key, row_elems, dtype):
        self.tables[key] = SpanTable(self.num_pages, self.max_slots, self.num_pages, self.span_len, row_elems, dtype, self.device)
        return self.tables[key]

    def add_state(self, key, shape):
        self.states[key] = torch.zeros(self.max_slots, *shape, dtype=torch.float32, device=self.device)
        return self.states[key]

    # -- requests ---------------------------------------------------------------------------------------------------
    def can_admit(self, tokens=0):
        return bool(self.free_slots) and self.pages_for(tokens) <= len(self.free_pages)

    def pages_for(self, tokens):
        return (tokens + self.span_len - 1) // self.span_len

    def admit(self, rid):
        if rid in self.live:
            raise KeyError(f"request {rid!r} is live already")
        if not self.free_slots:
            raise RuntimeError("no free state slot")
        s = Slot(self.free_slots.popleft())
        for st in self.states.values():
            st[s.index].zero_()
        self.live[rid] = s
        return s

    def reserve(self, rid, new_length):
        """pages for positions < new_length"""
        s = self.live[rid]
        need = self.pages_for(new_length)
        if need - len(s.pages) > len(self.free_pages):
            raise RuntimeError(f"the cache pool is exhausted ({self.num_pages} pages of {self.span_len} positions)")
        while len(s.pages) < need:
            p = self.free_pages.popleft()
            for t in self.tables.values():
                t.bind(s.index, len(s.pages), p)
            s.pages.append(p)
            self._dirty = True
        return s

    def upload(self):
        if self._dirty:
            for t in self.tables.values():
                t.upload()
            self._dirty = False

    def release(self, rid):
        s = self.live.pop(rid)
        self.free_pages.extend(s.pages)
        self.free_slots.append(s.index)
        s.pages = []

    def used_pages(self):
        return self.num_pages - len(self.free_pages)
