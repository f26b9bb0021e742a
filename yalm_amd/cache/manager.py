"""The cache: a slot for each live sequence, keys and values for each cache line,
each sequence with its own length.

Storage is paged: a group owns a pool of pages of PAGE tokens; a sequence's row of
the group's block table names the pages that hold its positions.  Cache lines
(one per schedule entry that writes a cache) with the same needs form a group
and share page numbers: groups that keep all keys and groups that keep a window
have pools and tables of their own.  A windowed group keeps, per sequence, a ring
of ceil(window / PAGE) + 1 pages: position p lives in table column (p // PAGE)
% ring_pages; if it also keeps attention sinks (the first positions of a
sequence, visible behind the window), their keys and values have a place of
their own per slot, because the ring overwrites their pages.  How the elements
lie inside a page is the kernels' matter (ops.kernels.page_layout); nothing here
looks inside one.  Beside the pages there is per-sequence state of fixed size
(StateGroup) for mixers that carry one; it is cleared when a slot is acquired,
because unlike keys behind the length, stale state is not harmless.

Everything here is host bookkeeping plus device tensors; the kernels read the
block tables and lengths from the device.  The reference has one sequence and
one flat cache per layer (src/model.h:241-243, src/model.cpp:201-202,
src/infer.cpp:486-488)."""
from dataclasses import dataclass
from typing import Tuple

import numpy as np
import torch

PAGE = 64


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    pass


@dataclass(frozen=True)
class KVRequest:
    """What an attention-like mixer asks of the cache for its line."""
    n_kv_heads: int
    head_dim: int
    window: int = 0            # 0: all keys
    sinks: int = 0             # with a window: the first `sinks` positions are kept beside it


@dataclass(frozen=True)
class StateRequest:
    """Per-sequence state of fixed size for a mixer's line."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


def pages_for(n_tokens):
    return (n_tokens + PAGE - 1) // PAGE


class SlotAllocator:
    """Slots of live sequences.  A slot is held by one sequence from its first
    step to its end; freed slots are handed out again, most recently freed first."""

    def __init__(self, n_slots):
        self.n_slots = n_slots
        self._free = list(range(n_slots - 1, -1, -1))
        self._held = set()

    def acquire(self):
        if not self._free:
            raise CacheFull("all %d sequence slots are in use" % self.n_slots)
        s = self._free.pop()
        self._held.add(s)
        return s

    def release(self, slot):
        if slot not in self._held:
            raise CacheError("slot %r is released but not held" % (slot,))
        self._held.remove(slot)
        self._free.append(slot)

    def is_held(self, slot):
        return slot in self._held

    def holds_all(self, slots):
        return self._held.issuperset(slots)

    @property
    def n_free(self):
        return len(self._free)

    @property
    def held(self):
        return set(self._held)


class PagePool:
    """Page numbers of one group."""

    def __init__(self, n_pages):
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))
        self._held = set()

    def take(self):
        if not self._free:
            raise CacheFull("the cache has no free page left (%d pages)" % self.n_pages)
        p = self._free.pop()
        self._held.add(p)
        return p

    def give_back(self, page):
        if page not in self._held:
            raise CacheError("page %r is given back but not held" % (page,))
        self._held.remove(page)
        self._free.append(page)

    @property
    def n_free(self):
        return len(self._free)


class KVGroup:
    """Pages and block table of the cache lines that share one KVRequest."""

    def __init__(self, request, lines, n_pages, n_slots, max_seq_len, dtype, device):
        self.request = request
        self.lines = list(lines)                       # cache line ids, in storage order
        self.line_index = {l: i for i, l in enumerate(self.lines)}
        self.dtype = dtype
        self.window = request.window
        full_pages = max(1, pages_for(max_seq_len))
        if self.window > 0:
            self.ring_pages = min(full_pages, pages_for(self.window) + 1)
        else:
            self.ring_pages = full_pages
        self.n_pages = n_pages
        self.pool = PagePool(n_pages)
        H, hd = request.n_kv_heads, request.head_dim
        n = len(self.lines)
        # keys [line, page, head, row, element]; values transposed inside a page
        self.k_pages = torch.empty((n, n_pages, H, PAGE, hd), dtype=dtype, device=device)
        self.v_pages = torch.empty((n, n_pages, H, hd, PAGE), dtype=dtype, device=device)
        self.table_host = np.full((n_slots, self.ring_pages), -1, dtype=np.int32)
        self.table = torch.full((n_slots, self.ring_pages), -1, dtype=torch.int32, device=device)
        self._dirty = set()
        # changed rows travel through two pinned copies of the table used in turn, so that the upload is queued
        # without the host waiting for the steps still running (a copy from pageable memory would wait)
        self._staging = self._staged = None
        if torch.device(device).type == "cuda":
            self._staging = [torch.empty((n_slots, self.ring_pages), dtype=torch.int32, pin_memory=True)
                             for _ in range(2)]
            self._staged = [None, None]               # the event behind the last upload from each copy
        self._turn = 0
        self.sinks = request.sinks if self.window > 0 else 0
        # A slot's sinks need no clearing when the slot is taken again: a sink is read only once its
        # position lies behind the window, and by then the slot's present sequence has written it.
        self.sink_k = self.sink_v = None
        if self.sinks:
            self.sink_k = torch.zeros((n, n_slots, H, self.sinks, hd), dtype=dtype, device=device)
            self.sink_v = torch.zeros((n, n_slots, H, self.sinks, hd), dtype=dtype, device=device)

    def line_pages(self, line):
        i = self.line_index[line]
        return self.k_pages[i], self.v_pages[i]

    def line_sinks(self, line):
        """The line's sink keys and values, [slot, head, sink, element] each."""
        i = self.line_index[line]
        return self.sink_k[i], self.sink_v[i]

    def pages_needed(self, old_len, new_len):
        """Pages to take so that positions < new_len of a sequence of old_len have a place."""
        have = min(pages_for(old_len), self.ring_pages)
        need = min(pages_for(new_len), self.ring_pages)
        return max(0, need - have)

    def grow(self, slots, old_lens, new_lens):
        """Takes the pages that the sequences in `slots` need to grow from old_lens to new_lens.
        The sequences take their pages in turn, a page each: a batch that advances together then
        reads neighbouring pages at the same time.  (Handing every sequence a run of its own puts
        equally long prompts a power of two apart, and the attention kernel's reads, which walk
        all sequences in step, crowd into few memory channels: measured 4.8 against 5.8 TB/s.)"""
        spans = []
        for slot, old_len, new_len in zip(slots, old_lens, new_lens):
            have = min(pages_for(old_len), self.ring_pages)
            need = min(pages_for(new_len), self.ring_pages)
            if need > have:
                spans.append((slot, have, need))
        if not spans:
            return
        for col in range(min(h for _, h, _ in spans), max(n for _, _, n in spans)):
            for slot, have, need in spans:
                if have <= col < need:
                    self.table_host[slot, col] = self.pool.take()
                    self._dirty.add(slot)

    def free_slot(self, slot):
        row = self.table_host[slot]
        for col in range(self.ring_pages):
            if row[col] >= 0:
                self.pool.give_back(int(row[col]))
                row[col] = -1
        self._dirty.add(slot)

    def flush(self):
        """Sends the changed rows of the block table to the device."""
        if not self._dirty:
            return
        lo, hi = min(self._dirty), max(self._dirty) + 1
        if self._staging is None:
            self.table[lo:hi].copy_(torch.from_numpy(self.table_host[lo:hi]))
        else:
            t = self._turn
            if self._staged[t] is not None:
                self._staged[t].synchronize()         # the upload before last: long done while the host is a step ahead
            else:
                self._staged[t] = torch.cuda.Event()
            self._staging[t].numpy()[lo:hi] = self.table_host[lo:hi]
            self.table[lo:hi].copy_(self._staging[t][lo:hi], non_blocking=True)
            self._staged[t].record()
            self._turn = t ^ 1
        self._dirty.clear()

    def bytes_per_token(self):
        H, hd = self.request.n_kv_heads, self.request.head_dim
        return 2 * len(self.lines) * H * hd * self.k_pages.element_size()


class StateGroup:
    """Fixed-size per-sequence state of the cache lines that share one StateRequest:
    a tensor [line, slot, *shape]."""

    def __init__(self, request, lines, n_slots, device):
        self.request = request
        self.lines = list(lines)
        self.line_index = {l: i for i, l in enumerate(self.lines)}
        self.data = torch.zeros((len(self.lines), n_slots) + tuple(request.shape), dtype=request.dtype, device=device)

    def line_state(self, line):
        return self.data[self.line_index[line]]

    def reset(self, slot):
        self.data[:, slot].zero_()


class CacheManager:
    """Slots, pages and state for all cache lines of a model.

    requests: {cache line id: KVRequest | StateRequest | None}
    max_tokens: the most tokens live sequences hold at any time, each sequence's
    count rounded up to a multiple of PAGE."""

    def __init__(self, requests, max_tokens, max_seq_len, dtype, device, n_slots=None):
        if max_tokens <= 0:
            raise CacheError("max_tokens must be positive")
        self.device = device
        self.dtype = dtype
        self.n_pages = pages_for(max_tokens)
        self.max_seq_len = min(max_seq_len, self.n_pages * PAGE)
        self.n_slots = n_slots if n_slots is not None else min(self.n_pages, 1024)
        self.slots = SlotAllocator(self.n_slots)
        self.seq_len = [0] * self.n_slots
        by_request = {}
        for line, req in requests.items():
            if req is not None:
                by_request.setdefault(req, []).append(line)
        self.kv_groups = []
        self.state_groups = []
        self._group_of_line = {}
        for req, lines in by_request.items():
            if isinstance(req, KVRequest):
                g = KVGroup(req, sorted(lines), self.n_pages, self.n_slots, self.max_seq_len, dtype, device)
                self.kv_groups.append(g)
            elif isinstance(req, StateRequest):
                g = StateGroup(req, sorted(lines), self.n_slots, device)
                self.state_groups.append(g)
            else:
                raise CacheError("unknown cache request %r" % (req,))
            for l in lines:
                self._group_of_line[l] = g
        self.unbounded = all(g.window > 0 for g in self.kv_groups)     # no group keeps every key

    def group_of(self, line):
        return self._group_of_line.get(line)

    # ------------------------------------------------------------------ sequences
    def acquire(self, n):
        """n fresh slots (length 0, state cleared)."""
        if self.slots.n_free < n:
            raise CacheFull("%d sequences wanted, %d slots free of %d" % (n, self.slots.n_free, self.n_slots))
        out = [self.slots.acquire() for _ in range(n)]
        for s in out:
            self.seq_len[s] = 0
            for g in self.state_groups:
                g.reset(s)
        return out

    def release(self, slots):
        for s in slots:
            self.slots.release(s)
            for g in self.kv_groups:
                g.free_slot(s)
            self.seq_len[s] = 0

    def extend(self, slots, n_new):
        """Makes room for n_new[i] more tokens of slots[i] and advances the lengths.
        Nothing changes if the pages do not suffice.  Returns the new lengths."""
        if not self.slots.holds_all(slots):
            bad = [s for s in slots if not self.slots.is_held(s)]
            raise CacheError("slot %r is not held by a live sequence" % (bad[0],))
        seq_len = self.seq_len
        old_lens = [seq_len[s] for s in slots]
        new_lens = [o + n for o, n in zip(old_lens, n_new)]
        if not self.unbounded and max(new_lens) > self.max_seq_len:
            raise CacheFull("a sequence of %d tokens exceeds the longest the cache holds (%d)"
                            % (max(new_lens), self.max_seq_len))
        # only a sequence that passes a page's end can need a page, in whatever group
        growing = [i for i, (o, n) in enumerate(zip(old_lens, new_lens)) if (o + PAGE - 1) // PAGE != (n + PAGE - 1) // PAGE]
        if growing:
            g_slots = [slots[i] for i in growing]
            g_old = [old_lens[i] for i in growing]
            g_new = [new_lens[i] for i in growing]
            for g in self.kv_groups:
                need = sum(g.pages_needed(o, n) for o, n in zip(g_old, g_new))
                if need > g.pool.n_free:
                    raise CacheFull("the step needs %d more cache pages, %d are free of %d (max_tokens too small)"
                                    % (need, g.pool.n_free, g.n_pages))
            for g in self.kv_groups:
                g.grow(g_slots, g_old, g_new)
        for g in self.kv_groups:
            g.flush()
        for s, nl in zip(slots, new_lens):
            seq_len[s] = nl
        return new_lens

    def tokens_held(self):
        return sum(pages_for(self.seq_len[s]) * PAGE for s in self.slots.held)
