"""The cache manager: pages of keys and values with a block table for each request,
and slots of fixed-size state.

Layers are sorted into *groups* by what they need: every position's keys and values, or
only a window of them, with a given number of heads and head size.  A group has pages of
its own (one pool for all its layers: page ``p`` means the same tokens in each of them,
as in the reference where one block id addresses every layer,
crates/infer-worker/src/application/runtime/mod.rs:311-332) and a block table for each
request.  Pages are taken when a request's tokens first need them, given back when the
request is released or, in a windowed group, when the window has passed them, and are
handed out again without being cleared: nothing reads beyond a request's length.
The reference's page is one token (crates/infer-protocol/src/config.rs:236-238); the
partially filled last page is this engine's own.

Fixed-size state: every live request holds one slot index, valid in every state
tensor (one tensor for each layer that asks for state).  A model without such layers
still takes and returns slots, so that admission counts them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Tuple

import numpy as np
import torch

from ..parts.base import PagedKVNeed, StateNeed
from .pages import CacheError, OutOfPages, PageAllocator


def pages_for(tokens: int, page_size: int) -> int:
    return (tokens + page_size - 1) // page_size


@dataclass
class KVCacheView:
    """What an attention layer gets: its layer's slice of the group's pools."""
    k: torch.Tensor          # [num_pages, num_kv_heads, page_size, head_dim]
    v: torch.Tensor          # [num_pages, num_kv_heads, head_dim, page_size]
    group: int               # index into StepContext.block_tables
    page_size: int
    write: bool


@dataclass
class StateView:
    """What a stateful mixer gets: ``state[slot]`` is a request's state in this layer."""
    state: torch.Tensor      # [num_slots, *shape]
    write: bool


class PageGroup:
    def __init__(self, index: int, need: PagedKVNeed, cache_ids: List[int], page_size: int,
                 num_pages: int, max_model_len: int, device, dtype):
        self.index = index
        self.need = need
        self.cache_ids = list(cache_ids)
        self.page_size = page_size
        self.num_pages = num_pages
        self.max_blocks = pages_for(max_model_len, page_size)
        self.allocator = PageAllocator(num_pages)
        self.tables: Dict[Hashable, List[int]] = {}
        self._np_tables: Dict[Hashable, np.ndarray] = {}     # the same tables as int32 rows, for the step's upload
        self.k_pool = self.v_pool = None
        if device is not None:
            n, h, hd = len(cache_ids), need.num_kv_heads, need.head_dim
            self.k_pool = torch.zeros((n, num_pages, h, page_size, hd), device=device, dtype=dtype)
            # values are kept position-contiguous: the layout the attention kernels multiply from
            self.v_pool = torch.zeros((n, num_pages, h, hd, page_size), device=device, dtype=dtype)

    def table_row(self, rid) -> np.ndarray:
        """The request's table as an int32 array (a view of length len(table); do not write)."""
        return self._np_tables[rid][:len(self.tables[rid])]

    def first_needed_page(self, next_pos: int) -> int:
        """Pages below this index are no longer read once the next query is at ``next_pos``."""
        if self.need.window is None:
            return 0
        return max(0, next_pos - self.need.window + 1) // self.page_size

    def new_pages_for(self, rid, kv_len: int, n: int) -> Tuple[int, int]:
        """(pages to take, pages to give back first) for appending ``n`` tokens at ``kv_len``."""
        table = self.tables[rid]
        drop_below = self.first_needed_page(kv_len)
        give_back = sum(1 for p in table[:drop_below] if p >= 0)
        take = max(0, pages_for(kv_len + n, self.page_size) - len(table))
        return take, give_back

    def bytes_per_page(self) -> int:
        el = self.k_pool.element_size() if self.k_pool is not None else 2
        return 2 * len(self.cache_ids) * self.need.num_kv_heads * self.page_size * self.need.head_dim * el


class CacheManager:
    def __init__(self, needs: Dict[int, object], page_size: int, num_pages: int,
                 max_requests: int, max_model_len: int, device=None,
                 dtype: torch.dtype = torch.bfloat16):
        """``needs``: cache id -> PagedKVNeed | StateNeed (from ``DecoderModel.cache_needs``).
        ``num_pages`` pages go to every paged group.  ``device=None`` keeps the bookkeeping
        only (tests of the manager without a GPU)."""
        if page_size <= 0 or num_pages < 0 or max_requests <= 0:
            raise ValueError("page_size and max_requests must be > 0, num_pages >= 0")
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_model_len = max_model_len
        self.groups: List[PageGroup] = []
        self._where: Dict[int, Tuple[str, int, int]] = {}     # cache id -> (kind, group/tensor, layer slot)
        by_need: Dict[PagedKVNeed, List[int]] = {}
        self.state_tensors: Dict[int, torch.Tensor] = {}
        for cid in sorted(needs):
            need = needs[cid]
            if isinstance(need, PagedKVNeed):
                by_need.setdefault(need, []).append(cid)
            elif isinstance(need, StateNeed):
                self._where[cid] = ("state", cid, 0)
                if device is not None:
                    # one slot more than requests: the scratch slot of rows that belong to no request
                    self.state_tensors[cid] = torch.zeros((max_requests + 1,) + tuple(need.shape),
                                                          device=device, dtype=need.dtype)
            else:
                raise TypeError(f"cache {cid}: unknown need {need!r}")
        for gi, (need, cids) in enumerate(by_need.items()):
            self.groups.append(PageGroup(gi, need, cids, page_size, num_pages, max_model_len,
                                         device, dtype))
            for slot, cid in enumerate(cids):
                self._where[cid] = ("kv", gi, slot)
        self.slots = PageAllocator(max_requests, what="slots")
        # Rows of a step that belong to no request (padding of a captured batch size, the rows a
        # graph is warmed up and captured on) point here: a mixer that updates state in place may
        # write this slot at will, and no request ever reads it.
        self.scratch_slot = max_requests
        self._slot_of: Dict[Hashable, int] = {}
        self._kv_len: Dict[Hashable, int] = {}

    # -- queries -------------------------------------------------------------
    def __contains__(self, cache_id: int) -> bool:
        return cache_id in self._where

    def has_request(self, rid) -> bool:
        return rid in self._kv_len

    def live_requests(self):
        return list(self._kv_len)

    def kv_len(self, rid) -> int:
        return self._kv_len[rid]

    def slot(self, rid) -> int:
        return self._slot_of[rid]

    def free_pages(self) -> int:
        """Free pages of the tightest group."""
        return min((g.allocator.available for g in self.groups), default=1 << 30)

    def table(self, group: int, rid) -> List[int]:
        return self.groups[group].tables[rid]

    def pages_held(self, rid) -> int:
        return sum(sum(1 for p in g.tables[rid] if p >= 0) for g in self.groups)

    def view(self, cache_id: int, write: bool = True):
        kind, where, slot = self._where[cache_id]
        if kind == "kv":
            g = self.groups[where]
            return KVCacheView(g.k_pool[slot], g.v_pool[slot], g.index, g.page_size, write)
        return StateView(self.state_tensors[where], write)

    # -- life of a request -----------------------------------------------------
    def add_request(self, rid) -> int:
        if rid in self._kv_len:
            raise CacheError(f"request {rid!r} is already live")
        slot = self.slots.alloc(1)[0]
        self._slot_of[rid] = slot
        self._kv_len[rid] = 0
        for g in self.groups:
            g.tables[rid] = []
            g._np_tables[rid] = np.full(g.max_blocks, -1, dtype=np.int32)
        return slot

    def can_append(self, wants: List[Tuple[Hashable, int]]) -> bool:
        """Would ``append`` succeed for all of ``wants`` = [(request, new tokens)] together?
        Requests not yet added count from length zero and need a slot each."""
        new_requests = sum(1 for rid, _ in wants if rid not in self._kv_len)
        if new_requests > self.slots.available:
            return False
        for g in self.groups:
            balance = g.allocator.available
            for rid, n in wants:
                if rid in self._kv_len:
                    take, give = g.new_pages_for(rid, self._kv_len[rid], n)
                else:
                    take, give = pages_for(n, g.page_size), 0
                balance += give - take
                if self._kv_len.get(rid, 0) + n > self.max_model_len:
                    return False
            if balance < 0:
                return False
        return True

    def append(self, rid, n: int) -> int:
        """Make room for ``n`` more tokens of ``rid`` and return where they start.
        Windowed groups first give back the pages the window has passed.  Either every
        group gets its pages or nothing changes (``OutOfPages``)."""
        if rid not in self._kv_len:
            raise CacheError(f"request {rid!r} is not live")
        if n <= 0:
            raise ValueError("n must be > 0")
        start = self._kv_len[rid]
        if start + n > self.max_model_len:
            raise CacheError(f"request {rid!r}: {start + n} tokens exceed max_model_len {self.max_model_len}")
        for g in self.groups:
            take, give = g.new_pages_for(rid, start, n)
            if take > g.allocator.available + give:
                raise OutOfPages(take, g.allocator.available + give)
        for g in self.groups:
            table = g.tables[rid]
            drop_below = g.first_needed_page(start)
            old = [p for p in table[:drop_below] if p >= 0]
            if old:
                g.allocator.free(old)
                for i in range(min(drop_below, len(table))):
                    table[i] = -1
                g._np_tables[rid][:min(drop_below, len(table))] = -1
            take = max(0, pages_for(start + n, g.page_size) - len(table))
            if take:
                new = g.allocator.alloc(take)
                g._np_tables[rid][len(table):len(table) + take] = new
                table.extend(new)
        self._kv_len[rid] = start + n
        return start

    def truncate(self, rid, length: int) -> None:
        """Undo appends: the request is ``length`` tokens long again, and the pages beyond that
        go back.  Pages that a window had already passed when those tokens were appended stay
        given back: no query at ``length`` or later can see them.  (The reference returns a failed
        step's fresh slots the same way, crates/infer-worker/src/application/worker_scheduler.rs:1090-1133.)"""
        if rid not in self._kv_len:
            raise CacheError(f"request {rid!r} is not live")
        if not (0 <= length <= self._kv_len[rid]):
            raise CacheError(f"request {rid!r}: cannot truncate {self._kv_len[rid]} tokens to {length}")
        for g in self.groups:
            keep = pages_for(length, g.page_size)
            if any(p < 0 for p in g.tables[rid][g.first_needed_page(length):keep]):
                raise CacheError(f"request {rid!r}: a window has given back pages that a query at "
                                 f"position {length} reads; it cannot be cut back that far")
        for g in self.groups:
            table = g.tables[rid]
            keep = pages_for(length, g.page_size)
            if keep < len(table):
                g.allocator.free([p for p in table[keep:] if p >= 0])
                g._np_tables[rid][keep:len(table)] = -1
                del table[keep:]
        self._kv_len[rid] = length

    def state_bytes(self) -> int:
        """Bytes of the fixed-size state tensors (all slots of all layers that ask for state)."""
        return sum(t.numel() * t.element_size() for t in self.state_tensors.values())

    def release(self, rid) -> None:
        """The request is finished, cancelled or preempted: everything it holds goes back."""
        if rid not in self._kv_len:
            raise CacheError(f"request {rid!r} is not live")
        for g in self.groups:
            g.allocator.free([p for p in g.tables.pop(rid) if p >= 0])
            del g._np_tables[rid]
        self.slots.free([self._slot_of.pop(rid)])
        del self._kv_len[rid]

    # -- invariants (tests) ----------------------------------------------------
    def check(self) -> None:
        for g in self.groups:
            for rid, t in g.tables.items():
                if g.table_row(rid).tolist() != t:
                    raise CacheError(f"group {g.index}: the array form of request {rid!r}'s table differs")
            held = [p for t in g.tables.values() for p in t if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError(f"group {g.index}: a page is held twice")
            if len(held) != g.allocator.outstanding:
                raise CacheError(f"group {g.index}: {g.allocator.outstanding} pages out, "
                                 f"{len(held)} in tables")
            for rid, t in g.tables.items():
                want = pages_for(self._kv_len[rid], g.page_size)
                if len(t) != want:
                    raise CacheError(f"group {g.index}: request {rid!r} has {len(t)} table entries "
                                     f"for {self._kv_len[rid]} tokens")
                if g.need.window is None and any(p < 0 for p in t):
                    raise CacheError(f"group {g.index}: request {rid!r} lost a page")
        if len(self._slot_of) != self.slots.outstanding:
            raise CacheError("slot count does not match live requests")
