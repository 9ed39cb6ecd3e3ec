"""The step function: a batch of (request, its next tokens) in, logits at the wanted
places out.

A request's entry is any portion of its tokens: a slice of a prompt or one decoded
token, cut anywhere.  The step runs exactly the tokens it is given, as one batch, reading
earlier tokens from the cache, and projects onto the vocabulary only the rows that were
asked for.  Counterpart of ``Runtime::step`` (crates/infer-worker/src/application/runtime/mod.rs:561-629)
with ``build_plan`` / ``upload_index`` (crates/infer-worker/src/application/runtime/plan.rs:24-154,
:293-369); unlike it, the step returns logits, and sampling is a separate call.
"""
from __future__ import annotations

import contextlib
import gc

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.pages import CacheError, OutOfPages
from ..parts.base import Runtime
from .markers import profile_range
from .context import StepContext, Workspace


class StepError(ValueError):
    """A batch the step function cannot run (crates/infer-worker/src/application/runtime/plan.rs:24-124)."""


@dataclass
class StepEntry:
    request_id: Hashable
    tokens: Sequence[int]          # token ids; -(k+1) stands for Engine.device_tokens[k]
    want: Sequence[int] = ()       # indices among ``tokens`` whose logits are wanted


def device_token(slot: int) -> int:
    """The id that stands for ``Engine.device_tokens[slot]`` in ``StepEntry.tokens``."""
    return -1 - int(slot)


class _Staging:
    """A ring of pinned host buffers for the step's control data, so that the copy of one
    step may still be in flight while the next is written, and the one device buffer they are
    copied to.  Captured graphs hold addresses inside the device buffer, so it is allocated once,
    at the size of the largest step the engine accepts, and never replaced (the reference keeps its
    index tensors address-stable for the same reason, crates/infer-core/src/kv.rs:22-39)."""

    def __init__(self, device, ints: int, depth: int = 4):
        self.device = device
        self.depth = depth
        self.ints = int(ints)
        pin = device.type == "cuda"
        self.host = [torch.empty(self.ints, dtype=torch.int32, pin_memory=pin) for _ in range(depth)]
        self.events: List[Optional[torch.cuda.Event]] = [None] * depth
        self.dev = torch.empty(self.ints, dtype=torch.int32, device=device)
        self.turn = 0

    def next(self, ints: int):
        if ints > self.ints:
            raise StepError(f"the step's control data ({ints} words) exceeds the staging buffer "
                            f"({self.ints}): the step is larger than the engine was built for")
        i = self.turn
        self.turn = (self.turn + 1) % self.depth
        if self.events[i] is not None:
            self.events[i].synchronize()
        return i, self.host[i]

    def upload(self, i: int, ints: int) -> torch.Tensor:
        self.dev[:ints].copy_(self.host[i][:ints], non_blocking=True)
        if self.device.type == "cuda":
            ev = torch.cuda.Event()
            ev.record()
            self.events[i] = ev
        return self.dev


def pick_graph_bucket(sizes: Sequence[int], batch: int, decode_only: bool) -> int:
    """The captured batch size a step replays: the smallest one that holds the batch, for
    steps of single tokens only; 0 means the step runs eagerly
    (crates/infer-worker/src/application/runtime/graph_exec.rs:99-135; its cases :476-501:
    sizes [4, 1, 2, 2] are [1, 2, 4]; batch 3 takes 4; batch 5 and ragged batches run eagerly)."""
    if not decode_only:
        return 0
    for s in sorted(set(int(x) for x in sizes if int(x) > 0)):
        if s >= batch:
            return s
    return 0


class Engine:
    """A model, its cache and the step function over them."""

    def __init__(self, model, rt: Runtime, page_size: int, num_pages: int, max_requests: int,
                 max_model_len: int, max_batch_tokens: int = 8192):
        self.model = model
        self.rt = rt
        self.max_batch_tokens = int(max_batch_tokens)
        self.max_model_len = int(max_model_len)
        self.max_requests = int(max_requests)
        self.page_size = int(page_size)
        model.prepare(rt, max_model_len)
        self.cache = CacheManager(model.cache_needs(), page_size, num_pages, max_requests,
                                  max_model_len, device=rt.device, dtype=rt.dtype)
        self.workspace = Workspace(rt.device)
        # the largest step: max_batch_tokens tokens (or max_requests single tokens padded to a
        # captured batch size) of max_requests rows, every table at full length
        t_max = max(self.max_batch_tokens, self.max_requests)
        # (per token: id, position, row, a wanted place; per row: offset, start, length, slot, and
        # the lists of the single tokens and of the longer rows)
        self._staging = _Staging(rt.device, 4 * t_max + 6 * self.max_requests + 2
                                 + self.max_requests * sum(g.max_blocks for g in self.cache.groups))
        self.vocab_size = model.vocab_size
        self.steps_run = 0
        # tokens sampled on the device that the next step may read without the host seeing them first
        self.device_tokens = torch.zeros(max(self.max_requests, 1), dtype=torch.int32, device=rt.device)
        pin = rt.device.type == "cuda"
        self._tok_host = [torch.zeros(max(self.max_requests, 1), dtype=torch.int32, pin_memory=pin) for _ in range(4)]
        self._tok_turn = 0
        self._graph_sizes: Tuple[int, ...] = ()
        self._mixed_tokens = 0
        self._mixed_after = 1
        self._mixed_seen: Dict[tuple, int] = {}
        self._mixed_used: Dict[tuple, int] = {}      # when a graph of a step with portions last ran
        self._mixed_tick = 0
        self._graphs: Dict[tuple, object] = {}       # (rows, key bucket) or ("mixed", tokens, rows, key bucket, single-token rows)
        self.graph_replays = 0
        self.mixed_graph_replays = 0
        # What set-up left on the host's heap (modules, parts, weights' wrappers: a million
        # objects with torch loaded) is taken out of the garbage collector's view: a full
        # collection over it takes tens of milliseconds and would fall into some step.
        gc.collect()
        gc.freeze()

    # -- sizing the pool ---------------------------------------------------------------
    def profile_forward(self) -> int:
        """Run the largest step the engine accepts once, eagerly, on requests of its own that are
        released again: ``max_batch_tokens`` tokens in as few rows as ``max_model_len`` allows.
        Afterwards the workspace, the GEMM library's buffers and whatever else a step allocates
        exist, and free device memory is what the cache pool may really take (the reference sizes
        its pool after such a pass, crates/infer-worker/src/application/runtime/mod.rs:943-984,
        crates/infer-worker/src/application/serve_loop.rs:391-501).  Returns the tokens it ran."""
        left = min(self.max_batch_tokens, self.max_requests * self.max_model_len)
        gen = torch.Generator().manual_seed(0)
        entries = []
        while left > 0 and len(entries) < self.max_requests:
            n = min(left, self.max_model_len)
            ids = torch.randint(0, self.vocab_size, (n,), generator=gen).tolist()
            entries.append(StepEntry(("profile", len(entries)), ids, [n - 1]))
            left -= n
        if not entries or not self.cache.can_append([(e.request_id, len(e.tokens)) for e in entries]):
            return 0                                     # a pool too small for it: nothing to learn
        graphs, mixed = self._graph_sizes, self._mixed_tokens
        self._graph_sizes, self._mixed_tokens = (), 0
        try:
            self.step(entries)
            if self.rt.device.type == "cuda":
                torch.cuda.synchronize(self.rt.device)
        finally:
            self._graph_sizes, self._mixed_tokens = graphs, mixed
            for e in entries:
                self.release(e.request_id)
        return sum(len(e.tokens) for e in entries)

    def resize_pool(self, num_pages: int) -> None:
        """Replace the cache pool by one of ``num_pages`` pages (the reference's ``resize_kv_pool``).
        Only while no request is live and no graph has been captured: both hold its addresses."""
        if self.cache.live_requests() or self._graphs:
            raise CacheError("the pool can only be resized before requests run and graphs are captured")
        old = self.cache
        self.cache = None
        for g in old.groups:
            g.k_pool = g.v_pool = None
        old.state_tensors.clear()
        del old
        if self.rt.device.type == "cuda":
            torch.cuda.empty_cache()
        self.cache = CacheManager(self.model.cache_needs(), self.page_size, int(num_pages), self.max_requests,
                                  self.max_model_len, device=self.rt.device, dtype=self.rt.dtype)

    # -- HIP graphs for steps of single tokens ---------------------------------------
    def enable_graphs(self, on: bool = True,
                      capture_sizes: Sequence[int] = (1, 2, 4, 8, 16, 24, 32, 40, 48, 56, 64),
                      mixed_tokens: int = 0, mixed_after: int = 1) -> None:
        """Steps in which every request brings one token are captured once per (padded batch
        size, key-length bucket) and replayed: the launches of a step cost more than its
        kernels otherwise.  Padding rows are inert (no request, no cache access), as the
        reference's (graph_exec.rs:320-328).  Graphs are captured when first needed.

        ``mixed_tokens`` > 0: steps that hold prompt portions are captured too, up to that many
        tokens, per (token bucket, padded batch size, key-length bucket, bucket of the rows of one
        token), if every entry wants at
        most the logits of its last token (what a scheduler asks for).  Tokens are padded to multiples
        of 16 (the reference's mixed graphs round to 64, crates/infer-worker/src/application/runtime/mixed_abc.rs:29-37,135-180;
        here a step of 264 tokens padded to 320 took 10 % longer than launched eagerly: its products
        are no longer bound by the weights alone); padding tokens belong to no row, padding rows
        have no tokens.  At most ``MIXED_GRAPH_BUDGET`` such graphs
        are kept; beyond that, a new shape takes the place of the one that has not run for the
        longest time.  ``mixed_after``: such a
        shape is captured the n-th time it is met and runs eagerly before (a capture keeps the GPU
        idle for 20-50 ms, ten steps' worth where launches bind; a shape met once is not worth it)."""
        self._graph_sizes = tuple(sorted(set(int(c) for c in capture_sizes
                                             if 0 < int(c) <= self.max_requests))) if on else ()
        self._mixed_tokens = min(int(mixed_tokens), self.max_batch_tokens) if on else 0
        self._mixed_after = max(int(mixed_after), 1)
        self._mixed_seen: Dict[tuple, int] = {}
        if not on:
            self._graphs.clear()
            self.workspace.frozen = False

    MIXED_GRAPH_BUDGET = 128
    PORTION_DIVIDE_MIN_PREFIX = 512      # cached tokens before a portion from which its attention may divide the keys

    KV_BUCKET = 1024

    def _stream_scope(self):
        """The ops' launch stream, looked up once for a whole forward pass."""
        scope = getattr(self.rt.ops, "stream_scope", None)
        return scope() if scope is not None else contextlib.nullcontext()

    def _capture(self, bucket: int, kvb: int, tokens: int = 0, singles: int = 0, divided: int = 0):
        """Warm up and capture the forward pass for ``bucket`` single-token rows (``tokens`` = 0)
        or for a step of ``tokens`` tokens in ``bucket`` rows, over keys up to ``kvb``, on rows that
        belong to no request (``row_of_token = -1``, no cache access, the
        scratch state slot): nothing a live request holds is touched before the first replay, so a
        part that updates state in place runs once for each real token, and what a captured pass
        may depend on is the batch's shape alone (the reference warms its graphs up on dummy rows
        too, crates/infer-worker/src/application/serve_loop.rs:503-510)."""
        if tokens:
            ctx = self._build_context([], [], pad_rows_to=bucket, pad_tokens_to=tokens, want_last=True)
            ctx.max_q_len = tokens                       # an upper bound: the grid of the attention over portions
            ctx.decode_only = False
            ctx.num_single = singles                     # an upper bound too; 0: no kernel for single tokens at all
            # rows of several tokens: the rows that cannot be single ones (their number was rounded
            # up to `singles` from more than the capture size below it)
            below = max((c for c in self._graph_sizes if c < singles), default=0) if singles else -1
            ctx.num_portion = max(bucket - (below + 1), 1)
            # whether the attention over portions divides the keys between blocks is part of the shape
            ctx.portion_prefix = kvb if divided else 0
            ctx.portion_kv_len = kvb
            ctx.host_q_lens = ctx.host_q_start = ctx.host_kv_lens = ctx.host_slots = ctx.request_ids = None
        else:
            ctx = self._build_context([], [], pad_rows_to=bucket, want_all=True)
        ctx.max_kv_len = kvb
        self.workspace.frozen = False
        side = torch.cuda.Stream(self.rt.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), self._stream_scope():
            self.model.forward(ctx, self.cache)          # allocates the workspace it needs
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize(self.rt.device)
        self.workspace.frozen = True
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g), self._stream_scope():
            logits = self.model.forward(ctx, self.cache)
        return g, logits

    @staticmethod
    def mixed_token_bucket(tokens: int) -> int:
        """The padded token count of a captured step with prompt portions."""
        return -(-tokens // 16) * 16

    def _mixed_graph_key(self, entries) -> Optional[Tuple[int, int, int]]:
        """(token bucket, row bucket, bucket of the rows of one token) if this step may replay a graph
        of steps with prompt portions."""
        if not self._mixed_tokens:
            return None
        T = 0
        for e in entries:
            n = len(e.tokens)
            T += n
            if len(e.want) > 1 or (len(e.want) == 1 and int(e.want[0]) != n - 1):
                return None                              # logits inside a portion: the general path
        if T > self._mixed_tokens:
            return None
        Tp = self.mixed_token_bucket(T)
        rows = next((c for c in self._graph_sizes if c >= len(entries)), None)
        if rows is None or Tp > max(self.max_batch_tokens, self.max_requests):
            return None
        singles = sum(1 for e in entries if len(e.tokens) == 1)
        if singles:                                      # rounded up as the rows are: it steers the split of the keys
            singles = next(c for c in self._graph_sizes if c >= singles)
        return Tp, rows, singles

    def capture_graphs(self, rows: Sequence[int], kv_len: int) -> int:
        """Capture now what steps of ``rows`` single tokens over up to ``kv_len`` keys would capture
        when they first run (the reference captures its sizes at start-up,
        crates/infer-worker/src/application/runtime/graph_exec.rs:305-397).  Returns the number of
        graphs captured.  A capture keeps the host busy and the GPU idle for some 20 ms; done ahead,
        it does not fall between a prompt and its first tokens."""
        if not self._graph_sizes or not getattr(self.model, "graph_safe", True):
            return 0
        kvb = min(-(-max(1, int(kv_len)) // self.KV_BUCKET) * self.KV_BUCKET, self.max_model_len)
        made = 0
        for n in rows:
            bucket = next((c for c in self._graph_sizes if c >= n), None)
            if bucket is not None and (bucket, kvb) not in self._graphs:
                self._graphs[(bucket, kvb)] = self._capture(bucket, kvb)
                made += 1
        return made

    def prewarm_graphs(self) -> int:
        """Capture, before any request runs, the graph of every capture size at every key-length
        bucket up to the longest request (the reference primes all its sizes at start-up,
        crates/infer-worker/src/application/runtime/graph_exec.rs:149-247).  Returns how many were
        captured.  Graphs of steps with prompt portions are still captured when first met: there
        are too many shapes of them to make ahead."""
        made = 0
        for kv in range(self.KV_BUCKET, self.max_model_len + self.KV_BUCKET, self.KV_BUCKET):
            made += self.capture_graphs(self._graph_sizes, min(kv, self.max_model_len))
        return made

    def _graph_step(self, entries, starts, bucket: int) -> torch.Tensor:
        B = len(entries)
        longest = max(s + 1 for s in starts)
        kvb = min(-(-longest // self.KV_BUCKET) * self.KV_BUCKET, self.max_model_len)
        key = (bucket, kvb)
        graph = self._graphs.get(key)
        if graph is None:
            graph = self._graphs[key] = self._capture(bucket, kvb)
        # the control data of the real rows goes where the captured kernels read it: the layout
        # in the staging buffer is a function of the bucket alone
        self._build_context(entries, starts, pad_rows_to=bucket, want_all=True)
        g, logits = graph
        g.replay()
        self.graph_replays += 1
        wanted = [i for i, e in enumerate(entries) if len(e.want)]
        if len(wanted) == B:
            return logits[:B]
        return logits[torch.tensor(wanted, dtype=torch.long, device=logits.device)]

    def _mixed_graph_step(self, entries, starts, key) -> Optional[torch.Tensor]:
        """Replay (capturing first if need be) the graph for a step with prompt portions; None if
        this shape has none and has not been met often enough to be given one."""
        Tp, rows, singles = key
        longest = max(s + len(e.tokens) for s, e in zip(starts, entries))
        kvb = min(-(-longest // self.KV_BUCKET) * self.KV_BUCKET, self.max_model_len)
        # a portion behind many cached keys has them divided between blocks (a kernel more): the
        # captured step says so, or a prompt's first portion beside long requests would pay for it
        prefix = max((s for s, e in zip(starts, entries) if len(e.tokens) > 1), default=0)
        divided = 1 if prefix >= self.PORTION_DIVIDE_MIN_PREFIX else 0
        gkey = ("mixed", Tp, rows, kvb, singles, divided)
        graph = self._graphs.get(gkey)
        if graph is None:
            if self._mixed_after > 1:
                if len(self._mixed_seen) > 4096:
                    self._mixed_seen.clear()
                seen = self._mixed_seen[gkey] = self._mixed_seen.get(gkey, 0) + 1
                if seen < self._mixed_after:
                    return None                          # not met often enough yet: eagerly
            held = [k for k in self._graphs if k[0] == "mixed"]
            if len(held) >= self.MIXED_GRAPH_BUDGET:
                # the budget is spent: the shape that has not run for the longest time makes room
                oldest = min(held, key=lambda k: self._mixed_used.get(k, 0))
                torch.cuda.synchronize(self.rt.device)   # its last replay may still be running
                del self._graphs[oldest]
                self._mixed_used.pop(oldest, None)
                self._mixed_seen.pop(oldest, None)
            graph = self._graphs[gkey] = self._capture(rows, kvb, tokens=Tp, singles=singles, divided=divided)
        self._mixed_tick += 1
        self._mixed_used[gkey] = self._mixed_tick
        self._build_context(entries, starts, pad_rows_to=rows, pad_tokens_to=Tp, want_last=True)
        g, logits = graph
        g.replay()
        self.graph_replays += 1
        self.mixed_graph_replays += 1
        wanted = [i for i, e in enumerate(entries) if len(e.want)]
        if len(wanted) == rows:
            return logits
        if not wanted:
            return logits[:0]
        if wanted == list(range(len(wanted))):
            return logits[:len(wanted)]
        return logits[torch.tensor(wanted, dtype=torch.long, device=logits.device)]

    # -- tokens that stay on the device ---------------------------------------------
    def synchronize(self) -> None:
        """Wait for everything queued on the engine's device."""
        torch.cuda.synchronize(self.rt.device)

    def read_device_tokens(self, n: int):
        """Start copying ``device_tokens[:n]`` to the host; returns ``(pinned tensor, event)``.
        The copy is ordered after everything queued so far, so later steps may overwrite the
        device buffer."""
        i = self._tok_turn
        self._tok_turn = (i + 1) % len(self._tok_host)
        host = self._tok_host[i]
        host[:n].copy_(self.device_tokens[:n], non_blocking=True)
        ev = torch.cuda.Event() if self.rt.device.type == "cuda" else None
        if ev is not None:
            ev.record()
        return host[:n], ev

    # -- requests --------------------------------------------------------------
    def release(self, request_id) -> None:
        """Give back everything a request holds (finished, cancelled or preempted)."""
        if self.cache.has_request(request_id):
            self.cache.release(request_id)

    # -- the step -----------------------------------------------------------------
    def validate(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise StepError("empty batch")
        if len(entries) > self.max_requests:
            raise StepError(f"{len(entries)} rows exceed max_requests {self.max_requests}")
        seen = set()
        total = 0
        V = self.vocab_size
        for e in entries:
            if e.request_id in seen:
                raise StepError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request_id!r}: no tokens")
            total += n
            # -(k+1) refers to device_tokens[k]; only a request's newest token can still be on
            # the device, so only the last token of an entry may be such a reference
            last = int(e.tokens[-1])
            if not (-self.max_requests <= last < V):
                raise StepError(f"request {e.request_id!r}: token id {last} outside [0, {V}) "
                                f"and no device token [-{self.max_requests}, -1]")
            if n > 1:
                arr = np.asarray(e.tokens[:-1])
                if arr.min() < 0 or arr.max() >= V:
                    bad = int(arr[(arr < 0) | (arr >= V)][0])
                    raise StepError(f"request {e.request_id!r}: token id {bad} outside [0, {V}) "
                                    f"(a device token may only be an entry's last)")
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise StepError(f"request {e.request_id!r}: wanted place {w} outside its {n} tokens")
            have = self.cache.kv_len(e.request_id) if self.cache.has_request(e.request_id) else 0
            if have + n > self.max_model_len:
                raise StepError(f"request {e.request_id!r}: {have + n} tokens exceed max_model_len {self.max_model_len}")
        if total > self.max_batch_tokens:
            raise StepError(f"{total} tokens exceed max_batch_tokens {self.max_batch_tokens}")

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run one batch; returns 32-bit logits ``[wanted, vocab]`` on the device, rows in the
        order of the entries and of each entry's ``want``.  The tensor is scratch that the next
        step overwrites.  Raises ``OutOfPages`` (nothing changed) if the cache cannot hold it.
        If the forward pass raises, every request is as long as it was before the step, its
        fixed-size state is what it was (eager steps copy the slots they touch first; a replayed
        graph either runs whole or not at all), requests
        the step started are gone, and the pages taken are free again (the reference gives a failed
        step's fresh slots back, crates/infer-worker/src/application/worker_scheduler.rs:1090-1133;
        its leases must be consumed or returned, crates/infer-worker/src/domain/global_kv_alloc.rs:393-461)."""
        self.validate(entries)
        cache = self.cache
        if not cache.can_append([(e.request_id, len(e.tokens)) for e in entries]):
            raise OutOfPages(sum(len(e.tokens) for e in entries), cache.free_pages() * cache.page_size,
                             "pages (in tokens)")
        taken: List[Tuple[Hashable, Optional[int]]] = []     # (request, its length before; None: new)
        saved_state = None
        try:
            starts = []
            for e in entries:
                if cache.has_request(e.request_id):
                    taken.append((e.request_id, cache.kv_len(e.request_id)))
                else:
                    cache.add_request(e.request_id)
                    taken.append((e.request_id, None))
                starts.append(cache.append(e.request_id, len(e.tokens)))
            self.steps_run += 1
            if self._graph_sizes and getattr(self.model, "graph_safe", True):
                bucket = pick_graph_bucket(self._graph_sizes, len(entries),
                                           all(len(e.tokens) == 1 for e in entries))
                if bucket:
                    with profile_range(f"step graph rows={len(entries)} bucket={bucket}"):
                        return self._graph_step(entries, starts, bucket)
                key = self._mixed_graph_key(entries)
                if key is not None:
                    with profile_range(f"step mixed graph rows={len(entries)} tokens={key[0]}"):
                        out = self._mixed_graph_step(entries, starts, key)
                    if out is not None:
                        return out
            with profile_range(f"step eager rows={len(entries)} tokens={sum(len(e.tokens) for e in entries)}"):
                with profile_range("context"):
                    ctx = self._build_context(entries, starts)
                if cache.state_tensors:
                    # fixed-size state is updated in place by the layers that own it: the slots of the
                    # step's requests are copied first, so that a step that fails half-way can be undone
                    slots = torch.tensor([cache.slot(e.request_id) for e in entries], dtype=torch.long,
                                         device=self.rt.device)
                    saved_state = (slots, {cid: t.index_select(0, slots) for cid, t in cache.state_tensors.items()})
                with profile_range("forward"), self._stream_scope():
                    return self.model.forward(ctx, cache)
        except BaseException:
            if saved_state is not None:
                slots, copies = saved_state
                for cid, copy in copies.items():
                    cache.state_tensors[cid].index_copy_(0, slots, copy)
            for rid, before in reversed(taken):
                if before is None:
                    cache.release(rid)
                else:
                    cache.truncate(rid, before)
            raise

    def _build_context(self, entries: Sequence[StepEntry], starts: List[int],
                       pad_rows_to: int = 0, want_all: bool = False,
                       pad_tokens_to: int = 0, want_last: bool = False) -> StepContext:
        """The step's control data, written to the staging buffer and copied to the device.
        ``pad_rows_to`` alone: a step of single tokens padded to a captured batch size, a padding
        token for each padding row.  With ``pad_tokens_to``: a step with portions padded to a
        captured shape; padding tokens belong to no row (``row_of_token = -1``) and padding rows
        have no tokens.  ``want_last``: one wanted place a row, the row's last token (token 0 for
        rows that want nothing or have no tokens; the caller drops those logits)."""
        cache = self.cache
        B = len(entries)
        q_lens = [len(e.tokens) for e in entries]
        T = sum(q_lens)
        want_rows: List[int] = []
        off = 0
        for e, q in zip(entries, q_lens):
            if want_last:
                want_rows.append(off + q - 1 if len(e.want) else 0)
            else:
                want_rows.extend(off + int(w) for w in e.want)
            off += q
        Bp = max(B, pad_rows_to)       # rows incl. inert padding
        Tp = max(T, pad_tokens_to) if pad_tokens_to else T + (Bp - B)
        if want_last:
            want_rows.extend([0] * (Bp - B))
        if want_all:
            want_rows = list(range(Tp))
        W = len(want_rows)
        in_order = W == Tp and all(w == i for i, w in enumerate(want_rows))
        groups = cache.groups
        sizes = [Tp, Tp, Tp, Bp + 1, Bp, Bp, Bp, max(W, 1), Bp, Bp] + [Bp * g.max_blocks for g in groups]
        offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        total = int(offs[-1])
        turn, host = self._staging.next(total)
        h = host.numpy()
        h[:total] = 0
        ids, pos, row = (h[offs[i]:offs[i + 1]] for i in range(3))
        cu, qs, kvl, slots, want, single, longer = (h[offs[i]:offs[i + 1]] for i in range(3, 10))
        single[:] = -1
        longer[:] = -1
        if T == B:                       # one token per row: no per-row slices needed
            ids[:B] = [e.tokens[0] for e in entries]
            pos[:B] = starts
            row[:B] = np.arange(B, dtype=np.int32)
            cu[:B] = row[:B]
            qs[:B] = starts
            kvl[:B] = pos[:B] + 1
            slots[:B] = [cache.slot(e.request_id) for e in entries]
        else:
            t = n_single = n_longer = 0
            for b, (e, q, s) in enumerate(zip(entries, q_lens, starts)):
                ids[t:t + q] = np.asarray(e.tokens, dtype=np.int32)
                pos[t:t + q] = np.arange(s, s + q, dtype=np.int32)
                row[t:t + q] = b
                cu[b] = t
                qs[b] = s
                kvl[b] = s + q
                slots[b] = cache.slot(e.request_id)
                if q == 1:               # the tokens of rows of one token, for the kernels that take only those
                    single[n_single] = t
                    n_single += 1
                elif q > 1:              # and the rows of several
                    longer[n_longer] = b
                    n_longer += 1
                t += q
        cu[B:] = T
        row[T:] = -1
        slots[B:] = cache.scratch_slot
        want[:W] = want_rows
        for gi, g in enumerate(groups):
            bt = h[offs[10 + gi]:offs[11 + gi]].reshape(Bp, g.max_blocks)
            for b, e in enumerate(entries):
                row_ = g.table_row(e.request_id)
                bt[b, :row_.shape[0]] = row_
        dev = self._staging.upload(turn, total)
        ctx = StepContext()
        ctx.num_tokens, ctx.num_rows, ctx.num_want = Tp, Bp, W
        ctx.token_ids, ctx.positions, ctx.row_of_token = (dev[offs[i]:offs[i + 1]] for i in range(3))
        ctx.cu_q, ctx.q_start, ctx.kv_lens, ctx.state_slots = (dev[offs[i]:offs[i + 1]] for i in range(3, 7))
        ctx.want_rows = dev[offs[7]:offs[7] + W]
        ctx.single_tokens = dev[offs[8]:offs[9]]
        ctx.portion_rows = dev[offs[9]:offs[10]]
        ctx.block_tables = [dev[offs[10 + gi]:offs[11 + gi]].view(Bp, g.max_blocks)
                            for gi, g in enumerate(groups)]
        ctx.workspace = self.workspace
        ctx.device_tokens = self.device_tokens
        ctx.max_q_len = max(q_lens, default=1)
        ctx.max_kv_len = max((s + q for s, q in zip(starts, q_lens)), default=1)
        ctx.host_q_lens, ctx.host_q_start = q_lens, list(starts)
        ctx.host_kv_lens = [s + q for s, q in zip(starts, q_lens)]
        ctx.host_slots = [cache.slot(e.request_id) for e in entries]
        ctx.request_ids = [e.request_id for e in entries]
        ctx.decode_only = ctx.max_q_len == 1
        ctx.want_all_in_order = in_order
        ctx.num_single = sum(1 for q in q_lens if q == 1) + (Bp - B if not pad_tokens_to else 0)
        ctx.num_portion = sum(1 for q in q_lens if q > 1) if not pad_tokens_to else Bp    # a captured step: an upper bound
        ctx.portion_prefix = max((s for s, q in zip(starts, q_lens) if q > 1), default=0)
        ctx.portion_kv_len = max((s + q for s, q in zip(starts, q_lens) if q > 1), default=0)
        return ctx
