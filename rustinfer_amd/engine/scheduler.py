"""Continuous batching with chunked prefill, in one process.

The reference splits this over two processes: its scheduler admits requests and cuts
prompts under token, sequence and cache budgets
(crates/infer-scheduler/src/domain/policy/continuous_batching.rs:62-210), its worker decodes
every live request each step and fuses pending prompt portions into the same batch
(crates/infer-worker/src/application/worker_scheduler.rs:386-1015).  Here one ``schedule()``
decides a whole step:

1. every request that is decoding runs, one token each, in admission order;
2. requests in the middle of their prompt continue ("they already hold cache",
   continuous_batching.rs:78-105), each with ``min(rest, chunked_prefill_size, budget)`` tokens;
3. waiting requests start, first come first served (or shortest first), while a sequence slot,
   token budget and pages are left; a prompt that does not fit whole is started with what fits
   (continuous_batching.rs:321-337).

When pages run out
------------------
* A prompt portion never evicts anything: it is shortened to the pages that are free, or waits.
  A new request starts only if the pool can take its whole prompt and one more page for every
  request already running.
* If the decoding requests cannot all get the page they need, requests are preempted until they
  can: the victim has the most generated tokens, then the shortest prompt
  (crates/infer-scheduler/src/application/control_fns.rs:322-338); everything it holds is given
  back and it returns to the FRONT of the queue, to be recomputed from ``prompt + generated``
  (crates/infer-scheduler/src/domain/inference_session/table.rs:767-815).
* A request that cannot run even alone (its tokens exceed the pool) finishes with reason
  ``"error"``.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache.manager import CacheManager, pages_for
from ..sampling.params import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"
PENDING = -1      # in Request.output: a token that was sampled but has not reached the host yet


@dataclass
class Request:
    request_id: Hashable
    prompt: List[int]
    params: SamplingParams
    seed: int = 0
    eos_ids: Tuple[int, ...] = ()
    output: List[int] = field(default_factory=list)
    num_computed: int = 0            # tokens whose keys and values are in the cache
    state: str = WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0
    arrival: int = 0
    pending_slot: int = -1           # where on the device the PENDING token lies
    # output index -> (ln p of the token, [(token, ln p)] of the five most probable), if asked for
    logprob_at: Dict[int, Tuple[float, List[Tuple[int, float]]]] = field(default_factory=dict)

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def num_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    @property
    def remaining(self) -> int:
        return self.num_tokens - self.num_computed


@dataclass
class ScheduledEntry:
    request: Request
    start: int          # first token of the portion (= tokens already cached)
    count: int          # tokens in the portion
    final: bool         # the portion ends the request's known tokens: its last logits are sampled

    @property
    def is_decode(self) -> bool:
        return self.count == 1 and self.final and len(self.request.output) > 0


@dataclass
class ScheduledStep:
    entries: List[ScheduledEntry]
    preempted: List[Request] = field(default_factory=list)
    failed: List[Request] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(e.count for e in self.entries)


class Scheduler:
    def __init__(self, cache: CacheManager, max_batch_tokens: int = 8192, max_batch_seqs: int = 32,
                 max_model_len: int = 4096, chunked_prefill_size: int = 0,
                 max_prefill_seqs_per_iter: int = 0, prefill_sjf: bool = False, token_align: int = 0):
        self.cache = cache
        self.align = int(token_align)
        self.max_batch_tokens = int(max_batch_tokens)
        self.max_batch_seqs = int(max_batch_seqs)
        self.max_model_len = int(max_model_len)
        self.chunk = int(chunked_prefill_size)
        self.max_new = int(max_prefill_seqs_per_iter)
        self.sjf = bool(prefill_sjf)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []          # stable admission order
        self.finished: List[Request] = []
        self._arrivals = 0
        self.stats = {"steps": 0, "preemptions": 0, "prefill_tokens": 0, "decode_tokens": 0,
                      "peak_pages": 0}

    # -- requests ------------------------------------------------------------
    def add(self, request: Request) -> Request:
        if not request.prompt:
            raise ValueError("a request needs at least one prompt token")
        request.params.validate()
        request.arrival = self._arrivals
        self._arrivals += 1
        request.state = WAITING
        self.waiting.append(request)
        return request

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _finish(self, req: Request, reason: str) -> None:
        if self.cache.has_request(req.request_id):
            self.cache.release(req.request_id)
        if req in self.running:
            self.running.remove(req)
        req.state = FINISHED
        req.finish_reason = reason
        self.finished.append(req)

    def abort(self, request_id) -> None:
        for req in list(self.running) + list(self.waiting):
            if req.request_id == request_id:
                if req in self.waiting:
                    self.waiting.remove(req)
                self._finish(req, "cancelled")

    # -- one step's decisions ----------------------------------------------------
    def _preempt(self, req: Request) -> None:
        self.cache.release(req.request_id)
        self.running.remove(req)
        req.num_computed = 0
        req.state = WAITING
        req.preemptions += 1
        self.stats["preemptions"] += 1
        self.waiting.appendleft(req)

    def _fit(self, wants, rid, n: int) -> int:
        """Largest m <= n such that the cache can take ``wants`` plus m tokens of ``rid``."""
        if self.cache.can_append(wants + [(rid, n)]):
            return n
        lo, hi = 0, n                    # can take lo, cannot take hi
        while hi - lo > 1:
            mid = (lo + hi) // 2
            if self.cache.can_append(wants + [(rid, mid)]):
                lo = mid
            else:
                hi = mid
        return lo

    def schedule(self) -> ScheduledStep:
        step = ScheduledStep([])
        budget = self.max_batch_tokens
        wants: List[Tuple[Hashable, int]] = []

        # 1. decoding requests: all of them, or preempt until the rest fits
        decoding = [r for r in self.running if r.remaining == 1 and r.output]
        while decoding:
            if self.cache.can_append([(r.request_id, 1) for r in decoding]):
                break
            if len(self.running) == 1:
                lone = self.running[0]
                self._finish(lone, "error")
                step.failed.append(lone)
                decoding = []
                break
            victim = max(self.running, key=lambda r: (len(r.output), -len(r.prompt), r.arrival))
            self._preempt(victim)
            step.preempted.append(victim)
            decoding = [r for r in decoding if r is not victim]
        for r in decoding[:budget]:
            step.entries.append(ScheduledEntry(r, r.num_computed, 1, True))
            wants.append((r.request_id, 1))
        budget -= len(step.entries)

        # 2. prompts under way.  If no row of the step runs and none of them gets a page, they
        # hold the whole pool between them: one is given up (the victims' order of the reference,
        # crates/infer-scheduler/src/application/control_fns.rs:322-338) until another can go on.
        while True:
            for r in self.running:
                if budget <= 0:
                    break
                if r.remaining == 1 and r.output:
                    continue
                n = min(r.remaining, budget, self.chunk or r.remaining)
                n = self._fit(wants, r.request_id, n)
                if n <= 0:
                    continue
                step.entries.append(ScheduledEntry(r, r.num_computed, n, n == r.remaining))
                wants.append((r.request_id, n))
                budget -= n
            if step.entries or not self.running:
                break
            if len(self.running) == 1:
                lone = self.running[0]               # alone and still without room: it can never run
                self._finish(lone, "error")
                step.failed.append(lone)
                break
            victim = max(self.running, key=lambda r: (len(r.output), -len(r.prompt), r.arrival))
            self._preempt(victim)
            step.preempted.append(victim)

        # 3. new requests
        started = 0
        queue = sorted(self.waiting, key=lambda r: r.num_tokens) if self.sjf else list(self.waiting)
        for r in queue:
            if budget <= 0 or len(self.running) >= self.max_batch_seqs:
                break
            if self.max_new and started >= self.max_new:
                break
            if r.num_tokens > self.max_model_len:
                self.waiting.remove(r)
                self._finish(r, "error")
                step.failed.append(r)
                continue
            need_pages = max((pages_for(r.num_tokens, g.page_size) for g in self.cache.groups), default=0)
            if need_pages > min((g.num_pages for g in self.cache.groups), default=need_pages):
                self.waiting.remove(r)              # can never run, not even alone
                self._finish(r, "error")
                step.failed.append(r)
                continue
            reserve = len(self.running) + 1
            # pages the running requests' prompts will still take
            reserve += sum(max(pages_for(q.num_tokens, self.cache.page_size)
                               - (pages_for(self.cache.kv_len(q.request_id), self.cache.page_size)
                                  if self.cache.has_request(q.request_id) else 0), 0)
                           for q in self.running)
            pending = sum(max(pages_for(self.cache.kv_len(rid) + m, self.cache.page_size)
                              - pages_for(self.cache.kv_len(rid), self.cache.page_size), 0)
                          if self.cache.has_request(rid) else pages_for(m, self.cache.page_size)
                          for rid, m in wants)
            if self.cache.groups and self.cache.free_pages() - pending < need_pages + reserve - 1 \
                    and (self.running or step.entries):
                break                                # wait for room rather than thrash
            n = min(r.remaining, budget, self.chunk or r.remaining)
            n = self._fit(wants, r.request_id, n)
            if n <= 0:
                break
            self.waiting.remove(r)
            r.state = RUNNING
            self.running.append(r)
            step.entries.append(ScheduledEntry(r, 0, n, n == r.remaining))
            wants.append((r.request_id, n))
            budget -= n
            started += 1
            if not self.sjf and n < r.remaining and budget <= 0:
                break
        self._trim_to_alignment(step)
        return step

    def _trim_to_alignment(self, step: ScheduledStep) -> None:
        """A step a few tokens over a multiple of ``token_align`` gives them up: the matrix products
        of a step work in tiles of rows, and the few rows over cost a whole tile (264 rows take 19 %
        longer than 256).  Only a portion that is not its prompt's last can give tokens up, and only
        if its prompt then still ends in as many portions as before: the tokens run with the next
        portion, and nobody's first token waits for them."""
        if self.align <= 0:
            return
        total = step.num_tokens
        over = total % self.align
        if total < self.align or over == 0 or over > self.align // 8:
            return
        most = self.chunk or self.max_batch_tokens               # what a later portion can hold
        for e in reversed(step.entries):
            left = e.request.remaining - e.count                 # for later portions
            if not e.final and e.count > over and -(-(left + over) // most) == -(-left // most):
                e.count -= over
                return

    # -- after the step ran ----------------------------------------------------------
    def commit(self, step: ScheduledStep, sampled: Optional[Dict[Hashable, int]] = None
               ) -> List[Tuple[Request, int]]:
        """``sampled``: request id -> token, for every final entry.  Returns (request, token)
        for each token produced, and finishes requests that are done: the token that ends a
        request is still emitted (crates/infer-worker/src/application/runtime/mod.rs:1198-1214).

        With ``sampled=None`` the tokens are not known yet (they are still on the device): a
        PENDING mark is appended instead, requests that end by length are finished now, and
        ``resolve`` supplies the tokens and the end-of-sequence check one step later."""
        out = []
        self.stats["steps"] += 1
        for e in step.entries:
            r = e.request
            if r.state == FINISHED:
                continue                     # ended while this step was in flight
            r.num_computed += e.count
            if e.is_decode:
                self.stats["decode_tokens"] += 1
            else:
                self.stats["prefill_tokens"] += e.count
            if not e.final:
                continue
            tok = PENDING if sampled is None else int(sampled[r.request_id])
            r.output.append(tok)
            out.append((r, tok))
            p = r.params
            if tok != PENDING and self._cut_at_stop(r, len(r.output) - 1):
                self._finish(r, "stop")
            elif tok != PENDING and not p.ignore_eos and tok in r.eos_ids:
                self._finish(r, "eos")
            elif len(r.output) >= p.max_tokens:
                self._finish(r, "length")
            elif r.num_tokens > self.max_model_len:
                self._finish(r, "length")
        held = sum(g.allocator.outstanding for g in self.cache.groups)
        self.stats["peak_pages"] = max(self.stats["peak_pages"], held)
        return out

    @staticmethod
    def _cut_at_stop(request: Request, index: int) -> bool:
        """If the output up to and including ``index`` ends with one of the request's stop
        sequences, take the longest such sequence (and whatever a step that ran ahead put after
        it) off the output.  crates/infer-scheduler/src/domain/inference_session/table.rs:541-560,
        :1031-1038."""
        stops = request.params.stop_sequences
        if not stops:
            return False
        known = request.output[:index + 1]
        longest = 0
        for stop in stops:
            n = len(stop)
            if n > longest and n <= len(known) and tuple(known[-n:]) == tuple(stop):
                longest = n
        if not longest:
            return False
        del request.output[index + 1 - longest:]
        return True

    def resolve(self, request: Request, index: int, token: int) -> bool:
        """The token at ``request.output[index]`` has arrived.  Returns False if the request had
        already ended before that token (the token is dropped).  An end-of-sequence token ends the
        request now; what a later step computed for it in the meantime is discarded."""
        if index >= len(request.output) or request.output[index] != PENDING:
            return False
        request.output[index] = int(token)
        if self._cut_at_stop(request, index):
            if request.state != FINISHED:
                if request in self.waiting:              # preempted in the meantime
                    self.waiting.remove(request)
                self._finish(request, "stop")
            else:
                request.finish_reason = "stop"
        elif not request.params.ignore_eos and int(token) in request.eos_ids:
            del request.output[index + 1:]               # marks of a step that ran ahead
            if request.state != FINISHED:
                if request in self.waiting:              # preempted in the meantime
                    self.waiting.remove(request)
                self._finish(request, "eos")
            else:
                request.finish_reason = "eos"            # had also reached its length
        return True
