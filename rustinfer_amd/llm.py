"""The Python entry point: ``LLM(...).generate(prompts, sampling_params)``.

The reference has no Python API (it is driven over HTTP); the launch options it reads from
its TOML keep their names here (``EngineConfig``).  Prompts are lists of token ids: a
tokenizer is not part of the engine.
"""
from __future__ import annotations

import os
import sys
import time
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Union

from .config.engine_config import EngineConfig, load_engine_config
from .config.registry import load_model_config
from .engine.factory import build_engine
from .engine.markers import profile_range
from .engine.scheduler import PENDING, Request, Scheduler
from .engine.step import StepEntry, device_token
from .sampling.params import SamplingParams
from .sampling.sampler import Sampler, fresh_seed


def _env_flag(name: str) -> bool:
    return os.environ.get(name, "").strip().lower() not in ("", "0", "false", "no", "off")


@dataclass
class GenerationResult:
    request_id: Hashable
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: str
    preemptions: int = 0
    # for requests whose SamplingParams.logprobs is set: ln p of each generated token, and the
    # five most probable tokens at its place with theirs (empty for greedy requests)
    logprobs: Optional[List[float]] = None
    top_logprobs: Optional[List[List[tuple]]] = None


class LLM:
    def __init__(self, model: Optional[str] = None, config: Optional[Union[str, EngineConfig]] = None,
                 **overrides):
        """``model``: a model folder; or ``config``: a launch file / EngineConfig.  Keyword
        arguments override single options (names as in the launch file)."""
        if isinstance(config, str):
            cfg = load_engine_config(config)
        elif config is None:
            cfg = EngineConfig(model=model or "")
        else:
            cfg = config
        if model:
            cfg.model = model
        for k, v in overrides.items():
            if not hasattr(cfg, k):
                raise TypeError(f"unknown option {k!r}")
            setattr(cfg, k, v)
        cfg.validate()
        self.config = cfg
        _, self.model_config = load_model_config(cfg.model)
        if cfg.gemm_tune or _env_flag("RUSTINFER_GEMM_TUNE"):
            from .kernels import ops as _ops
            _ops.set_gemm_tuning(True)
        if _env_flag("RUSTINFER_FORCE_GEMM"):
            from .kernels import ops as _ops
            _ops.FORCE_LIBRARY_GEMM = True
        self.engine = build_engine(cfg.model, dtype=cfg.dtype, device=cfg.device,
                                   page_size=cfg.paged_block_size, num_pages=cfg.num_blocks,
                                   max_requests=cfg.max_batch_seqs, max_model_len=cfg.max_model_len,
                                   max_batch_tokens=cfg.max_batch_tokens,
                                   mem_fraction=cfg.mem_fraction_static,
                                   random_weights_seed=cfg.random_weights_seed,
                                   tiled_weight_copy=cfg.tiled_weight_copy,
                                   tiled_weight_reserve=cfg.tiled_weight_reserve)
        self._say_slow_paths()
        # environment switches, named as the reference's (crates/infer-core/src/env_flags.rs:18-52)
        if not _env_flag("RUSTINFER_DISABLE_GRAPH"):
            mixed = cfg.mixed_graph_tokens
            if os.environ.get("RUSTINFER_MIXED_GRAPH", "").strip() != "":
                mixed = (mixed if mixed > 0 else 512) if _env_flag("RUSTINFER_MIXED_GRAPH") else 0
            if mixed < 0:
                mixed = 1024 if self._launch_bound() else 0
            self.engine.enable_graphs(True, cfg.capture_sizes, mixed_tokens=mixed, mixed_after=cfg.mixed_graph_after)
            if cfg.prewarm_graphs:
                self.engine.prewarm_graphs()
        self._trace_ms = float(os.environ.get("RUSTINFER_STEP_TRACE_MS", "20")) \
            if _env_flag("RUSTINFER_STEP_TRACE") else None
        # the forward pass and the sampling of every step timed apart, each waited for
        # (crates/infer-worker/src/application/runtime/mod.rs:610-627)
        self._ttft_trace = _env_flag("RUSTINFER_TTFT_TRACE")
        self.sampler = Sampler(self.engine.rt, cfg.max_batch_seqs)
        self.scheduler = Scheduler(self.engine.cache, cfg.max_batch_tokens, cfg.max_batch_seqs,
                                   cfg.max_model_len, cfg.chunked_prefill_size,
                                   cfg.max_prefill_seqs_per_iter, cfg.prefill_sjf, cfg.step_token_align)
        self.eos_ids = tuple(getattr(self.model_config, "eos_token_ids", ()))
        self._next_id = 0
        self._inflight = None
        self.last_stats: Dict[str, float] = {}

    def _say_slow_paths(self) -> None:
        """One line for each reason why a layer's attention misses the fast kernels (a launch file
        written for the reference says paged_block_size = 1, for one)."""
        why = getattr(self.engine.rt.ops, "attention_kernel_note", None)
        notes = set()
        for layer in getattr(self.engine.model, "layers", ()) if why is not None else ():
            m = getattr(layer, "mixer", None)
            if all(hasattr(m, a) for a in ("num_heads", "num_kv_heads", "head_dim")):
                note = why(self.engine.rt.dtype, m.num_heads, m.num_kv_heads, m.head_dim, self.engine.page_size)
                if note:
                    notes.add(note)
        for note in sorted(notes):
            print(f"[rustinfer_amd] {note}", file=sys.stderr, flush=True)

    def _launch_bound(self) -> bool:
        """Whether launching a step with a prompt portion kernel by kernel takes the host longer than
        the kernels run: then such steps are worth capturing.  A launch costs the host about 12 us,
        a block about nine of them; a step with a portion of a few hundred tokens takes about 2.8
        times as long as its weights need at 5 TB/s.  (Measured, 64 requests arriving beside
        decoding ones, portions of 256: at the 1B shape graphs gain 11 %, at the 3B shape they lose
        1.5 %, at the 8B shape nothing either way; the rule says yes, no and no.)"""
        model = self.engine.model
        el = 2 if self.config.dtype == "bfloat16" else 4
        weights = 0
        for spec in model.param_specs().values():
            n = 1
            for d in spec.shape:
                n *= int(d)
            weights += n * el
        host = 12e-6 * 9 * max(len(getattr(model, "schedule", ())), 1)
        return host > 2.8 * weights / 5e12

    # -- requests -----------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[Hashable] = None) -> Request:
        params = params or SamplingParams()
        if self.config.ignore_eos and not params.ignore_eos:
            params = SamplingParams(**{**params.__dict__, "ignore_eos": True})
        V = self.engine.vocab_size
        prompt = [int(t) for t in prompt]
        if any(not (0 <= t < V) for t in prompt):
            raise ValueError(f"prompt holds a token id outside [0, {V})")
        if request_id is None:
            request_id = self._next_id
            self._next_id += 1
        seed = params.seed if params.seed is not None else fresh_seed()
        return self.scheduler.add(Request(request_id, prompt, params, seed=seed, eos_ids=self.eos_ids))

    def capture_graphs(self, rows: int, kv_len: int) -> int:
        """Capture ahead the graphs that ``rows`` decoding requests with up to ``kv_len`` cached tokens
        will replay (else they are captured when first needed, between a prompt and its first
        tokens).  Returns how many were captured."""
        return self.engine.capture_graphs([min(int(rows), self.config.max_batch_seqs)], kv_len)

    def step(self):
        """One scheduler step.  The step is queued on the GPU and its sampled tokens stay there:
        the next step reads them from the device, so it can be prepared and queued while this one
        runs.  Returns [(request, token)] for the tokens that reached the host during this call,
        which are those of the step before."""
        t_start = time.perf_counter() if self._trace_ms is not None else 0.0
        with profile_range("schedule"):
            sched = self.scheduler.schedule()
        inflight = None
        if sched.entries:
            entries, finals = [], []
            for e in sched.entries:
                r = e.request
                toks = r.tokens[e.start:e.start + e.count]
                if toks[-1] == PENDING:                       # sampled by the step before, still on the device
                    toks[-1] = device_token(r.pending_slot)
                entries.append(StepEntry(r.request_id, toks, [e.count - 1] if e.final else []))
                if e.final:
                    finals.append(e)
            t_fwd = time.perf_counter() if self._ttft_trace else 0.0
            logits = self.engine.step(entries)
            if self._ttft_trace:
                self.engine.synchronize()
                print(f"[ttft-trace] forward ({sched.num_tokens} tokens in {len(entries)} rows, synced) = "
                      f"{(time.perf_counter() - t_fwd) * 1e3:.2f}ms", file=sys.stderr, flush=True)
                t_fwd = time.perf_counter()
            lp_host = None
            if finals:
                with profile_range("sample"):
                    lp = self.sampler.sample_into(logits, [e.request.params for e in finals],
                                                  [e.request.seed for e in finals],
                                                  [e.start + e.count for e in finals],
                                                  self.engine.device_tokens[:len(finals)])
                if self._ttft_trace:
                    self.engine.synchronize()
                    print(f"[ttft-trace] sample ({len(finals)} rows, synced) = "
                          f"{(time.perf_counter() - t_fwd) * 1e3:.2f}ms", file=sys.stderr, flush=True)
                if lp is not None:
                    # asked for rarely: read at once (this waits for the step) rather than a step late
                    lp_host = [t.tolist() for t in lp]
            self.scheduler.commit(sched, None)                # optimistic: marks instead of tokens
            marks = []
            for slot, e in enumerate(finals):
                r = e.request
                if r.output and r.output[-1] == PENDING:
                    r.pending_slot = slot
                marks.append((r, len(r.output) - 1, slot))
                if lp_host is not None and r.params.logprobs:
                    r.logprob_at[len(r.output) - 1] = (
                        lp_host[0][slot],
                        [(i, x) for i, x in zip(lp_host[1][slot], lp_host[2][slot]) if i >= 0])
            host, event = self.engine.read_device_tokens(len(finals)) if finals else (None, None)
            inflight = (marks, host, event)
        produced = self._resolve(self._inflight)
        self._inflight = inflight
        if self._trace_ms is not None:
            # a work iteration slower than the threshold, with its batch shape and the cache's state
            # (crates/infer-worker/src/application/serve_loop.rs:931-949)
            ms = (time.perf_counter() - t_start) * 1e3
            if ms >= self._trace_ms:
                cache = self.engine.cache
                print(f"[step-trace] {ms:.1f} ms rows={len(sched.entries)} tokens={sched.num_tokens} "
                      f"preempted={len(sched.preempted)} running={len(self.scheduler.running)} "
                      f"waiting={len(self.scheduler.waiting)} free_pages={cache.free_pages()}",
                      file=sys.stderr, flush=True)
        return produced

    def _resolve(self, inflight):
        """Wait for the tokens of a queued step and hand them to the scheduler."""
        if inflight is None:
            return []
        marks, host, event = inflight
        if host is None:
            return []
        if event is not None:
            event.synchronize()
        tokens = host.tolist()
        out = []
        for r, index, slot in marks:
            if self.scheduler.resolve(r, index, tokens[slot]):
                out.append((r, tokens[slot]))
        return out

    def drain(self):
        """Wait for the step that is still queued, if any."""
        produced = self._resolve(self._inflight)
        self._inflight = None
        return produced

    def generate(self, prompts: Sequence[Sequence[int]],
                 sampling_params: Union[None, SamplingParams, Sequence[SamplingParams]] = None
                 ) -> List[GenerationResult]:
        """Generate for every prompt (lists of token ids) and return results in their order."""
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            sampling_params = [sampling_params or SamplingParams()] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError("one SamplingParams for each prompt")
        reqs = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
        if prompts:
            self.capture_graphs(len(prompts), max(len(p) for p in prompts) + 1)
        t0 = time.perf_counter()
        before = dict(self.scheduler.stats)
        idle = 0
        while self.scheduler.has_work() or self._inflight is not None:
            steps_before = self.scheduler.stats["steps"]
            self.step()
            idle = idle + 1 if self.scheduler.stats["steps"] == steps_before else 0
            if idle > 3:
                raise RuntimeError("the scheduler can start nothing although requests are left; "
                                   "the cache pool is too small for them")
        dt = time.perf_counter() - t0
        st = self.scheduler.stats
        self.last_stats = {k: st[k] - before.get(k, 0) for k in st if k != "peak_pages"}
        self.last_stats.update(peak_pages=st["peak_pages"], seconds=dt)
        out = []
        for r in reqs:
            res = GenerationResult(r.request_id, r.prompt, list(r.output), r.finish_reason or "", r.preemptions)
            if r.params.logprobs:
                res.logprobs = [r.logprob_at[i][0] for i in range(len(r.output))]
                res.top_logprobs = [r.logprob_at[i][1] for i in range(len(r.output))]
            out.append(res)
        return out


def generate(model: str, prompts: Sequence[Sequence[int]],
             sampling_params: Union[None, SamplingParams, Sequence[SamplingParams]] = None,
             **options) -> List[GenerationResult]:
    """One-call form: build an engine for ``model`` and generate."""
    return LLM(model=model, **options).generate(prompts, sampling_params)
