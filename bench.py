#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, random weights.

    python bench.py --gpus 1 --steps K --warmup W [--shape 8b|3b|1b|7b|13b|70b] [--batch 8] [--layers L]

A step is one decode step of the whole batch: every request has prefilled a prompt of
``--context`` / 2 random tokens and decodes one more token a step, greedily, its sampled token
staying on the device for the next step (the serving loop's way).  Prints one JSON line:

  value, ms_per_step   decode tok/s of ``--batch`` requests over exactly ``--steps`` steps
  roofline             the bytes such a step has to read (every weight once, the live requests'
                       keys and values) / its time, against 8 TB/s
  prefill              one prompt of 2,048 tokens in one step; frac = flops / time / peak
  points               decode tok/s at batch 1 and 64 (at least 64 timed steps each)
  serving              the same 8 prompts through ``LLM.generate``'s loop (scheduler, sampler,
                       graphs): tok/s of its decode phase, 256 tokens a request
  serving_arrivals     64 requests that arrive one every other step, prompts cut into portions of 256
                       beside the requests that decode: tok/s generated from the first arrival to the
                       last token, and the share of steps that replayed a graph
  peaks                what a bare read, a copy, a loop of bfloat16 matrix instructions and a loop of
                       32-bit FMAs reach on this GPU now; ``frac_measured`` prices against these
  shape_1b, shape_3b   decode at batch 8 and prefill at the Llama-3.2-1B / 3B layer sizes
  fp32                 the true 32-bit path at the headline shape: decode at batch 8 and prefill
                       (the last three only with the default shape)
"""
import argparse
import json
import os
import sys
import tempfile
import time

SHAPES = {
    # the published Llama 3.2 1B / 3B and Llama 3.1 8B layer sizes
    "1b": dict(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32,
               num_key_value_heads=8, head_dim=64, vocab_size=128256, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0,
                                 high_freq_factor=4.0, original_max_position_embeddings=8192)),
    "3b": dict(hidden_size=3072, intermediate_size=8192, num_hidden_layers=28, num_attention_heads=24,
               num_key_value_heads=8, head_dim=128, vocab_size=128256, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0,
                                 high_freq_factor=4.0, original_max_position_embeddings=8192)),
    "8b": dict(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
               num_key_value_heads=8, head_dim=128, vocab_size=128256, tie_word_embeddings=False,
               rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                 high_freq_factor=4.0, original_max_position_embeddings=8192)),
    # Llama 2 7B / 13B: every head has keys and values of its own, no frequency scaling
    "7b": dict(hidden_size=4096, intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32,
               num_key_value_heads=32, head_dim=128, vocab_size=32000, tie_word_embeddings=False,
               rope_theta=10000.0),
    "13b": dict(hidden_size=5120, intermediate_size=13824, num_hidden_layers=40, num_attention_heads=40,
                num_key_value_heads=40, head_dim=128, vocab_size=32000, tie_word_embeddings=False,
                rope_theta=10000.0),
    # Llama 3.1 70B: 141 GB of bfloat16 weights, which one MI355X holds; measured with --layers
    "70b": dict(hidden_size=8192, intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64,
                num_key_value_heads=8, head_dim=128, vocab_size=128256, tie_word_embeddings=False,
                rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                  high_freq_factor=4.0, original_max_position_embeddings=8192)),
}
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PAGE = 16
MIN_POINT_STEPS = 64


class Bench:
    """One model shape: an ``LLM`` with random weights, and the measurements on it."""

    def __init__(self, shape_name, args, max_batch):
        import torch
        from rustinfer_amd.llm import LLM
        self.torch = torch
        self.args = args
        shape = dict(dict(rms_norm_eps=1e-5, rope_theta=500000.0), **SHAPES[shape_name],
                     architectures=["LlamaForCausalLM"], max_position_embeddings=args.context)
        self.full_layers = shape["num_hidden_layers"]
        if args.layers:
            shape["num_hidden_layers"] = args.layers
        self.prompt_len = args.context // 2
        self.dir = tempfile.TemporaryDirectory()
        with open(os.path.join(self.dir.name, "config.json"), "w") as f:
            json.dump(shape, f)
        self.llm = LLM(model=self.dir.name, random_weights_seed=0,
                       dtype="bfloat16" if args.dtype == "bf16" else "float32",
                       paged_block_size=PAGE, num_blocks=max_batch * (args.context // PAGE) + 8,
                       max_batch_seqs=max_batch, max_model_len=args.context,
                       max_batch_tokens=max(8192, self.prompt_len),
                       capture_sizes=sorted({1, 2, 4, 8, 16, 24, 32, 40, 48, 56, 64, args.batch}),
                       # the prompt's products of 2,048 rows: the library's fastest kernel for each
                       # shape, looked for once in an untimed pass (about a second a shape)
                       gemm_tune=not args.no_gemm_tune,
                       tiled_weight_copy=not getattr(args, "one_weight_copy", False),
                       step_token_align=0 if getattr(args, "no_token_align", False) else 256)
        self.engine = self.llm.engine
        if args.no_graph:
            self.engine.enable_graphs(False)
        self.cfg = cfg = self.llm.model_config
        el = 2 if args.dtype == "bf16" else 4
        L, d, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
        self.weight_bytes = el * (L * (cfg.qkv_dim * d + d * cfg.q_dim + 3 * I * d + 2 * d) + V * d + d)
        self.kv_bytes_per_token = 2 * L * cfg.kv_dim * el
        self.gen = torch.Generator(device="cuda").manual_seed(1)

    def release_all(self):
        for rid in list(self.engine.cache.live_requests()):
            self.engine.release(rid)

    def random_ids(self, n):
        return self.torch.randint(0, self.cfg.vocab_size, (n,), generator=self.gen, device="cuda").tolist()

    def start_requests(self, batch):
        """``batch`` requests prefill a prompt of random tokens each (one step a prompt) and
        sample their first token, which stays on the device."""
        from rustinfer_amd.engine import StepEntry
        self.release_all()
        # graphs are captured ahead, as the reference does at start-up: a capture between the
        # prompts and the first tokens leaves the GPU idle for 20 ms and the next 25 steps 3 % slow
        self.engine.capture_graphs([batch], self.prompt_len + 1)
        if self.args.fake_prompts:
            # keys and values of the size that real ones have, without running the prompts
            for g in self.engine.cache.groups:
                g.k_pool.normal_(0, 0.5, generator=self.gen)
                g.v_pool.normal_(0, 0.5, generator=self.gen)
            for b in range(batch):
                self.engine.cache.add_request(b)
                self.engine.cache.append(b, self.prompt_len)
            self.engine.device_tokens[:batch].copy_(self.torch.randint(
                0, self.cfg.vocab_size, (batch,), generator=self.gen, device="cuda", dtype=self.torch.int32))
            return
        for b in range(batch):
            logits = self.engine.step([StepEntry(b, self.random_ids(self.prompt_len), [self.prompt_len - 1])])
            self.engine.rt.ops.argmax(logits, self.engine.device_tokens[b:b + 1])

    def decode(self, batch, steps, warmup):
        """Greedy decoding as the serving loop does it: sampled tokens stay on the device for
        the next step, and the host reads them one step late, while the next step runs."""
        from rustinfer_amd.engine import StepEntry, device_token
        torch, engine = self.torch, self.engine
        self.start_requests(batch)
        entries = [StepEntry(b, [device_token(b)], [0]) for b in range(batch)]
        pending = [None]

        def one_step():
            logits = engine.step(entries)
            engine.rt.ops.argmax(logits, engine.device_tokens[:batch])
            snapshot = engine.read_device_tokens(batch)
            if pending[0] is not None:
                host, event = pending[0]
                event.synchronize()
                host.tolist()
            pending[0] = snapshot

        for _ in range(warmup):
            one_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            one_step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        mean_ctx = self.prompt_len + warmup + steps / 2.0
        step_bytes = self.weight_bytes + batch * mean_ctx * self.kv_bytes_per_token
        self.release_all()
        return batch * steps / dt, dt / steps, step_bytes

    def prefill(self, tokens_n=2048, reps=5):
        from rustinfer_amd.engine import StepEntry
        torch, cfg = self.torch, self.cfg
        self.release_all()
        ids = self.random_ids(tokens_n)
        times = []
        for r in range(reps + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            self.engine.step([StepEntry("p", ids, [tokens_n - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            self.engine.release("p")
        t = sorted(times[1:])[len(times[1:]) // 2]
        L, d, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
        flops = 2.0 * tokens_n * L * (cfg.qkv_dim * d + d * cfg.q_dim + 3 * I * d) \
            + L * cfg.num_attention_heads * 4.0 * cfg.head_dim * tokens_n * (tokens_n + 1) / 2 \
            + 2.0 * V * d
        return {"value": round(tokens_n / t, 1), "tokens": tokens_n, "ms": round(t * 1e3, 3),
                "frac": round(flops / t / PEAK_FLOPS[self.args.dtype], 4)}

    def prefill_long(self, tokens_n, chunk=8192, reps=3):
        """One prompt of ``tokens_n`` tokens in portions of ``chunk`` (the engine's largest step):
        seconds for the whole prompt, median of ``reps``."""
        from rustinfer_amd.engine import StepEntry
        torch = self.torch
        self.release_all()
        ids = self.random_ids(tokens_n)
        times = []
        for r in range(reps + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for lo in range(0, tokens_n, chunk):
                part = ids[lo:lo + chunk]
                self.engine.step([StepEntry("p", part, [len(part) - 1] if lo + chunk >= tokens_n else [])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            self.engine.release("p")
        return sorted(times[1:])[len(times[1:]) // 2]

    def serving(self, batch, new_tokens=256, sampled=False):
        """The same workload through the entry point's own loop: requests are added, the scheduler
        prefills them and decodes, the sampler chooses, graphs replay.  Returns tok/s of the decode
        phase (from the first step in which every request decodes) and its share of the whole.
        ``sampled``: temperature 0.8 with top-k 50 and top-p 0.95 instead of greedy choice."""
        from rustinfer_amd.sampling import SamplingParams
        torch, llm = self.torch, self.llm
        self.release_all()
        new_tokens = min(new_tokens, self.args.context - self.prompt_len)
        if sampled:
            sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True, temperature=0.8, top_k=50, top_p=0.95, seed=1)
        else:
            sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True)
        llm.capture_graphs(batch, self.prompt_len + 1)
        reqs = [llm.add_request(self.random_ids(self.prompt_len), sp) for _ in range(batch)]
        t_all = time.perf_counter()
        t0, n0 = None, 0
        while llm.scheduler.has_work() or llm._inflight is not None:
            if t0 is None and not llm.scheduler.waiting and len(llm.scheduler.running) == batch \
                    and all(r.remaining == 1 and r.output for r in llm.scheduler.running):
                torch.cuda.synchronize()
                t0, n0 = time.perf_counter(), sum(len(r.output) for r in reqs)
            llm.step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        tokens = sum(len(r.output) for r in reqs) - n0
        if t0 is None:                           # too few tokens for a step in which every request decodes
            return {"value": None, "unit": "tok/s", "requests": batch, "total_s": round(t1 - t_all, 3)}
        return {"value": round(tokens / (t1 - t0), 1), "unit": "tok/s", "requests": batch,
                "prompt_len": self.prompt_len, "new_tokens": new_tokens,
                "decode_ms_per_step": round((t1 - t0) / max(tokens // batch, 1) * 1e3, 4),
                "total_s": round(t1 - t_all, 3)}


    def mixed_step(self, batch, portion, steps, graphs=True):
        """Steps that hold a prompt portion of ``portion`` tokens beside ``batch`` decoding requests
        (the shape continuous batching produces while a prompt arrives): seconds a step, replayed
        as a graph or, with ``graphs=False``, launched eagerly."""
        from rustinfer_amd.engine import StepEntry, device_token
        torch, engine = self.torch, self.engine
        self.start_requests(batch)
        keep = engine._mixed_tokens
        if not graphs:
            engine._mixed_tokens = 0
        try:
            room = self.args.context - 8
            ids = self.random_ids(room)
            state = {"pos": 0, "n": 0}

            def one_step():
                if state["pos"] + portion > room:
                    engine.release(("p", state["n"]))
                    state["pos"], state["n"] = 0, state["n"] + 1
                entries = [StepEntry(b, [device_token(b)], [0]) for b in range(batch)]
                entries.append(StepEntry(("p", state["n"]), ids[state["pos"]:state["pos"] + portion], []))
                state["pos"] += portion
                logits = engine.step(entries)
                engine.rt.ops.argmax(logits, engine.device_tokens[:batch])

            for _ in range(4):
                one_step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                one_step()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / steps
        finally:
            engine._mixed_tokens = keep
            self.release_all()

    def serving_arrivals(self, requests=64, prompt_len=512, new_tokens=128, chunk=256, every=2):
        """Requests arrive while others run: one every ``every`` steps, each prompt cut into
        portions of ``chunk`` tokens that run beside the decoding requests.  Returns tok/s of
        generated tokens over the whole run and how many of its steps replayed a graph."""
        from rustinfer_amd.sampling import SamplingParams
        torch, llm = self.torch, self.llm
        self.release_all()
        sched = llm.scheduler
        old_chunk, sched.chunk = sched.chunk, chunk
        new_tokens = min(new_tokens, self.args.context - prompt_len)
        sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True)
        prompts = [self.random_ids(prompt_len) for _ in range(requests)]
        try:
            torch.cuda.synchronize()
            steps0, replays0, mixed0 = self.engine.steps_run, self.engine.graph_replays, self.engine.mixed_graph_replays
            t0 = time.perf_counter()
            reqs, n = [], 0
            while len(reqs) < requests or sched.has_work() or llm._inflight is not None:
                if len(reqs) < requests and n % every == 0:
                    reqs.append(llm.add_request(prompts[len(reqs)], sp))
                llm.step()
                n += 1
            llm.drain()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        finally:
            sched.chunk = old_chunk
        steps = self.engine.steps_run - steps0
        tokens = sum(len(r.output) for r in reqs)
        return {"value": round(tokens / dt, 1), "unit": "tok/s", "requests": requests, "prompt_len": prompt_len,
                "new_tokens": new_tokens, "chunk": chunk, "steps": steps, "ms_per_step": round(dt / max(steps, 1) * 1e3, 3),
                "graph_share": round((self.engine.graph_replays - replays0) / max(steps, 1), 4),
                "mixed_graph_steps": self.engine.mixed_graph_replays - mixed0, "total_s": round(dt, 3)}

    def close(self):
        """Give the model's memory back before another shape is built."""
        import gc
        self.release_all()
        self.llm = self.engine = None
        gc.collect()
        self.torch.cuda.empty_cache()


def other_shape(name, args, dtype, peaks):
    """Decode at the main batch and prefill of another shape or precision, as a sub-record."""
    sub = argparse.Namespace(**vars(args))
    sub.dtype = dtype
    s = Bench(name, sub, args.batch)
    tok_s, step_s, step_bytes = s.decode(args.batch, max(MIN_POINT_STEPS, args.steps) if dtype == "bf16" else args.steps,
                                         args.warmup)
    gbs = step_bytes / step_s / 1e9
    rec = {"value": round(tok_s, 1), "ms_per_step": round(step_s * 1e3, 4), "roofline_frac": round(gbs / PEAK_HBM_GBS, 4),
           "roofline_frac_measured": round(gbs / peaks["hbm_read_gbs"], 4), "prefill": s.prefill(reps=5 if dtype == "bf16" else 2)}
    flops_peak = peaks["mfma_bf16_tflops"] if dtype == "bf16" else peaks["fma_f32_tflops"]
    rec["prefill"]["frac_measured"] = round(rec["prefill"]["frac"] * PEAK_FLOPS[dtype] / (flops_peak * 1e12), 4)
    s.close()
    return rec


def sampling_times(ops, vocab, steps):
    """us a call of the sampling kernels (and of argmax) for rows of ``vocab`` random logits with one
    likely token, under some settings of temperature / top-k / top-p / min-p."""
    import torch
    dev = "cuda:0"
    settings = {"temperature 0.8": (0.8, 0, 1.0, 0.0), "top_k 50 top_p 0.95": (0.8, 50, 0.95, 0.0),
                "top_p 0.9": (1.0, 0, 0.9, 0.0), "min_p 0.05": (1.0, 0, 1.0, 0.05)}
    out = {"metric": "us a call of the sampling kernels", "vocab": vocab, "rows": {}}
    for rows in (1, 8, 64):
        g = torch.Generator(device=dev).manual_seed(rows)
        logits = torch.randn(rows, vocab, device=dev, generator=g) * 3.0
        logits[:, 17] += 18.0
        draws = torch.rand(rows, device=dev, dtype=torch.float64, generator=g)
        tok = torch.empty(rows, device=dev, dtype=torch.int32)

        def timed(f):
            for _ in range(3):
                f()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                f()
            torch.cuda.synchronize()
            return round((time.perf_counter() - t0) / steps * 1e6, 1)
        res = {"argmax": timed(lambda: ops.argmax(logits, tok))}
        for name, (t, k, p, mp) in settings.items():
            full = lambda v, dt: torch.full((rows,), v, device=dev, dtype=dt)
            a = (full(t, torch.float32), full(k, torch.int32), full(p, torch.float32), full(mp, torch.float32))
            res[name] = timed(lambda: ops.sample(logits, a[0], a[1], a[2], a[3], draws, tok))
        out["rows"][str(rows)] = res
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES))
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096, help="context length; prompts are half of it")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0 = all)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64, prefill, serving and the 1B shape")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--fake-prompts", action="store_true",
                    help="fill the cache with random keys and values instead of prefilling the prompts")
    ap.add_argument("--prompt", type=int, default=0, metavar="N",
                    help="only time the prefill of one prompt of N tokens in portions of 8,192 (needs --context >= N)")
    ap.add_argument("--mixed", type=int, default=0, metavar="P",
                    help="only time steps of a P-token prompt portion beside --batch decoding requests, as a graph and eagerly")
    ap.add_argument("--no-mixed-graph", action="store_true", help="steps with prompt portions launch eagerly")
    ap.add_argument("--arrivals", action="store_true", help="only the workload of requests that arrive while others run")
    ap.add_argument("--arrivals-prompt", type=int, default=512, metavar="N", help="prompt length of that workload")
    ap.add_argument("--one-weight-copy", action="store_true",
                    help="no second, tile-ordered copy of the weights: half their memory, slower single-token steps")
    ap.add_argument("--no-token-align", action="store_true",
                    help="steps a few tokens over a multiple of 256 keep them (launch option step_token_align = 0)")
    ap.add_argument("--sampling", action="store_true",
                    help="only time the sampling kernels on 1, 8 and 64 rows of the shape's vocabulary")
    ap.add_argument("--no-gemm-tune", action="store_true",
                    help="keep the GEMM library's own choice of kernel for the prompt's products")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    from rustinfer_amd.kernels import ops
    if args.sampling:
        print(json.dumps(sampling_times(ops, SHAPES[args.shape]["vocab_size"], args.steps)))
        return 0
    peaks = ops.measure_peaks()
    b = Bench(args.shape, args, max(args.batch, 16 if args.mixed else 1 if (args.no_points or args.prompt) else 64))
    cfg = b.cfg
    if args.no_mixed_graph:
        b.engine._mixed_tokens = 0
    if args.arrivals:
        b.serving_arrivals(prompt_len=args.arrivals_prompt)    # untimed: the graphs of its step shapes are captured here
        print(json.dumps({"shape": args.shape, "serving_arrivals": b.serving_arrivals(prompt_len=args.arrivals_prompt)}))
        return 0
    if args.prompt:
        t = b.prefill_long(args.prompt)
        print(json.dumps({"metric": "prefill of one prompt of %d tokens in portions of 8,192" % args.prompt, "shape": args.shape,
                          "ms": round(t * 1e3, 2), "tok_s": round(args.prompt / t, 1)}))
        return 0
    if args.mixed:
        # decoding requests run out of context after `context - prompt` steps: keep the timed steps below that
        steps = min(args.steps, (args.context - b.prompt_len) // 2 - 8)
        b.mixed_step(args.batch, args.mixed, steps, graphs=True)      # untimed: the graphs of its shapes are captured here
        g = b.mixed_step(args.batch, args.mixed, steps, graphs=True)
        e = b.mixed_step(args.batch, args.mixed, steps, graphs=False)
        print(json.dumps({"metric": "ms a step of a %d-token prompt portion beside %d decoding requests" % (args.mixed, args.batch),
                          "shape": args.shape, "graph_ms": round(g * 1e3, 4), "eager_ms": round(e * 1e3, 4), "steps": steps,
                          "mixed_graph_replays": b.engine.mixed_graph_replays}))
        return 0
    tok_s, step_s, step_bytes = b.decode(args.batch, args.steps, args.warmup)
    achieved = step_bytes / step_s / 1e9
    out = {
        "metric": "decode tok/s at batch %d (prefill tok/s at 2,048 tokens and batch 1/64 beside it)" % args.batch,
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights N(0, 0.02), prompts of uniform random token ids"
                + (" (cache filled with random keys and values, prompts not run)" if args.fake_prompts else ", prefilled"),
        "config": {"model": f"llama-3 {args.shape} shape", "global_batch": args.batch,
                   "seq_len": args.context, "prompt_len": b.prompt_len, "parallelism": "none (1 GPU)",
                   "layers": cfg.num_hidden_layers, "layers_of_shape": b.full_layers, "hidden_size": cfg.hidden_size,
                   "intermediate_size": cfg.intermediate_size, "num_attention_heads": cfg.num_attention_heads,
                   "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "vocab_size": cfg.vocab_size, "tie_word_embeddings": cfg.tie_word_embeddings,
                   "kv_page_size": PAGE, "rope_theta": cfg.rope_theta,
                   "rope_scaling_factor": cfg.rope_scaling.factor if cfg.rope_scaling else 1.0, "rms_norm_eps": cfg.rms_norm_eps,
                   "gemm_tuned": not args.no_gemm_tune,
                   # of the weights' bytes, how much has a second, tile-ordered copy (less than all
                   # where the model fills most of the device)
                   "second_copy_share": round(b.engine.rt.tiled_bytes / max(b.weight_bytes, 1), 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4),
                     "peak_measured": peaks["hbm_read_gbs"], "frac_measured": round(achieved / peaks["hbm_read_gbs"], 4)},
        "peaks": peaks,
    }
    flops_peak = (peaks["mfma_bf16_tflops"] if args.dtype == "bf16" else peaks["fma_f32_tflops"]) * 1e12
    if not args.no_points:
        out["prefill"] = b.prefill()
        out["prefill"]["frac_measured"] = round(out["prefill"]["frac"] * PEAK_FLOPS[args.dtype] / flops_peak, 4)
        pts = {}
        for batch in (1, 64):
            pts[f"decode_b{batch}"] = round(b.decode(batch, max(MIN_POINT_STEPS, args.steps), min(args.warmup, 4))[0], 1)
        out["points"] = pts
        b.serving(args.batch, new_tokens=8)      # untimed: the library's kernels for this many prompt rows are chosen here
        out["serving"] = b.serving(args.batch)
        out["serving"]["sampled_value"] = b.serving(args.batch, sampled=True)["value"]   # temperature, top-k and top-p
        b.serving_arrivals()                                 # untimed: the graphs of its step shapes are captured here
        out["serving_arrivals"] = b.serving_arrivals()
        if args.shape == "8b" and not args.layers and args.dtype == "bf16":
            # the other benchmark shapes and the exact path beside the headline
            b.close()
            out["shape_1b"] = other_shape("1b", args, "bf16", peaks)
            out["shape_3b"] = other_shape("3b", args, "bf16", peaks)
            out["fp32"] = other_shape("8b", args, "fp32", peaks)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
