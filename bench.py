#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, random weights.

    python bench.py --gpus 1 --steps K --warmup W [--shape 1b|3b|8b] [--batch 8] [--layers L]

A step is one decode step of the whole batch: every request has ``--context`` / 2 tokens
in the cache and decodes one more.  Prints one JSON line.
"""
import argparse
import json
import sys
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
}
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES))
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096, help="context length; prompts are half of it")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0 = all)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and prefill")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-gemm-tune", action="store_true",
                    help="keep the GEMM library's own choice of kernel for the prompt's products")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from rustinfer_amd.config import LlamaConfig
    from rustinfer_amd.engine import Engine, StepEntry, device_token, make_runtime
    from rustinfer_amd.models.llama import build_llama
    from rustinfer_amd.weights import init_random_weights

    shape = dict(SHAPES[args.shape], max_position_embeddings=args.context, rms_norm_eps=1e-5,
                 rope_theta=500000.0)
    full_layers = shape["num_hidden_layers"]
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    cfg = LlamaConfig.from_dict(shape)
    rt = make_runtime("bfloat16" if args.dtype == "bf16" else "float32", "cuda:0")
    if not args.no_gemm_tune:
        # the prompt's products of 2,048 rows: the library's fastest kernel for each shape, looked
        # for once in the untimed first pass (about a second a shape) and kept in a file
        rt.ops.set_gemm_tuning(True)
    model = build_llama(cfg)
    init_random_weights(model, seed=0, rt=rt)
    page = 16
    prompt_len = args.context // 2
    max_batch = max(args.batch, 1 if args.no_points else 64)
    num_pages = max_batch * (args.context // page) + 8
    engine = Engine(model, rt, page_size=page, num_pages=num_pages, max_requests=max_batch,
                    max_model_len=args.context, max_batch_tokens=max(8192, prompt_len))
    if hasattr(engine, "enable_graphs") and not args.no_graph:
        engine.enable_graphs(True, sorted({1, 2, 4, 8, 16, 24, 32, 40, 48, 56, 64, args.batch}))
    el = 2 if args.dtype == "bf16" else 4
    L, d, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    weight_bytes = el * (L * (cfg.qkv_dim * d + d * cfg.q_dim + 3 * I * d + 2 * d) + V * d + d)
    kv_bytes_per_token = 2 * L * cfg.kv_dim * el
    gen = torch.Generator(device="cuda").manual_seed(1)

    def fill_requests(batch):
        """Requests whose prompts are already in the cache (random keys and values of the size
        that real ones have; the timed steps only read them)."""
        for rid in list(engine.cache.live_requests()):
            engine.release(rid)
        for g in engine.cache.groups:
            g.k_pool.normal_(0, 0.5, generator=gen)
            g.v_pool.normal_(0, 0.5, generator=gen)
        for b in range(batch):
            engine.cache.add_request(b)
            engine.cache.append(b, prompt_len)

    def decode(batch, steps, warmup):
        """Greedy decoding as the serving loop does it: sampled tokens stay on the device for
        the next step, and the host reads them one step late, while the next step runs."""
        fill_requests(batch)
        engine.device_tokens[:batch].copy_(torch.randint(0, V, (batch,), generator=gen, device="cuda",
                                                         dtype=torch.int32))
        entries = [StepEntry(b, [device_token(b)], [0]) for b in range(batch)]
        pending = [None]

        def one_step():
            logits = engine.step(entries)
            rt.ops.argmax(logits, engine.device_tokens[:batch])
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
        mean_ctx = prompt_len + warmup + steps / 2.0
        step_bytes = weight_bytes + batch * mean_ctx * kv_bytes_per_token
        return batch * steps / dt, dt / steps, step_bytes

    def prefill(tokens_n=2048, reps=5):
        for rid in list(engine.cache.live_requests()):
            engine.release(rid)
        ids = torch.randint(0, V, (tokens_n,), generator=gen, device="cuda").tolist()
        times = []
        for r in range(reps + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.step([StepEntry("p", ids, [tokens_n - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            engine.release("p")
        t = sorted(times[1:])[len(times[1:]) // 2]
        flops = 2.0 * tokens_n * L * (cfg.qkv_dim * d + d * cfg.q_dim + 3 * I * d) \
            + L * cfg.num_attention_heads * 4.0 * cfg.head_dim * tokens_n * (tokens_n + 1) / 2 \
            + 2.0 * V * d
        return tokens_n / t, t, flops

    tok_s, step_s, step_bytes = decode(args.batch, args.steps, args.warmup)
    achieved = step_bytes / step_s / 1e9
    out = {
        "metric": "decode tok/s at batch %d (prefill tok/s at 2,048 tokens and batch 1/64 beside it)" % args.batch,
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
        "config": {"model": f"llama-3 {args.shape} shape", "global_batch": args.batch,
                   "seq_len": args.context, "prompt_len": prompt_len, "parallelism": "none (1 GPU)",
                   "layers": L, "layers_of_shape": full_layers, "hidden_size": d,
                   "intermediate_size": I, "num_attention_heads": cfg.num_attention_heads,
                   "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "vocab_size": V, "tie_word_embeddings": cfg.tie_word_embeddings,
                   "kv_page_size": page, "rope_theta": cfg.rope_theta,
                   "rope_scaling_factor": cfg.rope_scaling.factor, "rms_norm_eps": cfg.rms_norm_eps,
                   "gemm_tuned": not args.no_gemm_tune},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    if not args.no_points:
        p_tok_s, p_s, p_flops = prefill()
        out["prefill"] = {"value": round(p_tok_s, 1), "tokens": 2048, "ms": round(p_s * 1e3, 3),
                          "frac": round(p_flops / p_s / PEAK_FLOPS[args.dtype], 4)}
        pts = {}
        for b, steps in ((1, max(8, args.steps // 2)), (64, max(8, args.steps // 4))):
            pts[f"decode_b{b}"] = round(decode(b, steps, min(args.warmup, 4))[0], 1)
        out["points"] = pts
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
