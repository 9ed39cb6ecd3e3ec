"""Command line.  As the reference's binaries, it takes its options from one TOML file:
``--config <file>`` (default ``rustinfer.toml``; crates/infer-worker/src/bin/worker_main.rs:39-53).
Where the reference's worker then waits for requests over its sockets, this one takes
prompts as token ids from the command line or a file and prints the generated ids.

    python -m rustinfer_amd.cli --config run.toml --prompt-ids 1,2,3 --max-tokens 16
    python -m rustinfer_amd.cli random-model --model-config config.json --seed 0 --out DIR
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import List


def _parse_ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def cmd_random_model(argv) -> int:
    ap = argparse.ArgumentParser(prog="rustinfer random-model",
                                 description="write a model folder with random weights")
    ap.add_argument("--model-config", required=True, help="a config.json to take the sizes from")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--out", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--unit-norms", action="store_true", help="norm weights exactly 1")
    args = ap.parse_args(argv)
    import torch
    from .config.registry import resolve_architecture
    from .weights.random_init import write_random_model
    with open(args.model_config) as f:
        d = json.load(f)
    entry = resolve_architecture(d, args.model_config)
    cfg = entry.config_cls.from_dict(d, args.model_config)
    write_random_model(cfg, args.seed, args.out,
                       torch.bfloat16 if args.dtype == "bfloat16" else torch.float32,
                       norm_noise=not args.unit_norms)
    print(f"wrote {args.out}/config.json and model.safetensors (seed {args.seed})")
    return 0


def cmd_run(argv) -> int:
    ap = argparse.ArgumentParser(prog="rustinfer", description=__doc__.split("\n\n")[0])
    ap.add_argument("--config", default="rustinfer.toml", help="launch file (TOML)")
    ap.add_argument("--prompt-ids", action="append", default=[],
                    help="a prompt as token ids '1,2,3' (may be given several times)")
    ap.add_argument("--prompt-file", help="a file with one prompt of token ids per line")
    ap.add_argument("--max-tokens", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--stop", action="append", default=[],
                    help="a stop sequence as token ids '7,8' (may be given several times): a request "
                         "whose output ends with it is finished and the sequence is taken off")
    ap.add_argument("--logprobs", action="store_true",
                    help="also print ln p of every generated token and of the five most probable at its place")
    ap.add_argument("--profile-steps", type=int, default=0,
                    help="bracket this many steps with the profiler's start/stop "
                         "(the reference's --profile-cuda-steps)")
    args = ap.parse_args(argv)
    prompts = [_parse_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [_parse_ids(line) for line in f if line.strip()]
    if not prompts:
        ap.error("no prompt: give --prompt-ids or --prompt-file")
    from .config.model_config import ConfigError
    from .llm import LLM
    from .sampling.params import SamplingParams
    try:
        llm = LLM(config=args.config)
    except ConfigError as e:
        print(f"error: {e}", file=sys.stderr)
        return 2
    params = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k,
                            min_p=args.min_p, seed=args.seed, max_tokens=args.max_tokens,
                            ignore_eos=args.ignore_eos, logprobs=args.logprobs,
                            stop_sequences=tuple(tuple(_parse_ids(x)) for x in args.stop))
    if args.profile_steps > 0:
        import torch
        for p in prompts:
            llm.add_request(p, params)
        steps = 0
        torch.cuda.cudart().cudaProfilerStart()
        while llm.scheduler.has_work() and steps < args.profile_steps:
            llm.step()
            steps += 1
        torch.cuda.synchronize()
        torch.cuda.cudart().cudaProfilerStop()
        while llm.scheduler.has_work():
            llm.step()
        results = [r for r in llm.scheduler.finished]
        for r in sorted(results, key=lambda r: r.arrival):
            print(json.dumps({"request": r.request_id, "token_ids": r.output, "finish_reason": r.finish_reason}))
        return 0
    for res in llm.generate(prompts, params):
        line = {"request": res.request_id, "token_ids": res.token_ids, "finish_reason": res.finish_reason}
        if res.logprobs is not None:
            line["logprobs"] = res.logprobs
            line["top_logprobs"] = res.top_logprobs
        print(json.dumps(line))
    print(json.dumps({"stats": llm.last_stats}), file=sys.stderr)
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "random-model":
        return cmd_random_model(argv[1:])
    if argv and argv[0] == "run":
        argv = argv[1:]
    return cmd_run(argv)


if __name__ == "__main__":
    sys.exit(main())
