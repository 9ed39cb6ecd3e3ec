"""Shared test material: two tiny configurations that differ in every size and option,
random model folders, ways of cutting requests into steps, and tolerances."""
from __future__ import annotations

import functools
import json
import os
import subprocess
import sys
from typing import Dict, List, Sequence

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# name -> (config.json contents, page size, weight seed)
TINY = {
    "A": (dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=64,
               intermediate_size=176, num_hidden_layers=2, num_attention_heads=4,
               num_key_value_heads=2, head_dim=16, vocab_size=256, max_position_embeddings=128,
               rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True,
               hidden_act="silu", eos_token_id=[255]), 16, 0),
    "B": (dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=160,
               intermediate_size=416, num_hidden_layers=3, num_attention_heads=5,
               num_key_value_heads=1, head_dim=32, vocab_size=384, max_position_embeddings=256,
               rms_norm_eps=1e-6, rope_theta=500000.0, tie_word_embeddings=False,
               rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                 high_freq_factor=4.0, original_max_position_embeddings=32),
               hidden_act="silu", eos_token_id=383), 8, 1),
}

# Two more, sized so that the bfloat16 engine takes its matrix-core kernels (head sizes 64 and 128,
# pages of 16, products long enough to be split over K), still small enough for the plain
# implementation.
TINY_MFMA = {
    "C": (dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=256,
               intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
               num_key_value_heads=2, head_dim=64, vocab_size=512, max_position_embeddings=512,
               rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                 high_freq_factor=4.0, original_max_position_embeddings=64),
               hidden_act="silu", eos_token_id=[511]), 16, 2),
    "D": (dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=384,
               intermediate_size=1056, num_hidden_layers=2, num_attention_heads=6,
               num_key_value_heads=2, head_dim=128, vocab_size=777, max_position_embeddings=400,
               rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=False,
               hidden_act="silu", eos_token_id=776), 32, 3),
}

# Largest absolute difference of logits from the plain implementation, for the tiny configurations:
# their logits have a standard deviation of 0.16 (A) to 0.4 (D) and reach about 1.5.
TOL = {"float32": 2e-5, "bfloat16": 1.5e-2}


def scaled_tol(dtype: str, plain_logits) -> float:
    """The same bound for models whose logits are larger (a row's standard deviation grows with the
    root of the width: 0.02 * sqrt(hidden) with these random weights): ``TOL`` is for a standard
    deviation of 0.4 and grows in proportion beyond that.  Rounding errors are relative."""
    std = max(float(np.std(v)) for v in plain_logits.values())
    return TOL[dtype] * max(1.0, std / 0.4)


def check_rounding_noise(steps, results, plain_logits, label=""):
    """For bfloat16 runs of wide models, where a bound on single logits says little: the error of
    a row of logits must look like rounding noise, the same at every position.  With r_i the
    root-mean-square error of wanted row i against the plain implementation and s the standard
    deviation of the plain logits: the median r is at most 2 % of s (observed 0.5 % at two layers
    of width 384, 1.1 % at three of width 2,560; a wrong key, page or weight tile gives 10 % and
    more), no row's r is above 1.75 times the median (a fault at a page's edge or a portion's start
    stands out against its neighbours; observed 1.3), and no single logit is off by more than 6
    times that.  Returns (median r / s, largest r / median)."""
    pos: Dict[str, int] = {}
    rows = []
    for st in steps:
        got = results.get(st["step"])
        row = 0
        for e in st["entries"]:
            p0 = pos.get(e["id"], 0)
            for w in e["want"]:
                err = got[row].astype(np.float64) - plain_logits[e["id"]][p0 + w]
                rows.append((float(np.sqrt(np.mean(err * err))), float(np.abs(err).max()), st["step"], e["id"], p0 + w))
                row += 1
            pos[e["id"]] = p0 + len(e["tokens"])
    s = max(float(np.std(v)) for v in plain_logits.values())
    med = float(np.median([r[0] for r in rows]))
    assert med <= 0.02 * s, f"{label}: median row error {med:.3e} is {med / s:.1%} of the logits' deviation {s:.3f}"
    for rms, mx, step, rid, p in rows:
        assert rms <= 1.75 * med and mx <= 6 * 1.75 * med, (
            f"{label}: step {step} request {rid} position {p}: row error {rms:.3e} (largest {mx:.3e}) "
            f"against a median of {med:.3e}")
    return med / s, max(r[0] for r in rows) / med


def run_steps(engine, steps):
    """Run trace steps (as ``cut_*`` make them) on an engine in this process; step -> logits array."""
    from rustinfer_amd.engine import StepEntry
    results = {}
    for st in steps:
        lg = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]])
        if lg.shape[0]:
            results[st["step"]] = lg.cpu().numpy()
        for rid in st["end"]:
            engine.release(rid)
    return results


def make_model_dir(name: str, out_dir: str) -> str:
    from rustinfer_amd.config import LlamaConfig
    from rustinfer_amd.weights import write_random_model
    cfg_dict, _page, seed = {**TINY, **TINY_MFMA}[name]
    cfg = LlamaConfig.from_dict(cfg_dict)
    write_random_model(cfg, seed, out_dir)
    return out_dir


def page_size(name: str) -> int:
    return {**TINY, **TINY_MFMA}[name][1]


def random_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, vocab, n).tolist() for i, n in enumerate(lengths)}


# ---------------------------------------------------------------------------
# ways of cutting requests into steps; every token's logits are wanted
# ---------------------------------------------------------------------------
def _entry(rid, toks):
    return {"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}


def cut_whole(requests):
    """Each request alone and whole."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [_entry(rid, toks)], "end": [rid]})
    return steps


def cut_tail_single(requests, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail) if len(toks) > 1 else 1
        steps.append({"step": len(steps), "entries": [_entry(rid, toks[:head])], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [_entry(rid, toks[i:i + 1])], "end": []})
        steps[-1]["end"] = [rid]
    return steps


def cut_portions(requests, seed=0, sizes=(5, 2, 17, 3, 2, 31, 8, 2, 64, 1)):
    """Portions of changing size, down to two tokens, one request at a time."""
    steps = []
    rng = np.random.default_rng(seed)
    for rid, toks in requests.items():
        pos, k = 0, int(rng.integers(0, len(sizes)))
        while pos < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - pos)
            k += 1
            steps.append({"step": len(steps), "entries": [_entry(rid, toks[pos:pos + n])], "end": []})
            pos += n
        steps[-1]["end"] = [rid]
    return steps


def cut_mixed(requests, max_tokens, seed=0, max_live=4, tail=8):
    """Up to ``max_live`` live requests: portions of some beside single tokens of others,
    some left out of a step; a new request starts as soon as the pool (``max_tokens``, each
    request rounded up to 64) has room, so pages of finished requests are used again."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}          # rid -> position
    steps = []

    def rounded(n):
        return (n + 63) // 64 * 64

    while waiting or live:
        while waiting and len(live) < max_live:
            held = sum(rounded(len(requests[r])) for r in live)
            if held + rounded(len(waiting[0][1])) > max_tokens:
                break
            live[waiting.pop(0)[0]] = 0
        entries, ended = [], []
        rids = list(live)
        rng.shuffle(rids)
        for rid in rids:
            toks, pos = requests[rid], live[rid]
            if len(rids) > 1 and rng.random() < 0.25:
                continue                                    # left out of this step
            remaining = len(toks) - pos
            if remaining <= tail:
                n = 1                                       # decoding
            else:
                n = int(min(remaining - tail, rng.choice([2, 3, 5, 9, 16, 17, 24, 40])))
            entries.append(_entry(rid, toks[pos:pos + n]))
            live[rid] = pos + n
            if live[rid] == len(toks):
                ended.append(rid)
        if not entries:
            continue
        for rid in ended:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def cut_preempted(requests, max_tokens, seed=0, max_live=4, tail=8):
    """As ``cut_mixed``, but now and then the live request that has come furthest is ended after its
    entry of the step (what it holds goes back), returns to the front of the queue and starts again
    from its first token, as a preempted request is recomputed.  Each request is given up at most
    once.  Returns (steps, number of requests given up)."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}
    given_up = set()
    steps = []

    def rounded(n):
        return (n + 63) // 64 * 64

    while waiting or live:
        while waiting and len(live) < max_live:
            held = sum(rounded(len(requests[r])) for r in live)
            if held + rounded(len(waiting[0][1])) > max_tokens:
                break
            live[waiting.pop(0)[0]] = 0
        entries, ended = [], []
        rids = list(live)
        rng.shuffle(rids)
        for rid in rids:
            toks, pos = requests[rid], live[rid]
            if len(rids) > 1 and rng.random() < 0.2:
                continue
            remaining = len(toks) - pos
            n = 1 if remaining <= tail else int(min(remaining - tail, rng.choice([2, 3, 5, 9, 16, 17, 24, 40])))
            entries.append(_entry(rid, toks[pos:pos + n]))
            live[rid] = pos + n
            if live[rid] == len(toks):
                ended.append(rid)
        if not entries:
            continue
        ran = [e["id"] for e in entries if e["id"] not in ended and e["id"] not in given_up]
        if len(live) >= 3 and ran and rng.random() < 0.35:
            victim = max(ran, key=lambda r: live[r])
            if live[victim] >= 20:                          # it has something to lose
                given_up.add(victim)
                ended.append(victim)
                waiting.insert(0, (victim, requests[victim]))
        for rid in ended:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps, len(given_up)


def expected_tables(steps, page, num_pages):
    """The block tables a trace must produce under the rule "the smallest free page first": a
    simulation that shares nothing with the engine's cache manager.  A request takes pages when its
    tokens first need them, entry after entry in the order of the step, and gives them all back when
    it ends.  step -> [{"start": tokens cached before the entry, "table": pages after it}]."""
    free = list(range(num_pages))
    table: Dict[str, List[int]] = {}
    length: Dict[str, int] = {}
    out = {}
    for st in steps:
        rows = []
        for e in st["entries"]:
            rid, n = e["id"], len(e["tokens"])
            t, start = table.setdefault(rid, []), length.get(rid, 0)
            need = (start + n + page - 1) // page - len(t)
            free.sort()
            t.extend(free[:need])
            del free[:need]
            length[rid] = start + n
            rows.append({"start": start, "table": list(t)})
        for rid in st["end"]:
            free.extend(table.pop(rid, []))
            length.pop(rid, None)
        out[st["step"]] = rows
    return out


def cut_at_random(requests, max_tokens, seed=0, max_live=4):
    """A trace drawn at random: up to ``max_live`` live requests; a step takes some of them,
    each with one token, two, a random portion or all that is left; the places whose logits are
    wanted are none, the last, all or a random choice; now and then a request ends early."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}
    steps = []

    def rounded(n):
        return (n + 63) // 64 * 64

    while waiting or live:
        while waiting and len(live) < max_live:
            held = sum(rounded(len(requests[r])) for r in live)
            if held + rounded(len(waiting[0][1])) > max_tokens:
                break
            live[waiting.pop(0)[0]] = 0
        rids = list(live)
        rng.shuffle(rids)
        entries, ended = [], []
        for rid in rids:
            toks, pos = requests[rid], live[rid]
            if len(rids) > 1 and rng.random() < 0.3:
                continue
            rem = len(toks) - pos
            mode = rng.random()
            n = 1 if mode < 0.35 else min(2, rem) if mode < 0.5 else \
                int(rng.integers(1, min(rem, 48) + 1)) if mode < 0.9 else rem
            w = rng.random()
            want = [] if w < 0.2 else [n - 1] if w < 0.5 else list(range(n)) if w < 0.8 else \
                sorted(rng.choice(n, size=int(rng.integers(1, n + 1)), replace=False).tolist())
            entries.append({"id": rid, "tokens": toks[pos:pos + n], "want": want})
            live[rid] = pos + n
            if live[rid] == len(toks) or rng.random() < 0.03:
                ended.append(rid)
        if not entries:
            continue
        for rid in ended:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def check_steps_against(steps, results, plain_logits, tol, label=""):
    """``results``: step -> array [wanted, vocab].  Compares every wanted row with the plain
    implementation's logits at that request's position; returns the largest difference."""
    pos: Dict[str, int] = {}
    worst = 0.0
    for st in steps:
        got = results.get(st["step"])
        row = 0
        for e in st["entries"]:
            p0 = pos.get(e["id"], 0)
            for w in e["want"]:
                ref = plain_logits[e["id"]][p0 + w]
                diff = float(np.max(np.abs(got[row].astype(np.float64) - ref)))
                if not (diff <= tol):
                    raise AssertionError(
                        f"{label}: step {st['step']} request {e['id']} position {p0 + w} "
                        f"(place {w} of a portion of {len(e['tokens'])} starting at {p0}): "
                        f"|diff| = {diff:.3e} > {tol:.1e}")
                worst = max(worst, diff)
                row += 1
            pos[e["id"]] = p0 + len(e["tokens"])
        assert got is None or row == got.shape[0]
        for rid in st["end"]:
            pos.pop(rid, None)                  # a request that comes again starts from its first token
    return worst


def run_trace(model_dir, dtype, steps, out_dir, max_tokens, page=16, timeout=600):
    """Drive bin/trace_run as a user would; returns step -> logits array."""
    with open(os.path.join(model_dir, "config.json")) as f:
        vocab = json.load(f)["vocab_size"]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
           "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens),
           "--page-size", str(page)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {st['step']}", f"trace_run answered {line!r} to step {st['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    results = {}
    for st in steps:
        n = sum(len(e["want"]) for e in st["entries"])
        path = os.path.join(out_dir, f"{st['step']}.f32")
        if n:
            results[st["step"]] = np.fromfile(path, dtype="<f4").reshape(n, vocab)
        else:
            assert not os.path.exists(path)
    return results
