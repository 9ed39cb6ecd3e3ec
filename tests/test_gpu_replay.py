"""bin/trace_run driven as a user would, under four ways of cutting the same requests,
in 32-bit and in bfloat16, against the plain implementation."""
import numpy as np
import pytest

import plain_llama
from helpers import (TINY, TINY_MFMA, TOL, check_steps_against, cut_mixed, cut_portions, cut_tail_single,
                     cut_whole, page_size, random_requests, run_trace, scaled_tol)

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [1, 7, 33, 64, 100, 128, 2, 49], "B": [2, 3, 17, 40, 100, 129, 65, 200],
           "C": [1, 18, 130, 257, 64, 400, 33], "D": [2, 47, 129, 300, 16, 65]}


@pytest.fixture(scope="module")
def material(model_dirs, plain_models):
    out = {}
    for name in list(TINY) + list(TINY_MFMA):
        cfg, w = plain_models[name]
        reqs = random_requests(cfg["vocab_size"], LENGTHS[name], seed=11)
        out[name] = (reqs, {rid: plain_llama.forward(cfg, w, t) for rid, t in reqs.items()})
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("cut", ["whole", "tail_single", "portions", "mixed"])
def test_replay_matches_plain(model_dirs, material, tmp_path, name, dtype, cut):
    reqs, plain = material[name]
    max_tokens = 4 * 256
    if cut == "whole":
        steps = cut_whole(reqs)
    elif cut == "tail_single":
        steps = cut_tail_single(reqs, tail=32)
    elif cut == "portions":
        steps = cut_portions(reqs, seed=3)
    else:
        max_tokens = 384                      # so few pages that they are used again
        steps = cut_mixed(reqs, max_tokens, seed=5)
        assert max(len(s["entries"]) for s in steps) >= 3
    results = run_trace(model_dirs[name], dtype, steps, str(tmp_path), max_tokens, page=page_size(name))
    worst = check_steps_against(steps, results, plain, TOL[dtype], f"{name}/{dtype}/{cut}")
    print(f"{name} {dtype} {cut}: {len(steps)} steps, worst |diff| {worst:.3e}")


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name", ["C", "D"])
@pytest.mark.parametrize("cut", ["whole", "tail_single", "portions", "mixed"])
def test_replay_on_the_matrix_core_kernels(model_dirs, material, tmp_path, name, dtype, cut):
    """The same four cuts on configurations whose bfloat16 path runs the MFMA attention kernels,
    the fused projection/rotation kernel, tile-ordered weights and K-split products."""
    reqs, plain = material[name]
    max_tokens = 4 * 512
    if cut == "whole":
        steps = cut_whole(reqs)
    elif cut == "tail_single":
        steps = cut_tail_single(reqs, tail=32)
    elif cut == "portions":
        steps = cut_portions(reqs, seed=4)
    else:
        max_tokens = 1024
        steps = cut_mixed(reqs, max_tokens, seed=6)
        assert max(len(s["entries"]) for s in steps) >= 3
    results = run_trace(model_dirs[name], dtype, steps, str(tmp_path), max_tokens, page=page_size(name))
    worst = check_steps_against(steps, results, plain, scaled_tol(dtype, plain), f"{name}/{dtype}/{cut}")
    print(f"{name} {dtype} {cut}: {len(steps)} steps, worst |diff| {worst:.3e}")


def test_step_without_wanted_logits_writes_no_file(model_dirs, material, tmp_path):
    reqs, plain = material["A"]
    toks = reqs["r3"]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:40], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[40:], "want": [len(toks) - 41]}], "end": ["x"]}]
    results = run_trace(model_dirs["A"], "float32", steps, str(tmp_path), 64)
    assert 0 not in results
    assert np.max(np.abs(results[1][0] - plain["r3"][-1])) <= TOL["float32"]
