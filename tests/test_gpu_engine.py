"""The engine in process: the step function under different cuts, generation through the entry
point, sampling under cuts, running out of pages, long decoding, first tokens."""
import numpy as np
import pytest
import torch

import plain_llama
from helpers import TINY, TOL, check_steps_against, cut_at_random, page_size, random_requests

pytestmark = pytest.mark.gpu


def make_engine(model_dir, dtype, page, num_pages=64, max_requests=4, max_model_len=256, max_batch_tokens=512):
    from rustinfer_amd.engine import build_engine
    return build_engine(model_dir, dtype=dtype, page_size=page, num_pages=num_pages,
                        max_requests=max_requests, max_model_len=max_model_len,
                        max_batch_tokens=max_batch_tokens)


def plain_greedy(cfg, w, prompt, n, eos=()):
    toks, out = list(prompt), []
    for _ in range(n):
        t = plain_llama.greedy(plain_llama.forward(cfg, w, toks)[-1])
        out.append(t)
        toks.append(t)
        if t in eos:
            break
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_and_long_decoding(model_dirs, plain_models, name, dtype):
    """Positions 0, 1, 2 of a sequence, then decoding one by one to the model's longest length."""
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models[name]
    n = cfg["max_position_embeddings"]
    eng = make_engine(model_dirs[name], dtype, page_size(name), max_model_len=n)
    toks = random_requests(cfg["vocab_size"], [n], seed=21)["r0"]
    ref = plain_llama.forward(cfg, w, toks)
    worst = 0.0
    for i, t in enumerate(toks):
        lg = eng.step([StepEntry("x", [t], [0])])[0].double().cpu().numpy()
        d = np.max(np.abs(lg - ref[i]))
        assert d <= TOL[dtype], f"position {i}: {d}"
        worst = max(worst, d)
    eng.release("x")
    eng.cache.check()
    assert eng.cache.free_pages() == 64


@pytest.mark.parametrize("name", ["C", "D"])
def test_one_copy_of_the_weights(model_dirs, plain_models, name):
    """``tiled_weight_copy = False``: the projections keep the checkpoint's row-major weights
    only (half the memory); single tokens, short portions and long ones still give the plain
    logits, through the kernels that read row-major weights."""
    from rustinfer_amd.engine import StepEntry, build_engine
    cfg, w = plain_models[name]
    eng = build_engine(model_dirs[name], dtype="bfloat16", page_size=page_size(name), num_pages=64, max_requests=4,
                       max_model_len=256, max_batch_tokens=512, tiled_weight_copy=False)
    block = eng.model.layers[0]
    assert block.mixer.qkv.weight_tiled is None and block.mixer.qkv_fused is None and block.mixer.o.weight_tiled is None
    assert block.ffn.gate_up.weight_tiled is None and eng.model.lm_head.weight_tiled is None
    reqs = random_requests(cfg["vocab_size"], [120, 40, 30], seed=29)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    pos = {r: 0 for r in reqs}
    r0, r1, r2 = list(reqs)
    for step in ([(r0, 100)], [(r1, 5), (r2, 20)], [(r0, 1), (r1, 1), (r2, 1)], [(r0, 3), (r1, 1)], [(r0, 1), (r1, 30), (r2, 1)]):
        ents = [StepEntry(r, reqs[r][pos[r]:pos[r] + n], [n - 1]) for r, n in step]
        lg = eng.step(ents).double().cpu().numpy()
        for i, (r, n) in enumerate(step):
            assert np.max(np.abs(lg[i] - ref[r][pos[r] + n - 1])) <= TOL["bfloat16"], (step, r)
            pos[r] += n
    eng.cache.check()


@pytest.mark.parametrize("name", ["C", "D"])
def test_second_copies_of_the_first_weights_only(model_dirs, plain_models, name):
    """A budget that holds the second copies of the first layer and a little more (a model that
    fills most of the device): layers with and without them run side by side, one with the fused
    projection and the norms left to the products, the other with the plain kernels, and the
    logits are the plain implementation's; with random weights drawn part by part as well."""
    from rustinfer_amd.engine import StepEntry, build_engine
    cfg, w = plain_models[name]
    d, I = cfg["hidden_size"], cfg["intermediate_size"]
    qkv = (cfg["num_attention_heads"] + 2 * cfg["num_key_value_heads"]) * cfg["head_dim"]
    layer = 2 * (qkv * d + cfg["num_attention_heads"] * cfg["head_dim"] * d + 3 * I * d)
    eng = build_engine(model_dirs[name], dtype="bfloat16", page_size=page_size(name), num_pages=64, max_requests=4,
                       max_model_len=256, max_batch_tokens=512, tile_budget_bytes=layer + 2 * qkv * d)
    first, second = eng.model.layers[0], eng.model.layers[1]
    assert first.mixer.qkv_fused is not None and first.mixer.o.weight_tiled is not None
    assert first.ffn.gate_up.weight_tiled is not None and first.ffn.down.weight_tiled is not None
    assert second.mixer.qkv_fused is not None and second.mixer.o.weight_tiled is None       # what was left went to the next weight
    assert second.ffn.gate_up.weight_tiled is None and second.ffn.down.weight_tiled is None
    assert eng.model.lm_head.weight_tiled is None and eng.rt.tile_budget < 2 * qkv * d
    reqs = random_requests(cfg["vocab_size"], [120, 40, 30], seed=31)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    pos = {r: 0 for r in reqs}
    r0, r1, r2 = list(reqs)
    for step in ([(r0, 100)], [(r1, 5), (r2, 20)], [(r0, 1), (r1, 1), (r2, 1)], [(r0, 3), (r1, 1)], [(r0, 1), (r1, 30), (r2, 1)]):
        ents = [StepEntry(r, reqs[r][pos[r]:pos[r] + n], [n - 1]) for r, n in step]
        lg = eng.step(ents).double().cpu().numpy()
        for i, (r, n) in enumerate(step):
            assert np.max(np.abs(lg[i] - ref[r][pos[r] + n - 1])) <= TOL["bfloat16"], (step, r)
            pos[r] += n
    eng.cache.check()
    # random weights, drawn part by part: the same values whatever the budget
    full = build_engine(model_dirs[name], dtype="bfloat16", page_size=page_size(name), num_pages=16, max_requests=2,
                        max_model_len=64, random_weights_seed=3)
    part = build_engine(model_dirs[name], dtype="bfloat16", page_size=page_size(name), num_pages=16, max_requests=2,
                        max_model_len=64, random_weights_seed=3, tile_budget_bytes=layer)
    assert full.rt.tile_budget > 1 << 30 and part.model.layers[1].ffn.down.weight_tiled is None
    assert torch.equal(full.model.layers[1].ffn.down.weight, part.model.layers[1].ffn.down.weight)
    toks = reqs[r0][:20]
    a = full.step([StepEntry("x", toks, [19])]).double().cpu().numpy()
    b = part.step([StepEntry("x", toks, [19])]).double().cpu().numpy()
    assert np.max(np.abs(a - b)) <= 2 * TOL["bfloat16"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_does_not_grow_the_workspace_step_by_step(model_dirs, plain_models, dtype):
    """Steps launched eagerly: the buffers whose size follows the requests' lengths (partial
    results of the split attention kernels) are single buffers that grow now and then, not a new
    one for every length."""
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models["C"]
    eng = make_engine(model_dirs["C"], dtype, page_size("C"), num_pages=64, max_requests=4, max_batch_tokens=256)
    reqs = random_requests(cfg["vocab_size"], [150, 90], seed=23)
    eng.step([StepEntry(r, t[:40], []) for r, t in reqs.items()])
    seen = []
    for i in range(40, 90):
        eng.step([StepEntry(r, [t[i]], [0]) for r, t in reqs.items()])
        seen.append((len(eng.workspace._bufs), eng.workspace.nbytes()))
    assert seen[-1][0] == seen[5][0], seen[::8]                  # the same buffers after 50 steps as after 6
    assert seen[-1][1] <= 3 * seen[5][1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_traces_drawn_at_random(model_dirs, plain_models, name, dtype):
    """Several traces drawn at random (what a step holds, how long its portions are, which
    logits are wanted, when a request ends) in a pool so small that pages go round."""
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models[name]
    for max_tokens, seed in ((256, 0), (256, 1), (512, 2)):
        num_pages = max_tokens // 16
        eng = make_engine(model_dirs[name], dtype, 16, num_pages=num_pages, max_requests=8,
                          max_model_len=num_pages * 16, max_batch_tokens=8192)
        rng = np.random.default_rng(seed)
        longest = min(cfg["max_position_embeddings"], max_tokens)
        lengths = [int(rng.choice([1, 2, 3, rng.integers(4, 40), rng.integers(40, longest + 1)])) for _ in range(9)]
        requests = random_requests(cfg["vocab_size"], lengths, seed=seed + 100)
        plain = {r: plain_llama.forward(cfg, w, t) for r, t in requests.items()}
        steps = cut_at_random(requests, max_tokens, seed=seed)
        results = {}
        for st in steps:
            lg = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]])
            if lg.shape[0]:
                results[st["step"]] = lg.cpu().numpy()
            for rid in st["end"]:
                eng.release(rid)
        check_steps_against(steps, results, plain, TOL[dtype], f"{name} {dtype} seed {seed}")
        eng.cache.check()
        assert eng.cache.free_pages() == num_pages


@pytest.mark.parametrize("name", ["A", "B"])
def test_pages_are_not_cleared_and_stale_contents_do_not_matter(model_dirs, plain_models, name):
    """Poison every page, run; free, poison again with other values, run another request on the
    same pages: logits equal the plain implementation's both times."""
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models[name]
    eng = make_engine(model_dirs[name], "float32", page_size(name), num_pages=12, max_model_len=96)
    reqs = random_requests(cfg["vocab_size"], [90, 77], seed=22)
    for poison, (rid, toks) in zip((float("nan"), 1e30), reqs.items()):
        for g in eng.cache.groups:
            g.k_pool.fill_(poison)
            g.v_pool.fill_(poison)
        ref = plain_llama.forward(cfg, w, toks)
        lg = eng.step([StepEntry(rid, toks[:50], list(range(50)))]).double().cpu().numpy()
        assert np.max(np.abs(lg - ref[:50])) <= TOL["float32"]
        lg = eng.step([StepEntry(rid, toks[50:], list(range(len(toks) - 50)))]).double().cpu().numpy()
        assert np.max(np.abs(lg - ref[50:])) <= TOL["float32"]
        eng.release(rid)


def test_row_order_and_page_ids_do_not_matter(model_dirs, plain_models):
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models["A"]
    reqs = random_requests(cfg["vocab_size"], [20, 31, 9], seed=23)
    outs = []
    for order in (["r0", "r1", "r2"], ["r2", "r0", "r1"]):
        eng = make_engine(model_dirs["A"], "float32", 16)
        if order[0] == "r2":                       # shift page ids: another request holds the first pages
            eng.step([StepEntry("hold", [1] * 40, [])])
        lg = eng.step([StepEntry(r, reqs[r], [len(reqs[r]) - 1]) for r in order]).cpu()
        outs.append({r: lg[i] for i, r in enumerate(order)})
    for r in reqs:
        assert torch.allclose(outs[0][r], outs[1][r], atol=1e-6, rtol=0)
        ref = plain_llama.forward(cfg, w, reqs[r])[-1]
        assert np.max(np.abs(outs[0][r].double().numpy() - ref)) <= TOL["float32"]


def test_step_refuses_bad_batches(model_dirs):
    from rustinfer_amd.cache import OutOfPages
    from rustinfer_amd.engine import StepEntry, StepError
    eng = make_engine(model_dirs["A"], "float32", 16, num_pages=4, max_model_len=128, max_batch_tokens=100)
    with pytest.raises(StepError, match="empty batch"):
        eng.step([])
    with pytest.raises(StepError, match="no tokens"):
        eng.step([StepEntry("a", [], [])])
    with pytest.raises(StepError, match="outside"):
        eng.step([StepEntry("a", [256], [])])
    with pytest.raises(StepError, match="wanted place"):
        eng.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(StepError, match="twice"):
        eng.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(StepError, match="max_batch_tokens"):
        eng.step([StepEntry("a", [1] * 101, [])])
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1] * 65, [])])
    assert eng.cache.free_pages() == 4 and not eng.cache.has_request("a")   # nothing changed
    eng.step([StepEntry("a", [1] * 64, [])])
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1], [])])
    eng.cache.check()


@pytest.mark.parametrize("name", ["A", "B"])
def test_generate_greedy_matches_plain(model_dirs, plain_models, name):
    """Greedy generation through the entry point, 32-bit: the same tokens as the plain
    implementation, for prompts of 1..129 tokens, under two ways of batching."""
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models[name]
    lengths, steps = ([1, 7, 33, 64], 16) if name == "A" else ([2, 3, 17, 40, 100, 129], 24)
    prompts = list(random_requests(cfg["vocab_size"] - 1, lengths, seed=24).values())
    want = [plain_greedy(cfg, w, p, steps) for p in prompts]
    for opts in (dict(max_batch_tokens=4096, chunked_prefill_size=0, max_batch_seqs=8),
                 dict(max_batch_tokens=16, chunked_prefill_size=5, max_batch_seqs=3)):
        llm = LLM(model=model_dirs[name], dtype="float32", paged_block_size=page_size(name),
                  num_blocks=96, max_model_len=cfg["max_position_embeddings"], **opts)
        res = llm.generate(prompts, SamplingParams(max_tokens=steps, ignore_eos=True))
        assert [r.token_ids for r in res] == want
        assert all(r.finish_reason == "length" for r in res)
        llm.engine.cache.check()
        assert llm.engine.cache.free_pages() == 96


def test_generate_bfloat16_stays_close(model_dirs, plain_models):
    """bfloat16 generation: every generated token is one the plain implementation also ranks at
    the top, up to the bfloat16 tolerance on logits."""
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models["B"]
    prompts = list(random_requests(cfg["vocab_size"] - 1, [17, 40, 100], seed=25).values())
    llm = LLM(model=model_dirs["B"], dtype="bfloat16", paged_block_size=8, num_blocks=96,
              max_model_len=256, max_batch_seqs=4)
    res = llm.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    for p, r in zip(prompts, res):
        toks = list(p)
        for t in r.token_ids:
            logits = plain_llama.forward(cfg, w, toks)[-1]
            assert logits.max() - logits[t] <= 2 * TOL["bfloat16"]
            toks.append(t)


def test_eos_and_max_tokens_finish_requests(model_dirs, plain_models):
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models["A"]
    prompt = random_requests(255, [12], seed=26)["r0"]
    full = plain_greedy(cfg, w, prompt, 10)
    # make the fourth generated token the end-of-sequence id of this run
    llm = LLM(model=model_dirs["A"], dtype="float32", num_blocks=16, max_model_len=128)
    llm.eos_ids = (full[3],)
    res = llm.generate([prompt, prompt], [SamplingParams(max_tokens=10), SamplingParams(max_tokens=10, ignore_eos=True)])
    first = full.index(full[3])
    assert res[0].token_ids == full[:first + 1] and res[0].finish_reason == "eos"   # the token that ends it is emitted
    assert res[1].token_ids == full and res[1].finish_reason == "length"
    one = llm.generate([prompt], SamplingParams(max_tokens=1, ignore_eos=True))[0]
    assert one.token_ids == full[:1] and one.finish_reason == "length"


def test_stop_sequences_end_generation(model_dirs, plain_models):
    """A stop sequence of two generated tokens ends the request where it first appears, and is not
    part of the result; the pipelined loop has run a step ahead by then."""
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models["A"]
    prompt = random_requests(255, [12], seed=26)["r0"]
    full = plain_greedy(cfg, w, prompt, 10)
    stop = (full[4], full[5])
    first = next(i for i in range(9) if (full[i], full[i + 1]) == stop)
    llm = LLM(model=model_dirs["A"], dtype="float32", num_blocks=16, max_model_len=128)
    res = llm.generate([prompt, prompt], [SamplingParams(max_tokens=10, ignore_eos=True, stop_sequences=(stop,)),
                                          SamplingParams(max_tokens=10, ignore_eos=True)])
    assert res[0].token_ids == full[:first] and res[0].finish_reason == "stop"
    assert res[1].token_ids == full and res[1].finish_reason == "length"
    llm.engine.cache.check()
    assert llm.engine.cache.free_pages() == 16


def test_temperature_sampling_is_the_same_under_every_cut(model_dirs, plain_models):
    """Temperature 0.8 with a fixed seed: the same tokens alone, batched, and with prompts cut
    into small portions, and they are the plain sampler's tokens for the same draws."""
    from rustinfer_amd import LLM, SamplingParams
    from rustinfer_amd.sampling import uniform_draw
    cfg, w = plain_models["B"]
    prompts = list(random_requests(cfg["vocab_size"] - 1, [2, 3, 17, 40, 100, 129], seed=27).values())
    params = [SamplingParams(temperature=0.8, seed=1000 + i, max_tokens=24, ignore_eos=True,
                             top_k=(0, 40)[i % 2], top_p=(1.0, 0.95)[i % 2]) for i in range(len(prompts))]
    runs = []
    for opts in (dict(max_batch_seqs=1), dict(max_batch_seqs=8),
                 dict(max_batch_seqs=4, max_batch_tokens=12, chunked_prefill_size=5)):
        llm = LLM(model=model_dirs["B"], dtype="float32", paged_block_size=8, num_blocks=128,
                  max_model_len=256, **opts)
        runs.append([r.token_ids for r in llm.generate(prompts, params)])
    assert runs[0] == runs[1] == runs[2]
    for p, sp, got in zip(prompts[:3], params, runs[0]):
        toks = list(p)
        for t in got:
            logits = plain_llama.forward(cfg, w, toks)[-1]
            order, wts = plain_llama.filtered_distribution(logits, sp.temperature, sp.top_k, sp.top_p, sp.min_p)
            assert t == plain_llama.sample_from(order, wts, uniform_draw(sp.seed, len(toks)))
            toks.append(t)


def test_generate_returns_log_probabilities(model_dirs, plain_models):
    """SamplingParams.logprobs: ln p of each generated token and the five most probable tokens at
    its place, as the plain sampler computes them; a greedy request gets the log-softmax of the
    raw logits and no lists; the tokens are those of a run without log-probabilities, and a request
    that did not ask gets none."""
    from rustinfer_amd import LLM, SamplingParams
    from rustinfer_amd.sampling import uniform_draw
    cfg, w = plain_models["B"]
    prompts = list(random_requests(cfg["vocab_size"] - 1, [3, 17, 40, 9], seed=33).values())
    params = [SamplingParams(temperature=0.8, seed=7, max_tokens=10, ignore_eos=True, top_p=0.9, logprobs=True),
              SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True, logprobs=True),
              SamplingParams(temperature=1.2, seed=8, max_tokens=10, ignore_eos=True, top_k=4, logprobs=True),
              SamplingParams(temperature=0.9, seed=9, max_tokens=10, ignore_eos=True)]
    llm = LLM(model=model_dirs["B"], dtype="float32", paged_block_size=8, num_blocks=128, max_model_len=256,
              max_batch_seqs=4)
    res = llm.generate(prompts, params)
    import dataclasses
    plain_params = [dataclasses.replace(sp, logprobs=False) for sp in params]
    assert [r.token_ids for r in llm.generate(prompts, plain_params)] == [r.token_ids for r in res]
    assert res[3].logprobs is None and res[3].top_logprobs is None
    for p, sp, r in zip(prompts[:3], params, res):
        assert len(r.logprobs) == len(r.top_logprobs) == len(r.token_ids) == 10
        toks = list(p)
        for t, lp, top in zip(r.token_ids, r.logprobs, r.top_logprobs):
            logits = plain_llama.forward(cfg, w, toks)[-1]
            tok, want_lp, want_top = plain_llama.sample_with_logprobs(
                logits, sp.temperature or 1.0, sp.top_k, sp.top_p, sp.min_p,
                uniform_draw(sp.seed, len(toks)) if not sp.is_greedy else 0.0, sp.is_greedy)
            assert t == tok and abs(lp - want_lp) < 1e-3, (t, tok, lp, want_lp)
            assert [i for i, _ in top] == [i for i, _ in want_top]
            assert all(abs(a - b) < 1e-3 for (_, a), (_, b) in zip(top, want_top))
            toks.append(t)


def test_running_out_of_pages_preempts_and_recomputes(model_dirs, plain_models):
    """A pool too small for all requests at once: some are preempted, put back at the front and
    recomputed; every request still gets exactly the plain implementation's tokens."""
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models["A"]
    prompts = list(random_requests(255, [30, 28, 33, 5, 40], seed=28).values())
    want = [plain_greedy(cfg, w, p, 40) for p in prompts]
    llm = LLM(model=model_dirs["A"], dtype="float32", paged_block_size=16, num_blocks=11,
              max_model_len=128, max_batch_seqs=4, max_batch_tokens=64)
    res = llm.generate(prompts, SamplingParams(max_tokens=40, ignore_eos=True))
    assert [r.token_ids for r in res] == want
    assert llm.scheduler.stats["preemptions"] > 0 and sum(r.preemptions for r in res) > 0
    llm.engine.cache.check()
    assert llm.engine.cache.free_pages() == 11
    # a request that cannot run even alone ends with an error and holds nothing
    # a request that cannot run even alone ends with an error and holds nothing: a prompt of more
    # pages than the pool has, and one that outgrows the pool while it decodes alone
    res = llm.generate([[1] * 130, [2] * 5, [3] * 100],
                       [SamplingParams(max_tokens=100, ignore_eos=True), SamplingParams(max_tokens=3, ignore_eos=True),
                        SamplingParams(max_tokens=110, ignore_eos=True)])
    assert res[0].finish_reason == "error" and res[0].token_ids == []
    assert res[1].finish_reason == "length" and len(res[1].token_ids) == 3
    assert res[2].finish_reason == "length" and len(res[2].token_ids) == 29      # the token that would be the 129th is still emitted
    assert llm.engine.cache.free_pages() == 11
    small = LLM(model=model_dirs["A"], dtype="float32", paged_block_size=16, num_blocks=4,
                max_model_len=128, max_batch_seqs=2, max_batch_tokens=64)
    res = small.generate([[3] * 40, [4] * 70], SamplingParams(max_tokens=80, ignore_eos=True))
    assert res[0].finish_reason == "error" and len(res[0].token_ids) == 25       # 64 tokens fit, the 65th key does not
    assert res[1].finish_reason == "error" and res[1].token_ids == []            # five pages of prompt, four in the pool
    assert small.engine.cache.free_pages() == 4


def test_requests_that_arrive_while_others_run_under_a_small_pool(model_dirs, plain_models):
    """The serving loop as a server drives it: requests are added between steps, prompts are cut
    into portions of 7 under a budget of 48 tokens a step, graphs replay, sampled tokens reach the
    host a step late, and a pool of 10 pages for 8 live requests forces preemptions; every request
    ends with the plain implementation's greedy tokens (to its length, its end-of-sequence token
    or the model's longest length) and the pool is whole again."""
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models["A"]
    rng = np.random.default_rng(5)
    llm = LLM(model=model_dirs["A"], dtype="float32", paged_block_size=16, num_blocks=10, max_batch_seqs=8,
              max_model_len=128, chunked_prefill_size=7, max_batch_tokens=48, capture_sizes=(1, 2, 4, 8))
    prompts = [rng.integers(0, cfg["vocab_size"], int(rng.integers(1, 60))).tolist() for _ in range(24)]
    params = [SamplingParams(max_tokens=int(rng.integers(1, 70)), ignore_eos=bool(rng.random() < 0.3)) for _ in prompts]
    waiting, reqs, steps = list(range(len(prompts))), {}, 0
    while waiting or llm.scheduler.has_work() or llm._inflight is not None:
        for _ in range(int(rng.integers(0, 3))):
            if waiting:
                i = waiting.pop(0)
                reqs[i] = llm.add_request(prompts[i], params[i])
        llm.step()
        steps += 1
        assert steps < 5000
    llm.drain()
    memo = {}

    def plain_next(toks):
        if toks not in memo:
            memo[toks] = plain_llama.greedy(plain_llama.forward(cfg, w, list(toks))[-1])
        return memo[toks]

    for i, r in reqs.items():
        toks, want = tuple(prompts[i]), []
        for _ in range(min(params[i].max_tokens, 128 - len(prompts[i]) + 1)):
            want.append(plain_next(toks))
            toks += (want[-1],)
            if not params[i].ignore_eos and want[-1] in llm.eos_ids:
                break
        assert r.output == want, (i, r.finish_reason, r.preemptions)
    assert llm.scheduler.stats["preemptions"] > 0 and llm.engine.graph_replays > 100
    llm.engine.cache.check()
    assert llm.engine.cache.free_pages() == 10


def test_tokens_given_up_for_alignment_change_no_output(model_dirs, plain_models):
    """Steps a token or two over a multiple of 16 give them back to a prompt portion
    (``step_token_align``): the same greedy tokens as without, which are the plain implementation's."""
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models["A"]
    rng = np.random.default_rng(11)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in (3, 5, 90, 4, 70, 110)]
    outs, trimmed = [], []
    for align in (0, 16):
        llm = LLM(model=model_dirs["A"], dtype="float32", paged_block_size=16, num_blocks=64, max_batch_seqs=8,
                  max_model_len=160, chunked_prefill_size=16, max_batch_tokens=64, step_token_align=align)
        cut = llm.scheduler._trim_to_alignment

        def counting(step, cut=cut):
            before = step.num_tokens
            cut(step)
            trimmed.append(before - step.num_tokens)

        llm.scheduler._trim_to_alignment = counting
        reqs = []
        for i, p in enumerate(prompts):                 # a new request every third step, beside those that decode
            reqs.append(llm.add_request(p, SamplingParams(max_tokens=24, ignore_eos=True)))
            for _ in range(3):
                llm.step()
        while llm.scheduler.has_work() or llm._inflight is not None:
            llm.step()
        llm.drain()
        outs.append([r.output for r in reqs])
        llm.engine.cache.check()
        if align == 0:
            assert not any(trimmed)
    assert outs[0] == outs[1] and sum(1 for t in trimmed if t > 0) >= 3 and max(trimmed) <= 2
    toks = list(prompts[2])
    for want in outs[1][2][:6]:
        assert plain_llama.greedy(plain_llama.forward(cfg, w, toks)[-1]) == want
        toks.append(want)


def test_a_failing_kernel_leaves_the_cache_as_it_was(model_dirs, plain_models, monkeypatch):
    """A kernel refuses its operands in the third layer of a mixed step: every request is as long
    as before, the request the step started is gone, the pages are free again; the same step then
    runs and gives the plain implementation's logits."""
    from rustinfer_amd.engine import StepEntry
    from rustinfer_amd.kernels import ops
    cfg, w = plain_models["B"]
    reqs = random_requests(cfg["vocab_size"], [30, 21, 12], seed=41)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    eng = make_engine(model_dirs["B"], "float32", 8, num_pages=16)
    eng.step([StepEntry("r0", reqs["r0"][:11], []), StepEntry("r1", reqs["r1"][:20], [])])
    before = ({r: eng.cache.kv_len(r) for r in eng.cache.live_requests()}, eng.cache.free_pages(),
              eng.cache.slots.available, [list(eng.cache.table(0, r)) for r in ("r0", "r1")])
    step = [StepEntry("r0", reqs["r0"][11:], [18]), StepEntry("r2", reqs["r2"], [11]), StepEntry("r1", reqs["r1"][20:], [0])]
    real, calls = ops.paged_attention, [0]

    def fails_in_the_third_layer(*a, **k):
        calls[0] += 1
        if calls[0] == 3:
            raise ops.KernelError("paged_attention: refused for the test")
        return real(*a, **k)
    monkeypatch.setattr(ops, "paged_attention", fails_in_the_third_layer)
    with pytest.raises(ops.KernelError, match="refused for the test"):
        eng.step(step)
    eng.cache.check()
    assert before == ({r: eng.cache.kv_len(r) for r in eng.cache.live_requests()}, eng.cache.free_pages(),
                      eng.cache.slots.available, [list(eng.cache.table(0, r)) for r in ("r0", "r1")])
    assert not eng.cache.has_request("r2")
    monkeypatch.setattr(ops, "paged_attention", real)
    lg = eng.step(step).double().cpu().numpy()
    for row, r in enumerate(("r0", "r2", "r1")):
        assert np.max(np.abs(lg[row] - ref[r][-1])) <= TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_references_decoder_vector(tmp_path, dtype):
    """The reference's one model-level test (crates/infer-worker/src/models/decoder.rs:475-603):
    hidden 16, 2 heads of 8, intermediate 32, vocabulary 64, one layer, weights ((i % 7) - 3) * 0.01,
    norms 1; prompts [1, 2, 3, 4, 5] and [10, 20, 30] as one ragged batch give the first tokens
    that each gives alone.  Here also: the logits are the plain implementation's."""
    from rustinfer_amd.engine import StepEntry, build_engine
    from rustinfer_amd.weights import write_safetensors
    import json
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=16, num_attention_heads=2, num_key_value_heads=2,
               intermediate_size=32, vocab_size=64, num_hidden_layers=1, rms_norm_eps=1e-5, rope_theta=1e4,
               max_position_embeddings=64, tie_word_embeddings=False)
    pat = lambda *shape: (((torch.arange(int(np.prod(shape))) % 7) - 3).float() * 0.01).reshape(shape)
    p = "model.layers.0."
    w = {"model.embed_tokens.weight": pat(64, 16), "model.norm.weight": torch.ones(16), "lm_head.weight": pat(64, 16),
         p + "input_layernorm.weight": torch.ones(16), p + "post_attention_layernorm.weight": torch.ones(16),
         p + "self_attn.q_proj.weight": pat(16, 16), p + "self_attn.k_proj.weight": pat(16, 16),
         p + "self_attn.v_proj.weight": pat(16, 16), p + "self_attn.o_proj.weight": pat(16, 16),
         p + "mlp.gate_proj.weight": pat(32, 16), p + "mlp.up_proj.weight": pat(32, 16),
         p + "mlp.down_proj.weight": pat(16, 32)}
    if dtype == "bfloat16":
        w = {n: t.to(torch.bfloat16) for n, t in w.items()}
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    write_safetensors(str(tmp_path / "model.safetensors"), w)
    pcfg, pw = plain_llama.read_model(str(tmp_path))
    p0, p1 = [1, 2, 3, 4, 5], [10, 20, 30]
    batch = build_engine(str(tmp_path), dtype=dtype, page_size=1, num_pages=16, max_requests=3, max_model_len=16)
    # pages of one token and the reference's block tables, [0..4] and [8, 9, 10]: a third request
    # holds the pages in between
    lg = batch.step([StepEntry(0, p0, [4]), StepEntry("between", [0, 0, 0], []), StepEntry(1, p1, [2])])
    assert batch.cache.table(0, 0) == [0, 1, 2, 3, 4] and batch.cache.table(0, 1) == [8, 9, 10]
    lg = lg.double().cpu().numpy()
    alone = []
    for prompt in (p0, p1):
        eng = build_engine(str(tmp_path), dtype=dtype, page_size=1, num_pages=8, max_requests=1, max_model_len=8)
        alone.append(eng.step([StepEntry(0, prompt, [len(prompt) - 1])])[0].double().cpu().numpy())
    for i, prompt in enumerate((p0, p1)):
        want = plain_llama.forward(pcfg, pw, prompt)[-1]
        assert np.max(np.abs(lg[i] - want)) <= TOL[dtype] and np.max(np.abs(alone[i] - want)) <= TOL[dtype]
        # 32-bit: the same sums in the same order; bfloat16: products of 11 rows and of 5 are cut
        # differently over K, and a logit of 0.25 has steps of 1e-3
        assert np.max(np.abs(lg[i] - alone[i])) <= (1e-6 if dtype == "float32" else 2e-3)
        assert int(np.argmax(lg[i])) == int(np.argmax(alone[i])) and 0 <= int(np.argmax(lg[i])) < 64
        if dtype == "float32":
            assert int(np.argmax(lg[i])) == plain_llama.greedy(want)


def test_command_line_and_toml(model_dirs, plain_models, tmp_path):
    import json
    import subprocess
    import sys
    from helpers import ROOT
    cfg, w = plain_models["A"]
    prompt = random_requests(255, [9], seed=29)["r0"]
    toml = tmp_path / "run.toml"
    toml.write_text(f'model = "{model_dirs["A"]}"\ndtype = "float32"\nmax_model_len = 128\n'
                    f'num_blocks = 16\npaged_block_size = 16\nmax_batch_seqs = 2\nport = 8102\n'
                    f'capture_sizes = [1, 2]\n[cuda_memory]\nkernel_workspace_mib = 256\n')
    r = subprocess.run([sys.executable, f"{ROOT}/bin/rustinfer", "--config", str(toml), "--prompt-ids",
                        ",".join(map(str, prompt)), "--max-tokens", "6", "--ignore-eos"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["token_ids"] == plain_greedy(cfg, w, prompt, 6)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_graph_replay_equals_eager_launches(model_dirs, plain_models, dtype):
    """Steps of single tokens replay a captured graph.  Every replay is checked against an
    engine that launches eagerly and against the plain implementation, with batches that
    shrink and grow (padding rows), prompt steps in between and requests that end."""
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models["A"]
    reqs = random_requests(cfg["vocab_size"], [50, 23, 64, 31, 50], seed=31)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    eager = make_engine(model_dirs["A"], dtype, 16, max_requests=8)
    graph = make_engine(model_dirs["A"], dtype, 16, max_requests=8)
    graph.enable_graphs(True, (1, 2, 4, 8))
    pos = {r: 0 for r in reqs}
    live = []
    plan = [("prefill", "r0", 20), ("prefill", "r1", 9), ("decode", 6), ("prefill", "r2", 33), ("decode", 5),
            ("end", "r1"), ("decode", 4), ("prefill", "r3", 12), ("prefill", "r4", 30), ("decode", 9),
            ("end", "r0"), ("decode", 8)]
    for op in plan:
        if op[0] == "prefill":
            _, r, n = op
            ents = [StepEntry(r, reqs[r][:n], [n - 1])]
            for e in (eager, graph):
                lg = e.step(ents)
            pos[r] = n
            live.append(r)
        elif op[0] == "end":
            live.remove(op[1])
            eager.release(op[1])
            graph.release(op[1])
        else:
            for _ in range(op[1]):
                ents = [StepEntry(r, [reqs[r][pos[r]]], [0]) for r in live]
                a = eager.step(ents).clone()
                b = graph.step(ents).clone()
                torch.cuda.synchronize()
                assert torch.equal(a, b)
                for i, r in enumerate(live):
                    assert np.max(np.abs(b[i].double().cpu().numpy() - ref[r][pos[r]])) <= TOL[dtype]
                    pos[r] += 1
    assert graph.graph_replays == 32 and eager.graph_replays == 0
    assert sorted(graph._graphs) == [(2, 256), (4, 256)]         # batches 2..4 pad to 2 and 4 rows


def test_graphs_captured_ahead_are_the_ones_the_steps_replay(model_dirs, plain_models):
    """``capture_graphs`` captures, before any request exists, what the first single-token steps
    would capture; the steps then only replay, with the results of eager launches."""
    from rustinfer_amd import LLM, SamplingParams
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models["A"]
    reqs = random_requests(cfg["vocab_size"], [40, 30, 35], seed=33)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    eng = make_engine(model_dirs["A"], "float32", 16, max_requests=8)
    assert eng.capture_graphs([3], 41) == 0                       # graphs are off
    eng.enable_graphs(True, (1, 2, 4, 8))
    assert eng.capture_graphs([3], 41) == 1 and eng.capture_graphs([3, 4], 30) == 0
    assert sorted(eng._graphs) == [(4, 256)]
    for r, t in reqs.items():
        eng.step([StepEntry(r, t[:20], [])])
    for p in range(20, 30):
        lg = eng.step([StepEntry(r, [t[p]], [0]) for r, t in reqs.items()])
        for i, r in enumerate(reqs):
            assert np.max(np.abs(lg[i].double().cpu().numpy() - ref[r][p])) <= TOL["float32"]
    assert eng.graph_replays == 10 and sorted(eng._graphs) == [(4, 256)]
    llm = LLM(model=model_dirs["A"], dtype="float32", max_batch_seqs=4, max_model_len=128, paged_block_size=16, num_blocks=64)
    assert llm.capture_graphs(9, 50) == 1 and sorted(llm.engine._graphs) == [(4, 128)]     # rows capped at max_batch_seqs
    out = llm.generate([reqs["r0"][:7]], SamplingParams(max_tokens=5))
    assert out[0].token_ids == plain_greedy(cfg, w, reqs["r0"][:7], 5)
    assert (1, 128) in llm.engine._graphs


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_captured_graphs_outlive_steps_with_much_control_data(plain_models, tmp_path, dtype):
    """Captured graphs read the step's control data (tokens, positions, tables) at fixed device
    addresses.  With the default context length (256 table entries a row) a graph for two rows is
    captured; then a step of two prompt portions of 3,100 tokens and a step of 64 rows pass, each
    with more control data than any step before; the two-row graph still computes the plain
    implementation's logits afterwards, and so does the 64-row graph on its second use."""
    from rustinfer_amd.config import LlamaConfig
    from rustinfer_amd.engine import StepEntry
    from rustinfer_amd.weights import write_random_model
    cfg = dict(TINY["A"][0], max_position_embeddings=4096)
    write_random_model(LlamaConfig.from_dict(cfg), 0, str(tmp_path))
    w = plain_llama.read_model(str(tmp_path))[1]
    lengths = [56, 40, 3104, 3104] + [2 + i % 3 for i in range(60)]
    reqs = random_requests(cfg["vocab_size"], lengths, seed=51)
    names = list(reqs)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    eager = make_engine(str(tmp_path), dtype, 16, num_pages=600, max_requests=64, max_model_len=4096,
                        max_batch_tokens=8192)
    graph = make_engine(str(tmp_path), dtype, 16, num_pages=600, max_requests=64, max_model_len=4096,
                        max_batch_tokens=8192)
    graph.enable_graphs(True, (1, 2, 4, 8, 64))
    pos = {r: 0 for r in reqs}
    tol = TOL[dtype]

    def run(entries, compare=True):
        """entries: [(request, tokens)]; the last token's logits of each are checked."""
        ents = [StepEntry(r, reqs[r][pos[r]:pos[r] + n], [n - 1]) for r, n in entries]
        a = eager.step(ents).clone()
        b = graph.step(ents).clone()
        torch.cuda.synchronize()
        for i, (r, n) in enumerate(entries):
            pos[r] += n
            want = ref[r][pos[r] - 1]
            assert np.max(np.abs(a[i].double().cpu().numpy() - want)) <= tol, ("eager", r, pos[r])
            assert np.max(np.abs(b[i].double().cpu().numpy() - want)) <= tol, ("graph", r, pos[r])

    run([("r0", 40), ("r1", 25)])
    for _ in range(3):
        run([("r0", 1), ("r1", 1)])                      # the two-row graph is captured and replayed
    assert sorted(graph._graphs) == [(2, 1024)] and graph.graph_replays == 3
    staging = graph._staging.dev.data_ptr()
    run([("r2", 3100), ("r3", 3100)])                    # 6,200 tokens in one step
    for _ in range(2):
        run([("r0", 1), ("r1", 1)])
    run([(r, 1) for r in names[4:]] + [("r0", 1), ("r1", 1), ("r2", 1), ("r3", 1)])   # 64 rows: a new graph
    run([("r1", 1), ("r0", 1)])                          # the two-row graph again
    run([(r, 1) for r in names[4:]] + [("r0", 1), ("r1", 1), ("r2", 1), ("r3", 1)])   # the 64-row graph again
    run([("r0", 1), ("r1", 1)])
    assert graph._staging.dev.data_ptr() == staging
    assert sorted(graph._graphs) == [(2, 1024), (64, 4096)] and graph.graph_replays == 3 + 2 + 2 + 2
    graph.cache.check()


@pytest.mark.parametrize("name", ["C", "D"])
def test_many_single_tokens_on_the_matrix_core_kernels(model_dirs, plain_models, name):
    """Seventy requests decode together, bfloat16, head sizes 64 and 128: so many (token, kv
    head) pairs that one block takes all the keys of a pair; eagerly and as a graph of 80 rows,
    10 of them padding; prompts of 1 to 70 tokens, so that some requests have one chunk of keys
    and others several."""
    from rustinfer_amd.engine import StepEntry
    cfg, w = plain_models[name]
    lengths = [1 + (13 * i) % 70 for i in range(70)]
    reqs = random_requests(cfg["vocab_size"], [n + 4 for n in lengths], seed=77)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    page = page_size(name)
    pages = sum((len(t) + page - 1) // page for t in reqs.values()) + 4
    engines = [make_engine(model_dirs[name], "bfloat16", page, num_pages=pages, max_requests=80, max_batch_tokens=4096)
               for _ in range(2)]
    engines[1].enable_graphs(True, (80,))
    for e in engines:
        lg = e.step([StepEntry(r, reqs[r][:n], [n - 1]) for r, n in zip(reqs, lengths)])
        for i, (r, n) in enumerate(zip(reqs, lengths)):
            assert np.max(np.abs(lg[i].double().cpu().numpy() - ref[r][n - 1])) <= TOL["bfloat16"]
    for k in range(4):
        ents = [StepEntry(r, [reqs[r][n + k]], [0]) for r, n in zip(reqs, lengths)]
        a = engines[0].step(ents).clone()
        b = engines[1].step(ents).clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b)
        for i, (r, n) in enumerate(zip(reqs, lengths)):
            assert np.max(np.abs(b[i].double().cpu().numpy() - ref[r][n + k])) <= TOL["bfloat16"], (k, r)
    assert engines[1].graph_replays == 4 and sorted(engines[1]._graphs) == [(80, 256)]


@pytest.mark.parametrize("name", ["C", "D"])
@pytest.mark.parametrize("rows", [1, 2, 4, 7, 16])
def test_few_tokens_leave_the_norms_to_the_products_around_them(model_dirs, plain_models, monkeypatch, name, rows):
    """Up to 16 tokens in a step, bfloat16: no norm between two sub-layers runs as a kernel of its
    own (the product before it adds to the residual stream and prepares the next product's rows,
    the product after it applies the factor); only the first norm of a step does.  The logits stay
    those of the plain implementation and close to those of the engine with norm kernels."""
    from rustinfer_amd.engine import StepEntry
    from rustinfer_amd.kernels import ops
    cfg, w = plain_models[name]
    reqs = random_requests(cfg["vocab_size"], [20 + 7 * i for i in range(rows)], seed=78)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    calls = {"norm": 0, "residual": 0}
    attended = {"n": 0}
    real_norm, real_res, real_attn = ops.add_rmsnorm, ops.linear_residual, ops.paged_attention

    def count_attention(*a, **k):
        attended["n"] += 1
        return real_attn(*a, **k)
    monkeypatch.setattr(ops, "paged_attention", count_attention)

    def count(key, real):
        def f(*a, **k):
            calls[key] += 1
            return real(*a, **k)
        return f
    monkeypatch.setattr(ops, "add_rmsnorm", count("norm", real_norm))
    monkeypatch.setattr(ops, "linear_residual", count("residual", real_res))
    page = page_size(name)
    L = cfg["num_hidden_layers"]
    deferred = make_engine(model_dirs[name], "bfloat16", page, num_pages=128, max_requests=16, max_batch_tokens=2048)
    apart = make_engine(model_dirs[name], "bfloat16", page, num_pages=128, max_requests=16, max_batch_tokens=2048)
    heads = [StepEntry(r, t[:-6], []) for r, t in reqs.items()]
    deferred.step(heads)
    # no logits wanted: the last block only fills its cache (its norm and projection; no attention, no feed-forward)
    assert attended["n"] == L - 1
    if sum(len(e.tokens) for e in heads) > 16:
        assert calls == {"norm": 2 * L - 1, "residual": 0}            # long portions keep the norms' own kernels
    else:
        assert calls == {"norm": 1, "residual": 2 * L - 2}
    apart.step(heads)
    for k in range(6):
        ents = [StepEntry(r, [t[len(t) - 6 + k]], [0]) for r, t in reqs.items()]
        calls.update(norm=0, residual=0)
        a = deferred.step(ents).clone()
        assert calls == {"norm": 1, "residual": 2 * L}                 # the step's first norm only
        monkeypatch.setattr(ops, "DEFERRED_NORM_MAX_ROWS", 0)
        calls.update(norm=0, residual=0)
        b = apart.step(ents).clone()
        monkeypatch.setattr(ops, "DEFERRED_NORM_MAX_ROWS", 16)
        assert calls == {"norm": 2 * L + 1, "residual": 0}
        for i, (r, t) in enumerate(reqs.items()):
            want = ref[r][len(t) - 6 + k]
            assert np.max(np.abs(a[i].double().cpu().numpy() - want)) <= TOL["bfloat16"], (k, r)
            assert np.max(np.abs(b[i].double().cpu().numpy() - want)) <= TOL["bfloat16"], (k, r)
    # a step of two short portions (2 and 3 tokens) beside single tokens takes the same path; logits wanted out of order do not
    if rows >= 4:
        names = list(reqs)
        for r in names:
            deferred.release(r)
        deferred.step([StepEntry(r, reqs[r][:9], []) for r in names[:3]])
        calls.update(norm=0, residual=0)
        lg = deferred.step([StepEntry(names[0], reqs[names[0]][9:11], [0, 1]), StepEntry(names[1], reqs[names[1]][9:12], [0, 1, 2]),
                            StepEntry(names[2], reqs[names[2]][9:10], [0])]).double().cpu().numpy()
        assert calls == {"norm": 1, "residual": 2 * L}
        want = np.concatenate([ref[names[0]][9:11], ref[names[1]][9:12], ref[names[2]][9:10]])
        assert np.max(np.abs(lg - want)) <= TOL["bfloat16"]
        calls.update(norm=0, residual=0)
        lg = deferred.step([StepEntry(names[0], reqs[names[0]][11:13], [1, 0])]).double().cpu().numpy()
        assert calls == {"norm": 2, "residual": 2 * L - 1}             # the final norm gathers its rows itself
        assert np.max(np.abs(lg - ref[names[0]][[12, 11]])) <= TOL["bfloat16"]


def test_graph_bucket_choice():
    from rustinfer_amd.engine import pick_graph_bucket
    # the reference's cases (crates/infer-worker/src/application/runtime/graph_exec.rs:476-501)
    sizes = [4, 1, 2, 2]
    assert [pick_graph_bucket(sizes, b, True) for b in (1, 2, 3, 4, 5)] == [1, 2, 4, 4, 0]
    assert pick_graph_bucket(sizes, 2, False) == 0


def test_random_weights_seed_and_environment_switches(model_dirs, tmp_path, monkeypatch, capfd):
    """A folder with config.json only runs with weights drawn from `random_weights_seed`;
    RUSTINFER_DISABLE_GRAPH and RUSTINFER_STEP_TRACE are honoured."""
    import shutil
    from rustinfer_amd import LLM, SamplingParams
    shutil.copy(f"{model_dirs['A']}/config.json", tmp_path / "config.json")
    monkeypatch.setenv("RUSTINFER_DISABLE_GRAPH", "1")
    monkeypatch.setenv("RUSTINFER_STEP_TRACE", "1")
    monkeypatch.setenv("RUSTINFER_STEP_TRACE_MS", "0")
    outs = []
    for _ in range(2):
        llm = LLM(model=str(tmp_path), dtype="float32", num_blocks=16, max_model_len=128, random_weights_seed=5)
        outs.append(llm.generate([[1, 2, 3]], SamplingParams(max_tokens=5, ignore_eos=True))[0].token_ids)
        assert llm.engine.graph_replays == 0
    assert outs[0] == outs[1] and len(outs[0]) == 5
    assert "[step-trace]" in capfd.readouterr().err
    monkeypatch.delenv("RUSTINFER_DISABLE_GRAPH")
    llm = LLM(model=str(tmp_path), dtype="float32", num_blocks=16, max_model_len=128, random_weights_seed=5)
    assert llm.generate([[1, 2, 3]], SamplingParams(max_tokens=5, ignore_eos=True))[0].token_ids == outs[0]
    assert llm.engine.graph_replays > 0


def test_force_gemm_and_first_token_trace_switches(model_dirs, plain_models, monkeypatch, capfd):
    """RUSTINFER_FORCE_GEMM sends every bfloat16 product through the GEMM library (no few-row kernel
    runs, fused or not) and the logits stay the plain implementation's; RUSTINFER_TTFT_TRACE times
    the forward pass and the sampling of each step."""
    from rustinfer_amd import LLM, SamplingParams
    from rustinfer_amd.engine import StepEntry
    from rustinfer_amd.kernels import ops
    cfg, w = plain_models["C"]
    toks = np.random.default_rng(3).integers(0, cfg["vocab_size"], 12).tolist()
    ref = plain_llama.forward(cfg, w, toks)
    monkeypatch.setenv("RUSTINFER_FORCE_GEMM", "1")
    monkeypatch.setenv("RUSTINFER_TTFT_TRACE", "1")
    monkeypatch.setattr(ops, "FORCE_LIBRARY_GEMM", False)            # the switch sets it; put back afterwards
    lib, few_row = ops._lib(), []
    for name in ("ri_gemm_skinny_bf16", "ri_gemm_qkv_rope", "ri_gemm_skinny_residual", "ri_gemm_rows_bf16", "ri_gemm_rows_qkv_rope"):
        entry = getattr(lib, name)
        monkeypatch.setattr(lib, name, lambda *a, entry=entry, name=name: few_row.append(name) or entry(*a))
    llm = LLM(model=model_dirs["C"], dtype="bfloat16", paged_block_size=page_size("C"), num_blocks=32, max_model_len=64)
    assert ops.FORCE_LIBRARY_GEMM
    lg = llm.engine.step([StepEntry("a", toks[:9], [8])]).double().cpu().numpy()
    assert np.max(np.abs(lg[0] - ref[8])) <= TOL["bfloat16"]
    for i in range(9, 12):                                           # single tokens as well
        lg = llm.engine.step([StepEntry("a", toks[i:i + 1], [0])]).double().cpu().numpy()
        assert np.max(np.abs(lg[0] - ref[i])) <= TOL["bfloat16"]
    llm.engine.release("a")
    assert few_row == []
    out = llm.generate([toks[:5]], SamplingParams(max_tokens=3, ignore_eos=True))[0].token_ids
    assert len(out) == 3 and few_row == []
    err = capfd.readouterr().err
    assert "[ttft-trace] forward (5 tokens in 1 rows, synced)" in err and "[ttft-trace] sample (1 rows, synced)" in err


def test_a_launch_that_misses_the_fast_attention_kernels_says_so(model_dirs, capfd):
    """Pages of 8 tokens (model B's test size; the reference's own launch files say 1) run the plain
    attention kernels in bfloat16: one line says so and why; pages of 16 say nothing."""
    from rustinfer_amd import LLM
    LLM(model=model_dirs["B"], dtype="bfloat16", paged_block_size=8, num_blocks=32, max_model_len=64)
    err = capfd.readouterr().err
    assert "attention runs on the plain kernels" in err and "pages of 8 tokens" in err
    LLM(model=model_dirs["C"], dtype="bfloat16", paged_block_size=16, num_blocks=32, max_model_len=64)
    assert "plain kernels" not in capfd.readouterr().err
