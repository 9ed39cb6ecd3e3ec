"""Schedules that the other engine tests do not reach: decoding under graphs across a multiple
of 1,024 keys (another captured graph, other split counts), bfloat16 generation through the
scheduler, graphs and sampler on the matrix-core kernels, and replay traces with block tables
and with a request that is given up mid-way and run again from its first token."""
import json
import os

import numpy as np
import pytest
import torch

import plain_llama
from helpers import (TINY_MFMA, TOL, check_steps_against, cut_mixed, cut_preempted, expected_tables,
                     page_size, random_requests, run_trace, scaled_tol)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """Configuration C with room for 4,096 positions: (folder, config, plain weights)."""
    from rustinfer_amd.config import LlamaConfig
    from rustinfer_amd.weights import write_random_model
    d = str(tmp_path_factory.mktemp("tiny_C_long"))
    cfg = dict(TINY_MFMA["C"][0], max_position_embeddings=4096)
    write_random_model(LlamaConfig.from_dict(cfg), 2, d)
    return d, cfg, plain_llama.read_model(d)[1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [1, 4])
def test_decoding_under_graphs_across_a_key_bucket(long_model, dtype, rows):
    """Graphs are kept per (rows, keys rounded up to 1,024).  The longest request decodes from
    position 1,020 to 1,027 and from 2,044 to 2,051: between two tokens the step changes to
    another captured graph (other numbers of key chunks).  Every step is compared with an engine
    that launches eagerly and with the plain implementation; with four rows the other requests are
    shorter, one of them crossing 1,024 keys itself a few steps later."""
    from rustinfer_amd.engine import StepEntry, build_engine
    d, cfg, w = long_model
    # (tokens before the first decode phase, tokens between the phases); 8 single tokens a phase
    shapes = [(1020, 1016), (300, 0), (1018, 0), (17, 40)][:rows]
    reqs = random_requests(cfg["vocab_size"], [a + 8 + b + 8 for a, b in shapes], seed=61)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    tol = scaled_tol(dtype, ref)
    engines = [build_engine(d, dtype=dtype, page_size=16, num_pages=320, max_requests=4, max_model_len=4096,
                            max_batch_tokens=4096) for _ in range(2)]
    eager, graph = engines
    graph.enable_graphs(True, (1, 2, 4))
    pos = {r: 0 for r in reqs}

    def portion(r, n):
        ents = [StepEntry(r, reqs[r][pos[r]:pos[r] + n], [n - 1])]
        for e in engines:
            lg = e.step(ents)
            assert np.max(np.abs(lg[0].double().cpu().numpy() - ref[r][pos[r] + n - 1])) <= tol, (r, pos[r], n)
        pos[r] += n

    def decode(steps):
        for _ in range(steps):
            ents = [StepEntry(r, [reqs[r][pos[r]]], [0]) for r in reqs]
            a = eager.step(ents).clone()
            b = graph.step(ents).clone()
            torch.cuda.synchronize()
            assert torch.equal(a, b), {r: pos[r] for r in reqs}
            for i, r in enumerate(reqs):
                assert np.max(np.abs(b[i].double().cpu().numpy() - ref[r][pos[r]])) <= tol, (r, pos[r])
                pos[r] += 1

    for r, (a, _) in zip(reqs, shapes):
        portion(r, a)
    decode(8)
    bucket = 1 if rows == 1 else 4
    assert sorted(graph._graphs) == [(bucket, 1024), (bucket, 2048)]
    for r, (_, b) in zip(reqs, shapes):
        if b:
            portion(r, b)
    decode(8)
    assert sorted(graph._graphs) == [(bucket, 1024), (bucket, 2048), (bucket, 3072)]
    assert graph.graph_replays == 16 and eager.graph_replays == 0
    assert all(pos[r] == len(t) for r, t in reqs.items())
    graph.cache.check()


def test_portions_behind_many_cached_keys(long_model):
    """A short portion behind hundreds of cached keys has the keys divided between blocks of the
    attention kernel; a captured step says in its key whether it does.  Eager and captured steps
    against the plain logits, portions of 48, 2 and 130 tokens behind 600 and more keys, beside
    a single token of another request."""
    from rustinfer_amd.engine import StepEntry, build_engine
    d, cfg, w = long_model
    reqs = random_requests(cfg["vocab_size"], [800, 60], seed=67)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    tol = scaled_tol("bfloat16", ref)
    engines = [build_engine(d, dtype="bfloat16", page_size=16, num_pages=80, max_requests=4, max_model_len=4096,
                            max_batch_tokens=1024) for _ in range(2)]
    eager, graph = engines
    graph.enable_graphs(True, (1, 2, 4), mixed_tokens=256)
    r0, r1 = list(reqs)
    pos = {r: 0 for r in reqs}
    for step in ([(r0, 600)], [(r1, 30)], [(r0, 48), (r1, 1)], [(r1, 1), (r0, 2)], [(r0, 130), (r1, 1)], [(r0, 20)]):
        ents = [StepEntry(r, reqs[r][pos[r]:pos[r] + n], [n - 1]) for r, n in step]
        a = eager.step(ents).clone()
        b = graph.step(ents).clone()
        torch.cuda.synchronize()
        for i, (r, n) in enumerate(step):
            for lg in (a, b):
                diff = np.max(np.abs(lg[i].double().cpu().numpy() - ref[r][pos[r] + n - 1]))
                assert diff <= tol, (step, r, diff)
            pos[r] += n
    mixed = sorted(k[1:] for k in graph._graphs if k[0] == "mixed")
    # (tokens, rows, keys, rows of one token, keys divided): the first portions are not, those behind 600 keys are
    assert mixed == [(16, 2, 1024, 1, 1), (32, 1, 1024, 0, 0), (32, 1, 1024, 0, 1), (64, 2, 1024, 1, 1),
                     (144, 2, 1024, 1, 1)], mixed
    graph.cache.check()


@pytest.mark.parametrize("name", ["C", "D"])
def test_generate_bfloat16_on_the_matrix_core_kernels(model_dirs, plain_models, name):
    """bfloat16 generation through the scheduler, graphs, device-resident tokens and the sampler at
    head sizes 64 and 128 (MFMA attention, the fused projection, tile-ordered weights): prompts cut
    into portions of 7 beside decoding requests; every generated token is one the plain
    implementation ranks at the top too, up to the bfloat16 tolerance on logits."""
    from rustinfer_amd import LLM, SamplingParams
    cfg, w = plain_models[name]
    prompts = list(random_requests(cfg["vocab_size"] - 1, [5, 33, 64, 90, 18], seed=26).values())
    llm = LLM(model=model_dirs[name], dtype="bfloat16", paged_block_size=page_size(name), num_blocks=64,
              max_model_len=cfg["max_position_embeddings"], max_batch_seqs=4, max_batch_tokens=24,
              chunked_prefill_size=7, capture_sizes=(1, 2, 4))
    res = llm.generate(prompts, SamplingParams(max_tokens=14, ignore_eos=True))
    assert llm.engine.graph_replays > 0
    worst = 0.0
    for p, r in zip(prompts, res):
        assert len(r.token_ids) == 14 and r.finish_reason == "length"
        toks = list(p)
        for t in r.token_ids:
            logits = plain_llama.forward(cfg, w, toks)[-1]
            worst = max(worst, float(logits.max() - logits[t]))
            assert logits.max() - logits[t] <= 2 * scaled_tol("bfloat16", {"x": logits}), (len(p), len(toks))
            toks.append(t)
    print(f"{name}: largest gap of a chosen token to the plain top logit {worst:.3e}")
    llm.engine.cache.check()
    assert llm.engine.cache.free_pages() == 64


def _read_tables(out_dir, steps):
    got = {}
    for st in steps:
        with open(os.path.join(out_dir, f"{st['step']}.tables.json")) as f:
            got[st["step"]] = json.load(f)
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_writes_the_block_tables_it_used(model_dirs, plain_models, tmp_path, dtype):
    """Beside the logits, every step leaves the block table of each of its entries.  The allocator
    hands out the smallest free page first, so the tables of a trace are fixed: they are compared
    with a simulation of that rule (pages taken when a request's tokens first need them, given back
    when it ends), and the pool is so small that pages go round."""
    cfg, w = plain_models["A"]
    reqs = random_requests(cfg["vocab_size"], [1, 7, 33, 64, 100, 128, 2, 49], seed=11)
    plain = {rid: plain_llama.forward(cfg, w, t) for rid, t in reqs.items()}
    steps = cut_mixed(reqs, 384, seed=5)
    results = run_trace(model_dirs["A"], dtype, steps, str(tmp_path), 384, page=16)
    check_steps_against(steps, results, plain, TOL[dtype], f"A/{dtype}/mixed+tables")
    got = _read_tables(str(tmp_path), steps)
    want = expected_tables(steps, page=16, num_pages=384 // 16)
    reused = set()
    seen = {}
    for st in steps:
        rec = got[st["step"]]
        assert [e["id"] for e in rec["entries"]] == [e["id"] for e in st["entries"]]
        for e, exp in zip(rec["entries"], want[st["step"]]):
            assert e["start"] == exp["start"] and e["tables"] == [exp["table"]], (st["step"], e, exp)
            for p in exp["table"]:
                if seen.setdefault(p, e["id"]) != e["id"]:
                    reused.add(p)
    assert len(reused) >= 4                       # pages did go from one request to another


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_replay_of_requests_given_up_and_run_again(model_dirs, plain_models, tmp_path, name, dtype):
    """The mixed trace with preemptions: now and then the request that has come furthest is ended
    mid-way, the others go on and take its pages, and it starts again from its first token beside
    them (recompute-resume, crates/infer-scheduler/src/domain/inference_session/table.rs:767-815).
    Every position's logits, the first run's and the second's, are the plain implementation's."""
    cfg, w = plain_models[name]
    lengths = {"B": [40, 100, 129, 65, 17, 200], "C": [130, 257, 64, 400, 33, 18]}[name]
    reqs = random_requests(cfg["vocab_size"], lengths, seed=12)
    plain = {rid: plain_llama.forward(cfg, w, t) for rid, t in reqs.items()}
    max_tokens = {"B": 448, "C": 896}[name]
    steps, given_up = cut_preempted(reqs, max_tokens, seed=9)
    assert given_up >= 2 and max(len(s["entries"]) for s in steps) >= 3
    page = page_size(name)
    results = run_trace(model_dirs[name], dtype, steps, str(tmp_path), max_tokens, page=page)
    worst = check_steps_against(steps, results, plain, scaled_tol(dtype, plain), f"{name}/{dtype}/preempted")
    got = _read_tables(str(tmp_path), steps)
    want = expected_tables(steps, page=page, num_pages=max_tokens // page)
    for st in steps:
        for e, exp in zip(got[st["step"]]["entries"], want[st["step"]]):
            assert e["start"] == exp["start"] and e["tables"] == [exp["table"]], (st["step"], e, exp)
    print(f"{name} {dtype} preempted: {len(steps)} steps, {given_up} requests given up, worst |diff| {worst:.3e}")


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_steps_with_portions_replay_graphs(model_dirs, plain_models, name, dtype):
    """Steps that hold prompt portions are captured per (token bucket, row bucket, key bucket) and
    replayed.  Shapes come again with other rows and lengths, with eager steps and other graphs
    between the replays; every replay is compared with an engine that launches eagerly and with
    the plain implementation.  A step
    that wants logits inside a portion, or more tokens than the limit, launches eagerly."""
    from rustinfer_amd.engine import StepEntry, build_engine
    cfg, w = plain_models[name]
    lengths = [150, 90, 40, 33, 260, 21, 300]
    reqs = random_requests(cfg["vocab_size"], lengths, seed=71)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    tol = scaled_tol(dtype, ref)
    page = page_size(name)
    engines = [build_engine(model_dirs[name], dtype=dtype, page_size=page, num_pages=1024 // page + 8, max_requests=8,
                            max_model_len=512, max_batch_tokens=512) for _ in range(2)]
    eager, graph = engines
    graph.enable_graphs(True, (1, 2, 4, 8), mixed_tokens=256)
    pos = {r: 0 for r in reqs}

    def run(step, want_inner=False):
        ents = []
        for r, n in step:
            want = list(range(n)) if want_inner else ([n - 1] if (pos[r] + n) % 3 else [])
            ents.append(StepEntry(r, reqs[r][pos[r]:pos[r] + n], want))
        a = eager.step(ents).clone()
        b = graph.step(ents).clone()
        torch.cuda.synchronize()
        # the padded step may take other forms of a kernel than the eager one (products of 128 rows
        # for 103, attention tiled for more tokens): the same logits to rounding, not to the bit
        assert a.shape == b.shape and (a.shape[0] == 0 or float((a - b).abs().max()) <= tol), step
        row = 0
        for e, (r, n) in zip(ents, step):
            for wpl in e.want:
                diff = np.max(np.abs(b[row].double().cpu().numpy() - ref[r][pos[r] + wpl]))
                assert diff <= tol, (step, r, pos[r] + wpl, diff)
                row += 1
            pos[r] += n

    run([("r0", 100), ("r1", 3)])                              # 103 tokens -> 112, two rows -> 2
    run([("r0", 1), ("r1", 1)])                                # single tokens: the other kind of graph
    run([("r1", 70), ("r0", 1), ("r2", 30), ("r3", 2)])        # 103 tokens -> 112, four rows -> 4
    run([("r0", 5), ("r1", 1), ("r2", 1), ("r3", 7)])          # 14 -> 16 tokens
    run([("r3", 9), ("r0", 1), ("r2", 1), ("r1", 3)])          # 14 -> 16 tokens, two single tokens: the same graph
    run([("r4", 120)])                                         # -> 128 tokens, one row
    run([("r0", 1), ("r1", 1), ("r2", 1), ("r3", 1), ("r4", 1)])
    run([("r4", 100), ("r3", 1), ("r2", 3)])                   # 104 -> 112, 3 rows -> 4: the graph of the third step again
    run([("r5", 17), ("r0", 1)], want_inner=True)              # logits inside a portion: eagerly
    replays = graph.mixed_graph_replays
    assert replays == 6
    run([("r4", 39), ("r0", 20), ("r1", 6), ("r2", 2), ("r3", 1), ("r5", 2)])   # 70 -> 80 tokens, 6 rows -> 8
    eager.release("r3"), graph.release("r3")
    reqs["r3b"], ref["r3b"], pos["r3b"] = reqs["r3"], ref["r3"], 0              # a new request on pages used before
    run([("r3b", 33), ("r0", 10), ("r5", 1)])                  # 44 -> 48 tokens
    mixed = sorted(k[1:] for k in graph._graphs if k[0] == "mixed")
    # (tokens, rows, keys, rows of one token, whether a portion lies behind so many keys that they are divided)
    assert mixed == [(16, 4, 512, 2, 0), (48, 4, 512, 1, 0), (80, 8, 512, 1, 0), (112, 2, 512, 0, 0),
                     (112, 4, 512, 1, 0), (128, 1, 512, 0, 0)], mixed
    assert graph.mixed_graph_replays == 8 and eager.graph_replays == 0
    run([("r6", 300)])                                         # more tokens than the limit: eagerly
    assert graph.mixed_graph_replays == 8
    graph.cache.check()


def test_a_step_shape_with_portions_is_captured_when_it_is_met_again(model_dirs, plain_models):
    """``mixed_after = 3``: the first two steps of a shape launch eagerly, the third is captured and
    replayed; a shape met once costs no capture.  All give the plain logits."""
    from rustinfer_amd.engine import StepEntry
    from test_gpu_engine import make_engine
    cfg, w = plain_models["C"]
    eng = make_engine(model_dirs["C"], "bfloat16", page_size("C"), num_pages=64, max_requests=4, max_batch_tokens=256)
    eng.enable_graphs(True, (1, 2, 4), mixed_tokens=128, mixed_after=3)
    reqs = random_requests(cfg["vocab_size"], [90, 60], seed=71)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    r0, r1 = list(reqs)
    pos = {r: 0 for r in reqs}
    seen = []
    for step in ([(r0, 10), (r1, 3)], [(r0, 9), (r1, 5)], [(r0, 12), (r1, 2)], [(r0, 11), (r1, 4)], [(r0, 40)]):
        ents = [StepEntry(r, reqs[r][pos[r]:pos[r] + n], [n - 1]) for r, n in step]
        lg = eng.step(ents).double().cpu().numpy()
        for i, (r, n) in enumerate(step):
            assert np.max(np.abs(lg[i] - ref[r][pos[r] + n - 1])) <= TOL["bfloat16"], (step, r)
            pos[r] += n
        seen.append((eng.mixed_graph_replays, sum(1 for k in eng._graphs if k[0] == "mixed")))
    # four steps of 13-15 tokens in two rows (one shape: 16 tokens), then one of another shape
    assert seen == [(0, 0), (0, 0), (1, 1), (2, 1), (2, 1)], seen


def test_graphs_of_steps_with_portions_make_room_for_new_shapes(model_dirs, plain_models, monkeypatch):
    """With the budget of such graphs spent, a new shape takes the place of the one that has not run
    for the longest time; the steps go on giving the plain logits."""
    from rustinfer_amd.engine import StepEntry
    from rustinfer_amd.engine.step import Engine
    from test_gpu_engine import make_engine
    monkeypatch.setattr(Engine, "MIXED_GRAPH_BUDGET", 2)
    cfg, w = plain_models["C"]
    eng = make_engine(model_dirs["C"], "bfloat16", page_size("C"), num_pages=64, max_requests=4, max_batch_tokens=256)
    eng.enable_graphs(True, (1, 2, 4), mixed_tokens=128)
    reqs = random_requests(cfg["vocab_size"], [200], seed=73)
    r0 = list(reqs)[0]
    ref = plain_llama.forward(cfg, w, reqs[r0])
    pos = 0
    held = []
    for n in (10, 20, 12, 40, 25, 14):                   # token buckets 16, 32, 16, 48, 32, 16
        lg = eng.step([StepEntry(r0, reqs[r0][pos:pos + n], [n - 1])]).double().cpu().numpy()
        assert np.max(np.abs(lg[0] - ref[pos + n - 1])) <= TOL["bfloat16"], (pos, n)
        pos += n
        held.append(sorted(k[1] for k in eng._graphs if k[0] == "mixed"))
    # 48 takes the place of 32 (16 ran after it), 32 comes back in the place of 16, and 16 in that of 48
    assert held == [[16], [16, 32], [16, 32], [16, 48], [32, 48], [16, 32]], held
    eng.cache.check()


def test_pool_sized_from_free_memory_after_a_worst_case_step(model_dirs, plain_models):
    """``num_pages = 0``: a bootstrap pool, the largest step once (workspace and library buffers
    exist afterwards), then the real pool in its place: as many pages as the requests can use at
    most, here.  The engine then computes the plain logits, and prewarming captures every size."""
    from rustinfer_amd.engine import StepEntry, build_engine
    cfg, w = plain_models["C"]
    eng = build_engine(model_dirs["C"], dtype="bfloat16", page_size=16, num_pages=0, max_requests=3,
                       max_model_len=256, max_batch_tokens=300)
    assert eng.cache.groups[0].num_pages == 3 * 16 and eng.cache.free_pages() == 48
    assert eng.workspace.nbytes() > 300 * cfg["hidden_size"] * 4 and not eng.cache.live_requests()
    reqs = random_requests(cfg["vocab_size"], [200, 77], seed=91)
    ref = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    lg = eng.step([StepEntry(r, t, [len(t) - 1]) for r, t in reqs.items()]).double().cpu().numpy()
    for i, (r, t) in enumerate(reqs.items()):
        assert np.max(np.abs(lg[i] - ref[r][-1])) <= scaled_tol("bfloat16", ref)
    for r in reqs:
        eng.release(r)
    eng.enable_graphs(True, (1, 2, 3))
    assert eng.prewarm_graphs() == 3 and sorted(eng._graphs) == [(1, 256), (2, 256), (3, 256)]
