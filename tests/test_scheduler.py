"""The scheduler's decisions (no GPU): admission, portions under a token budget, decoding,
finishing, and what happens when pages run out.  The cache manager keeps books only."""
import pytest

from rustinfer_amd.cache import CacheManager
from rustinfer_amd.engine.scheduler import Request, Scheduler
from rustinfer_amd.parts import PagedKVNeed
from rustinfer_amd.sampling import SamplingParams


def make(num_pages=64, page=4, **kw):
    cache = CacheManager({0: PagedKVNeed(1, 16)}, page, num_pages, kw.get("max_batch_seqs", 4),
                         kw.get("max_model_len", 4096), device=None)
    return Scheduler(cache, **kw), cache


def req(rid, n, max_tokens=8, **kw):
    return Request(rid, list(range(1, n + 1)), SamplingParams(max_tokens=max_tokens, **kw), eos_ids=(0,))


def run_step(s, cache, token=7):
    """What the engine does with a scheduled step, on the books only."""
    st = s.schedule()
    for e in st.entries:
        rid = e.request.request_id
        if not cache.has_request(rid):
            cache.add_request(rid)
        assert cache.append(rid, e.count) == e.start
    produced = s.commit(st, {e.request.request_id: (token(e.request) if callable(token) else token)
                             for e in st.entries if e.final})
    cache.check()
    return st, produced


def portions(st):
    return [(e.request.request_id, e.start, e.count, e.final) for e in st.entries]


# The reference's expectations (crates/infer-scheduler/src/domain/policy/continuous_batching.rs:306-440)
def test_empty_queue_gives_an_empty_step():
    s, _ = make()
    assert s.schedule().entries == [] and not s.has_work()


def test_requests_fill_the_token_budget_and_the_last_is_partial():
    s, c = make(max_batch_tokens=25)
    for r in "abc":
        s.add(req(r, 10))
    st = s.schedule()
    assert portions(st) == [("a", 0, 10, True), ("b", 0, 10, True), ("c", 0, 5, False)]
    assert st.num_tokens == 25


def test_sequence_budget():
    s, c = make(max_batch_seqs=2)
    for r in "abc":
        s.add(req(r, 5))
    assert [e.request.request_id for e in s.schedule().entries] == ["a", "b"]


def test_chunked_prefill_splits_a_long_prompt():
    s, c = make(chunked_prefill_size=10)
    s.add(req("long", 25))
    assert portions(s.schedule()) == [("long", 0, 10, False)]


def test_continuation_comes_before_new_work():
    s, c = make(chunked_prefill_size=10, max_batch_tokens=12)
    s.add(req("cont", 25))
    run_step(s, c)                                   # cont has 10 of 25 cached
    s.add(req("new", 5))
    st = s.schedule()
    assert portions(st) == [("cont", 10, 10, False), ("new", 0, 2, False)]


def test_without_chunking_the_prompt_goes_whole_or_as_the_budget_allows():
    s, c = make()
    s.add(req("full", 100))
    assert portions(s.schedule()) == [("full", 0, 100, True)]
    s, c = make(max_batch_tokens=32)
    s.add(req("large", 100))
    assert portions(s.schedule()) == [("large", 0, 32, False)]


def test_shortest_first_and_cap_on_new_requests():
    s, c = make(prefill_sjf=True, max_prefill_seqs_per_iter=2, max_batch_seqs=8)
    for r, n in (("a", 30), ("b", 5), ("c", 12)):
        s.add(req(r, n))
    assert [e.request.request_id for e in s.schedule().entries] == ["b", "c"]


def test_a_step_a_few_tokens_over_a_multiple_of_the_alignment_gives_them_up():
    """Portions of 256 beside 8 decoding requests make steps of 264 tokens, which cost the matrix
    products a tile of rows more than 256 do: the portion gives 8 tokens up, unless it is the last
    of its prompt."""
    s, c = make(num_pages=1024, page=16, max_batch_seqs=16, chunked_prefill_size=256, token_align=256)
    for i in range(8):
        s.add(req(i, 3, max_tokens=100))
    run_step(s, c)                                      # eight short prompts; they decode from here on
    s.add(req("long", 700, max_tokens=4))
    st, _ = run_step(s, c)
    assert st.num_tokens == 256 and portions(st)[-1] == ("long", 0, 248, False)
    st, _ = run_step(s, c)
    assert st.num_tokens == 256 and portions(st)[-1] == ("long", 248, 248, False)
    st, _ = run_step(s, c)                              # the rest is the prompt's last portion: whole
    assert portions(st)[-1] == ("long", 496, 204, True)
    # a last portion is never cut, and a step far over the multiple is left alone
    s.add(req("exact", 256, max_tokens=4))
    st, _ = run_step(s, c)
    assert ("exact", 0, 256, True) in portions(st) and st.num_tokens == 265
    s2, c2 = make(num_pages=1024, page=16, max_batch_seqs=64, chunked_prefill_size=256, token_align=256)
    for i in range(40):
        s2.add(req(i, 2, max_tokens=100))
    run_step(s2, c2)
    s2.add(req("long", 700, max_tokens=4))
    assert run_step(s2, c2)[0].num_tokens == 296
    # off
    s3, c3 = make(num_pages=1024, page=16, max_batch_seqs=16, chunked_prefill_size=256)
    for i in range(8):
        s3.add(req(i, 3, max_tokens=100))
    run_step(s3, c3)
    s3.add(req("long", 700, max_tokens=4))
    assert run_step(s3, c3)[0].num_tokens == 264
    # every token of the prompt runs once, whatever was given up on the way, and in no more portions
    # than without: 1000 tokens in portions of up to 64 are 16 portions with 24 tokens to spare,
    # so four portions can give five tokens up each
    s4, c4 = make(num_pages=1024, page=16, max_batch_seqs=16, chunked_prefill_size=64, token_align=64)
    for i in range(5):
        s4.add(req(i, 3, max_tokens=400))
    run_step(s4, c4)
    long = s4.add(req("long", 1000, max_tokens=2))
    seen = []
    while long.state != "finished" and len(seen) < 100:
        st, _ = run_step(s4, c4)
        seen += [(e.start, e.count) for e in st.entries if e.request is long and not e.is_decode]
    assert sum(n for _, n in seen) == 1000 and all(a + n == b for (a, n), (b, _) in zip(seen, seen[1:]))
    assert [n for _, n in seen] == [59] * 4 + [64] * 11 + [60]
    # a prompt that is a whole number of portions gives nothing up: it would need one portion more
    s5, c5 = make(num_pages=1024, page=16, max_batch_seqs=16, chunked_prefill_size=256, token_align=256)
    for i in range(8):
        s5.add(req(i, 3, max_tokens=100))
    run_step(s5, c5)
    s5.add(req("even", 512, max_tokens=4))
    assert portions(run_step(s5, c5)[0])[-1] == ("even", 0, 256, False)
    assert portions(run_step(s5, c5)[0])[-1] == ("even", 256, 256, True)


def test_decoding_requests_run_every_step_before_prompts():
    s, c = make(max_batch_tokens=16, chunked_prefill_size=8)
    s.add(req("a", 3))
    s.add(req("b", 4))
    st, out = run_step(s, c)
    assert [(r.request_id, t) for r, t in out] == [("a", 7), ("b", 7)]      # first tokens from the prompts' last logits
    s.add(req("p", 40))
    st, out = run_step(s, c)
    assert portions(st) == [("a", 3, 1, True), ("b", 4, 1, True), ("p", 0, 8, False)]
    st, out = run_step(s, c)
    assert portions(st)[:2] == [("a", 4, 1, True), ("b", 5, 1, True)] and portions(st)[2] == ("p", 8, 8, False)
    assert s.stats["decode_tokens"] == 4 and s.stats["prefill_tokens"] == 3 + 4 + 16


def test_finishing_rules():
    # finished = eos (unless ignored) or generated >= max_tokens; the ending token is emitted
    # (crates/infer-worker/src/application/runtime/mod.rs:1198-1214, cases :1488-1505)
    s, c = make()
    a, b, d = s.add(req("a", 3, max_tokens=3)), s.add(req("b", 3, max_tokens=5, ignore_eos=True)), s.add(req("d", 2, max_tokens=1))
    toks = iter([5, 0, 9,  0, 0,  6, 1,  2])
    seq = {"a": [5, 0], "b": [0, 0, 6, 1, 2], "d": [9]}
    pos = {k: 0 for k in seq}

    def token(r):
        t = seq[r.request_id][pos[r.request_id]]
        pos[r.request_id] += 1
        return t
    while s.has_work():
        run_step(s, c, token)
    assert (a.output, a.finish_reason) == ([5, 0], "eos")
    assert (b.output, b.finish_reason) == ([0, 0, 6, 1, 2], "length")
    assert (d.output, d.finish_reason) == ([9], "length")                  # finished on its first token
    assert c.free_pages() == 64 and c.slots.available == 4


def test_model_length_ends_a_request():
    s, c = make(max_model_len=12)
    a = s.add(req("a", 10, max_tokens=50, ignore_eos=True))
    s.add(req("long", 13))
    while s.has_work():
        run_step(s, c)
    assert a.finish_reason == "length" and len(a.prompt) + len(a.output) == 13 and c.kv_len if True else None
    assert [r.finish_reason for r in s.finished if r.request_id == "long"] == ["error"]


def test_prompts_wait_or_shrink_when_pages_are_short():
    s, c = make(num_pages=8, page=4, max_batch_tokens=64)        # 32 tokens of cache
    s.add(req("a", 20, max_tokens=4))
    s.add(req("b", 20, max_tokens=4))
    st, _ = run_step(s, c)
    assert portions(st) == [("a", 0, 20, True)]                    # b would not fit whole beside a: it waits
    assert [r.request_id for r in s.waiting] == ["b"]
    while any(r.request_id == "a" for r in s.running):
        st, _ = run_step(s, c)
    assert c.free_pages() >= 5
    st, _ = run_step(s, c)
    assert ("b", 0, 20, True) in portions(st)


def test_prompts_under_way_that_hold_the_whole_pool_do_not_stall():
    """Two long prompts taken in portions can come to hold every page between them with neither
    finished; then one is given up so that the other goes on, and both finish in the end."""
    s, c = make(num_pages=10, page=8, max_batch_tokens=16, chunked_prefill_size=5, max_batch_seqs=4)
    s.add(req("a", 41, max_tokens=3, ignore_eos=True))
    s.add(req("b", 61, max_tokens=3, ignore_eos=True))
    # bring about the state by hand: both admitted, 40 tokens each, no page free
    for r in list(s.waiting):
        s.waiting.remove(r)
        s.running.append(r)
        c.add_request(r.request_id)
        c.append(r.request_id, 40)
        r.num_computed = 40
    assert c.free_pages() == 0
    st, _ = run_step(s, c)
    assert [r.request_id for r in st.preempted] == ["a"]            # shortest prompt among those without output
    assert portions(st) and portions(st)[0][0] == "b"
    for _ in range(200):
        if not s.has_work():
            break
        run_step(s, c)
    assert not s.has_work() and c.free_pages() == 10
    assert sorted((r.request_id, r.finish_reason, len(r.output)) for r in s.finished) == \
        [("a", "length", 3), ("b", "length", 3)]
    # and admission keeps room for what running prompts will still take: b (61 tokens, 8 pages)
    # is not started beside a (41 tokens, 6 pages) in a pool of 10
    s, c = make(num_pages=10, page=8, max_batch_tokens=16, chunked_prefill_size=5, max_batch_seqs=4)
    s.add(req("a", 41, max_tokens=3, ignore_eos=True))
    s.add(req("b", 61, max_tokens=3, ignore_eos=True))
    for _ in range(6):
        st, _ = run_step(s, c)
        assert all(e.request.request_id == "a" for e in st.entries)


def test_running_out_of_pages_preempts_by_the_reference_order():
    # victim: most generated tokens, then shortest prompt
    # (crates/infer-scheduler/src/application/control_fns.rs:322-338); it goes back to the front
    # with prompt + generated and is recomputed (inference_session/table.rs:767-815)
    s, c = make(num_pages=12, page=4, max_batch_tokens=64)
    a = s.add(req("a", 7, max_tokens=30, ignore_eos=True))
    b = s.add(req("b", 6, max_tokens=30, ignore_eos=True))
    st, _ = run_step(s, c)
    assert len(st.entries) == 2
    preempted = None
    for _ in range(40):
        st, _ = run_step(s, c)
        if st.preempted:
            preempted = st
            break
    assert preempted is not None
    victim = preempted.preempted[0]
    assert victim is b                                  # equal output, shorter prompt
    assert victim.num_computed == 0 and victim.preemptions == 1 and s.waiting[0] is victim
    assert not c.has_request("b")
    assert [e.request.request_id for e in preempted.entries] == ["a"]
    n_out = len(victim.output)
    while s.has_work():
        st, _ = run_step(s, c)
        for e in st.entries:
            if e.request is victim and e.start == 0:
                assert e.count == len(victim.prompt) + n_out >= 7   # recomputed from prompt + generated
    assert len(a.output) == 30 and len(b.output) == 30
    assert s.stats["preemptions"] >= 1 and c.free_pages() == 12


def test_a_request_too_large_for_the_pool_fails_alone():
    s, c = make(num_pages=4, page=4)
    big = s.add(req("big", 17))
    ok = s.add(req("ok", 10, max_tokens=20, ignore_eos=True))
    while s.has_work():
        run_step(s, c)
    assert big.finish_reason == "error" and big.output == []
    assert ok.finish_reason == "error" and len(ok.prompt) + len(ok.output) >= 16   # grew until the pool was full
    assert c.free_pages() == 4


def test_abort_gives_everything_back():
    s, c = make()
    s.add(req("a", 9))
    s.add(req("b", 9))
    run_step(s, c)
    s.abort("a")
    assert not c.has_request("a") and [r.request_id for r in s.running] == ["b"]
    assert s.finished[0].finish_reason == "cancelled"


# -- tokens that reach the host one step late ------------------------------------------
def lagged_run(s, cache, tokens_of, max_steps=200):
    """Drive the scheduler as the pipelined loop does: commit with marks, resolve a step later."""
    from rustinfer_amd.engine.scheduler import PENDING
    prev, n = None, 0
    while (s.has_work() or prev) and n < max_steps:
        st = s.schedule()
        marks = None
        if st.entries:
            for e in st.entries:
                rid = e.request.request_id
                if not cache.has_request(rid):
                    cache.add_request(rid)
                assert cache.append(rid, e.count) == e.start
                toks = e.request.tokens[e.start:e.start + e.count]
                assert PENDING not in toks[:-1]
            s.commit(st, None)
            marks = [(e.request, len(e.request.output) - 1) for e in st.entries if e.final]
        if prev:
            for r, index in prev:
                s.resolve(r, index, tokens_of(r, index))
        prev = marks
        cache.check()
        n += 1
    assert n < max_steps


def test_late_tokens_give_the_same_outputs():
    seqs = {"a": [5, 6, 0, 9, 9], "b": [1, 2, 3, 4, 5, 6, 7], "c": [0], "d": [4, 4, 4]}
    s, c = make(max_batch_tokens=8, chunked_prefill_size=3)
    a = s.add(req("a", 7, max_tokens=5))                       # ends on its third token (eos 0)
    b = s.add(req("b", 2, max_tokens=4, ignore_eos=True))      # ends by length
    cc = s.add(req("c", 5, max_tokens=3))                      # ends on its first token
    d = s.add(req("d", 3, max_tokens=3))                       # length, no eos
    # a step that ran ahead of an end-of-sequence token produces a token nobody wants: 99
    lagged_run(s, c, lambda r, i: seqs[r.request_id][i] if i < len(seqs[r.request_id]) else 99)
    assert (a.output, a.finish_reason) == ([5, 6, 0], "eos")
    assert (b.output, b.finish_reason) == ([1, 2, 3, 4], "length")
    assert (cc.output, cc.finish_reason) == ([0], "eos")
    assert (d.output, d.finish_reason) == ([4, 4, 4], "length")
    assert c.free_pages() == 64 and c.slots.available == 4 and len(s.finished) == 4


def test_late_end_of_sequence_on_the_last_allowed_token():
    s, c = make()
    a = s.add(req("a", 3, max_tokens=2))
    lagged_run(s, c, lambda r, i: [7, 0, 99][min(i, 2)])
    assert (a.output, a.finish_reason) == ([7, 0], "eos")


def test_preemption_with_a_token_still_on_the_device():
    s, c = make(num_pages=12, page=4, max_batch_tokens=64)
    a = s.add(req("a", 7, max_tokens=30, ignore_eos=True))
    b = s.add(req("b", 6, max_tokens=30, ignore_eos=True))
    lagged_run(s, c, lambda r, i: 10 + i)
    assert a.output == [10 + i for i in range(30)] and b.output == [10 + i for i in range(30)]
    assert s.stats["preemptions"] >= 1 and c.free_pages() == 12


# -- stop sequences (crates/infer-scheduler/src/domain/inference_session/table.rs:541-560) ------
def test_stop_sequences_end_a_request_and_are_taken_off_the_output():
    s, c = make()
    a = s.add(req("a", 3, max_tokens=9, stop_sequences=((4, 5), (3, 4, 5))))     # the longest match goes
    b = s.add(req("b", 3, max_tokens=9, stop_sequences=((2,),)))                  # ends on its first token
    d = s.add(req("d", 3, max_tokens=4, stop_sequences=((8, 9),)))                # never matches
    seq = {"a": [1, 3, 4, 5, 6], "b": [2, 2], "d": [9, 8, 8, 8, 8]}
    pos = {k: 0 for k in seq}

    def token(r):
        pos[r.request_id] += 1
        return seq[r.request_id][pos[r.request_id] - 1]
    while s.has_work():
        run_step(s, c, token)
    assert (a.output, a.finish_reason) == ([1], "stop")
    assert (b.output, b.finish_reason) == ([], "stop")
    assert (d.output, d.finish_reason) == ([9, 8, 8, 8], "length")
    assert c.free_pages() == 64 and c.slots.available == 4


def test_stop_sequences_with_late_tokens():
    seqs = {"a": [1, 3, 4, 5, 6, 6, 6], "b": [7, 7, 4, 5]}
    s, c = make()
    a = s.add(req("a", 3, max_tokens=9, stop_sequences=((4, 5),)))
    b = s.add(req("b", 2, max_tokens=4, stop_sequences=((4, 5),)))   # the match ends on the last allowed token
    lagged_run(s, c, lambda r, i: seqs[r.request_id][i] if i < len(seqs[r.request_id]) else 99)
    assert (a.output, a.finish_reason) == ([1, 3], "stop")
    assert (b.output, b.finish_reason) == ([7, 7], "stop")
    assert c.free_pages() == 64 and c.slots.available == 4 and len(s.finished) == 2


def test_stop_sequences_are_token_ids():
    with pytest.raises(ValueError):
        SamplingParams(stop_sequences=("ab",)).validate()
