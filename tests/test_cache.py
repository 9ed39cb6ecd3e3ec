"""Page allocator and cache manager bookkeeping (no GPU): no page lost, held twice or freed
twice, under random orders of requests."""
import random

import pytest

from rustinfer_amd.cache import CacheError, CacheManager, OutOfPages, PageAllocator, pages_for
from rustinfer_amd.parts import PagedKVNeed, StateNeed


# -- allocator: the reference's cases (crates/infer-worker/src/domain/global_kv_alloc.rs:470-723)
def test_alloc_is_ascending_and_smallest_first():
    a = PageAllocator(8)
    assert a.alloc(3) == [0, 1, 2] and a.alloc(2) == [3, 4]
    a.free([1, 3])
    assert a.available == 5 and a.outstanding == 3
    assert a.alloc(3) == [1, 3, 5]                 # freed ids come back first, in order
    assert a.alloc(0) == []


def test_alloc_full_reports_need_and_available():
    a = PageAllocator(4)
    a.alloc(3)
    with pytest.raises(OutOfPages) as e:
        a.alloc(2)
    assert (e.value.need, e.value.available) == (2, 1)
    assert a.available == 1                        # nothing was taken


def test_double_free_and_out_of_range_are_errors():
    a = PageAllocator(4)
    ids = a.alloc(2)
    a.free(ids)
    for bad in ([0], [7], [-1]):
        with pytest.raises(CacheError):
            a.free(bad)
    b = a.alloc(1)
    with pytest.raises(CacheError):
        a.free(b + b)
    assert a.is_held(b[0])                         # a refused free changes nothing


def test_allocator_fuzz_conserves_pages_and_replays():
    def run(seed):
        rng = random.Random(seed)
        a = PageAllocator(64)
        held, log = [], []
        for _ in range(1000):
            if held and rng.random() < 0.45:
                k = rng.randrange(1, min(len(held), 8) + 1)
                out = [held.pop(rng.randrange(len(held))) for _ in range(k)]
                a.free(out)
            else:
                n = rng.randrange(0, 9)
                try:
                    got = a.alloc(n)
                except OutOfPages:
                    got = []
                assert not set(got) & set(held)
                held += got
                log.append(tuple(got))
            assert a.outstanding + a.available == a.total and a.outstanding == len(held)
        return log
    assert run(3) == run(3)                        # same history, same ids


# -- manager
def manager(num_pages=16, page=4, window=None, max_requests=4, max_len=64, extra=None):
    needs = {0: PagedKVNeed(2, 16), 1: PagedKVNeed(2, 16)}
    if window:
        needs[2] = PagedKVNeed(2, 16, window)
    if extra:
        needs.update(extra)
    return CacheManager(needs, page, num_pages, max_requests, max_len, device=None)


def test_layers_with_the_same_need_share_a_group():
    m = manager(window=6, extra={3: StateNeed((4,)), 4: PagedKVNeed(1, 32)})
    assert len(m.groups) == 3
    assert m.groups[0].cache_ids == [0, 1] and m.groups[1].cache_ids == [2] and m.groups[2].cache_ids == [4]
    assert 3 in m and 5 not in m


def test_pages_follow_the_tokens():
    m = manager()
    m.add_request("a")
    assert m.append("a", 5) == 0 and m.table(0, "a") == [0, 1]
    assert m.append("a", 3) == 5 and m.table(0, "a") == [0, 1]          # fills the last page
    assert m.append("a", 1) == 8 and m.table(0, "a") == [0, 1, 2]       # a new page at the edge
    m.add_request("b")
    m.append("b", 4)
    assert m.table(0, "b") == [3] and m.kv_len("b") == 4 and m.pages_held("a") == 3
    m.release("a")
    m.add_request("c")
    m.append("c", 9)
    assert m.table(0, "c") == [0, 1, 2]                                  # pages are used again
    m.check()


def test_out_of_pages_changes_nothing():
    m = manager(num_pages=3)
    m.add_request("a")
    m.append("a", 8)
    assert m.can_append([("a", 4)]) and not m.can_append([("a", 5)])
    assert m.can_append([("new", 4)]) and not m.can_append([("a", 1), ("new", 1)])
    with pytest.raises(OutOfPages):
        m.append("a", 5)
    assert m.kv_len("a") == 8 and m.table(0, "a") == [0, 1]
    m.check()


def test_misuse_is_refused():
    m = manager(max_requests=1, max_len=8)
    with pytest.raises(CacheError):
        m.append("ghost", 1)
    m.add_request("a")
    with pytest.raises(CacheError):
        m.add_request("a")
    with pytest.raises(OutOfPages):
        m.add_request("b")                          # no state slot left
    assert not m.can_append([("b", 1)])
    with pytest.raises(CacheError):
        m.append("a", 9)                            # longer than the model allows
    m.release("a")
    with pytest.raises(CacheError):
        m.release("a")


def test_state_slots_are_taken_and_returned():
    m = manager(max_requests=3, extra={7: StateNeed((5,))})
    slots = [m.add_request(r) for r in "abc"]
    assert slots == [0, 1, 2]
    m.release("b")
    assert m.add_request("d") == 1 and m.slot("d") == 1
    m.check()


def test_window_gives_pages_back_as_it_passes():
    m = manager(num_pages=8, page=4, window=6, max_len=64)
    m.add_request("a")
    total = 0
    for n in (5, 1, 1, 7, 2, 1, 9, 3, 1, 1, 1):
        start = m.append("a", n)
        assert start == total
        total += n
        full, win = m.table(0, "a"), m.table(1, "a")
        assert len(full) == len(win) == pages_for(total, 4)
        first = max(0, start - 6 + 1) // 4          # first page the earliest query of this step reads
        assert all(p == -1 for p in win[:first]) and all(p >= 0 for p in win[first:])
        assert all(p >= 0 for p in full)
        m.check()
    assert m.groups[1].allocator.outstanding <= 5
    m.release("a")
    assert all(g.allocator.available == 8 for g in m.groups)


def test_truncate_undoes_appends():
    m = manager(num_pages=8, page=4, window=6, max_len=64)
    m.add_request("a")
    m.append("a", 9)
    tables = [list(m.table(g, "a")) for g in range(2)]
    free = [g.allocator.available for g in m.groups]
    start = m.append("a", 11)                      # the window gives its first page back here
    assert start == 9 and m.table(1, "a")[0] == -1
    m.truncate("a", 9)
    m.check()
    assert m.kv_len("a") == 9 and m.table(0, "a") == tables[0]
    assert m.table(1, "a") == [-1] + tables[1][1:]  # no query at 9 or later reads that page
    assert [g.allocator.available for g in m.groups] == [free[0], free[1] + 1]
    assert m.append("a", 11) == 9                  # and the same tokens can be appended again
    m.check()
    with pytest.raises(CacheError, match="cannot truncate"):
        m.truncate("a", 21)
    with pytest.raises(CacheError, match="window has given back"):
        m.truncate("a", 3)                         # position 3 would read the page that is gone
    with pytest.raises(CacheError, match="not live"):
        m.truncate("b", 0)
    m.truncate("a", 20)
    m.truncate("a", 20)
    m.release("a")
    assert all(g.allocator.available == 8 for g in m.groups)


def test_state_tensors_hold_a_scratch_slot_beyond_the_requests():
    import torch
    m = CacheManager({0: PagedKVNeed(1, 16), 5: StateNeed((3, 2))}, 4, 4, 3, 16, device="cpu",
                     dtype=torch.float32)
    assert m.scratch_slot == 3 and tuple(m.state_tensors[5].shape) == (4, 3, 2)
    assert [m.add_request(r) for r in "abc"] == [0, 1, 2]       # requests never get the scratch slot
    with pytest.raises(OutOfPages):
        m.add_request("d")
    assert m.state_bytes() == 4 * 6 * 4


def test_random_orders_of_requests():
    rng = random.Random(11)
    m = manager(num_pages=24, page=4, window=10, max_requests=4, max_len=48)
    live, next_id, peak = {}, 0, 0
    for _ in range(3000):
        r = rng.random()
        if live and r < 0.15:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        elif len(live) < 4 and r < 0.35:
            m.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 5, 8, 13])
            if live[rid] + n > 48:
                continue
            ok = m.can_append([(rid, n)])
            try:
                start = m.append(rid, n)
                assert ok
                live[rid] += n
                if rng.random() < 0.2:             # the step failed: the append is undone
                    m.truncate(rid, start)
                    live[rid] = start
            except OutOfPages:
                assert not ok
        m.check()
        assert {rid: m.kv_len(rid) for rid in live} == live
        for g in m.groups:
            held = sorted(p for t in g.tables.values() for p in t if p >= 0)
            assert len(held) == len(set(held)) == g.allocator.outstanding
            if g.need.window is None:
                assert len(held) == sum(pages_for(n, 4) for n in live.values())
        peak = max(peak, m.groups[0].allocator.outstanding)
    for rid in list(live):
        m.release(rid)
    assert all(g.allocator.available == g.num_pages for g in m.groups) and m.slots.available == 4
    assert peak > 12


def test_workspace_buffers_grow_by_half_and_are_kept_only_for_graphs():
    """Scratch buffers: steps of slowly growing sizes do not allocate a buffer each, and an
    outgrown buffer is kept alive only once a captured graph may point into it."""
    import torch
    from rustinfer_amd.engine.context import Workspace
    ws = Workspace(torch.device("cpu"))
    a = ws.get("x", 10, 4, torch.float32)
    assert a.shape == (10, 4) and ws.get("x", 7, 4, torch.float32).data_ptr() == a.data_ptr()
    grown = [ws.get("x", n, 4, torch.float32).data_ptr() for n in range(11, 60)]
    assert len(set(grown)) <= 5 and not ws._retired            # 10 -> 15 -> 22 -> 33 -> 49 -> 73
    assert ws.get("x", 1000, 4, torch.float32).shape == (1000, 4)          # a jump is taken as it is
    ws.frozen = True                                           # a graph has been captured
    ws.frozen = False
    before = ws.get("x", 1000, 4, torch.float32)
    ws.get("x", 1001, 4, torch.float32)
    assert len(ws._retired) == 1 and ws._retired[0].data_ptr() == before.data_ptr()
    assert ws.get("y", 3, 8, torch.bfloat16).dtype == torch.bfloat16 and ws.nbytes() > 0
