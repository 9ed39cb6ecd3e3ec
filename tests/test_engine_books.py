"""The step function's bookkeeping, without a GPU: a model that computes nothing stands in
for the real one, so that what a failed step leaves behind, what the validation refuses and
the size of the control buffer can be tested on the CPU."""
import pytest
import torch

from rustinfer_amd.cache import OutOfPages
from rustinfer_amd.engine import Engine, StepEntry, StepError, device_token
from rustinfer_amd.parts import PagedKVNeed, Runtime, StateNeed


class NothingModel:
    """Has the interface the engine uses; its forward pass returns zeros or raises."""
    vocab_size = 50
    graph_safe = True

    def __init__(self, window=None):
        self.window = window
        self.fail = None
        self.seen = []

    def prepare(self, rt, max_positions):
        pass

    def cache_needs(self):
        needs = {0: PagedKVNeed(1, 16), 1: PagedKVNeed(1, 16), 2: StateNeed((4,))}
        if self.window:
            needs[3] = PagedKVNeed(1, 16, self.window)
        return needs

    def forward(self, ctx, caches):
        self.seen.append(ctx)
        if self.fail is not None:
            raise self.fail
        return torch.zeros(ctx.num_want, self.vocab_size)


def engine(window=None, **kw):
    rt = Runtime(device=torch.device("cpu"), dtype=torch.float32, ops=None)
    opts = dict(page_size=4, num_pages=12, max_requests=3, max_model_len=40, max_batch_tokens=32)
    opts.update(kw)
    return Engine(NothingModel(window), rt, **opts)


def books(eng):
    c = eng.cache
    return ({r: c.kv_len(r) for r in c.live_requests()}, [g.allocator.available for g in c.groups],
            c.slots.available, {r: [list(g.tables[r]) for g in c.groups] for r in c.live_requests()})


@pytest.mark.parametrize("window", [None, 6])
def test_a_failed_step_is_undone(window):
    """The forward pass raises: every request is as long as before, requests the step started are
    gone, the pages are free again, and the same step runs afterwards
    (crates/infer-worker/src/application/worker_scheduler.rs:1090-1133)."""
    eng = engine(window)
    eng.step([StepEntry("a", [1] * 9, [8]), StepEntry("b", [2] * 3, [])])
    before = books(eng)
    step = [StepEntry("a", [3] * 11, [10]), StepEntry("c", [4] * 6, [5]), StepEntry("b", [5], [0])]
    eng.model.fail = RuntimeError("kernel refused")
    with pytest.raises(RuntimeError, match="kernel refused"):
        eng.step(step)
    eng.cache.check()
    after = books(eng)
    if window:
        # the window group gave back a page of "a" that no query from position 9 on reads; it stays free
        assert after[0] == before[0] and after[2] == before[2]
        assert after[1][:1] == before[1][:1] and after[1][1] == before[1][1] + 1
    else:
        assert after == before
    assert not eng.cache.has_request("c")
    eng.model.fail = None
    assert tuple(eng.step(step).shape) == (3, 50)
    assert eng.cache.kv_len("a") == 20 and eng.cache.kv_len("c") == 6 and eng.cache.kv_len("b") == 4
    eng.cache.check()
    # KeyboardInterrupt and the like are undone too
    eng.model.fail = KeyboardInterrupt()
    before = books(eng)
    with pytest.raises(KeyboardInterrupt):
        eng.step([StepEntry("b", [1, 2, 3, 4, 5], [])])
    assert books(eng) == before


def test_a_failed_step_leaves_fixed_size_state_as_it_was():
    """A layer with state of its own updates its slot in place.  A step that fails after such a
    layer ran is undone there too: the same step, run again, starts from the state before it."""
    eng = engine()
    state = eng.cache.state_tensors[2]

    def forward(ctx, caches, fail=False):
        view = caches.view(2)
        for slot, q in zip(ctx.host_slots, ctx.host_q_lens):
            view.state[slot] += q                      # the layer's update, in place
        if fail:
            raise RuntimeError("a later layer refused")
        return torch.zeros(ctx.num_want, 50)

    eng.model.forward = forward
    eng.step([StepEntry("a", [1] * 5, []), StepEntry("b", [2] * 2, [])])
    sa, sb = eng.cache.slot("a"), eng.cache.slot("b")
    assert state[sa].tolist() == [5.0] * 4 and state[sb].tolist() == [2.0] * 4
    eng.model.forward = lambda ctx, caches: forward(ctx, caches, fail=True)
    step = [StepEntry("a", [1] * 3, []), StepEntry("c", [3] * 4, []), StepEntry("b", [2], [0])]
    with pytest.raises(RuntimeError, match="later layer"):
        eng.step(step)
    assert state[sa].tolist() == [5.0] * 4 and state[sb].tolist() == [2.0] * 4
    assert not eng.cache.has_request("c")
    eng.model.forward = forward
    eng.step(step)
    assert state[sa].tolist() == [8.0] * 4 and state[sb].tolist() == [3.0] * 4
    eng.cache.check()


def test_out_of_pages_changes_nothing_and_is_told_before_the_forward():
    eng = engine(num_pages=3)
    eng.step([StepEntry("a", [1] * 8, [])])
    before = books(eng)
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1], []), StepEntry("b", [1] * 5, [])])
    assert books(eng) == before and len(eng.model.seen) == 1


def test_a_device_token_may_only_be_an_entrys_last():
    eng = engine()
    eng.step([StepEntry("a", [1, 2, device_token(2)], [2])])
    eng.step([StepEntry("a", [device_token(0)], [0])])
    for bad in ([device_token(0), 1], [1, -1, 2], [-1, -1]):
        with pytest.raises(StepError, match="only be an entry's last"):
            eng.step([StepEntry("b", bad, [])])
    with pytest.raises(StepError, match="no device token"):
        eng.step([StepEntry("b", [1, device_token(3)], [])])      # three slots: -1, -2, -3
    with pytest.raises(StepError, match="outside"):
        eng.step([StepEntry("b", [50], [])])
    assert not eng.cache.has_request("b")


def test_the_control_buffer_is_sized_once_for_the_largest_step():
    """Captured graphs hold addresses inside the device buffer: it must never be replaced."""
    eng = engine(window=6, max_batch_tokens=32, max_requests=3, max_model_len=40, num_pages=40)
    dev = eng._staging.dev
    eng.step([StepEntry("a", [1] * 14, list(range(14))), StepEntry("b", [1] * 9, list(range(9))),
              StepEntry("c", [1] * 9, list(range(9)))])                # 32 tokens, every place wanted
    for _ in range(26):
        eng.step([StepEntry(r, [1], [0]) for r in "abc"])               # up to the longest request
    assert eng.cache.kv_len("a") == 40
    assert eng._staging.dev is dev and eng._staging.dev.data_ptr() == dev.data_ptr()
    ctx = eng.model.seen[-1]
    assert ctx.state_slots.tolist() == [0, 1, 2]
    with pytest.raises(StepError, match="exceeds the staging buffer"):
        eng._staging.next(eng._staging.ints + 1)


def test_rows_of_no_request_point_at_the_scratch_slot():
    eng = engine()
    ctx = eng._build_context([], [], pad_rows_to=2, want_all=True)
    assert ctx.num_rows == 2 and ctx.num_tokens == 2 and ctx.num_want == 2
    assert ctx.row_of_token.tolist() == [-1, -1] and ctx.state_slots.tolist() == [3, 3]
    assert ctx.kv_lens.tolist() == [0, 0] and ctx.max_q_len == 1
    eng.step([StepEntry("a", [1], [0])])
    ctx = eng._build_context([StepEntry("a", [1], [0])], [1], pad_rows_to=2, want_all=True)
    assert ctx.row_of_token.tolist() == [0, -1] and ctx.state_slots.tolist() == [0, 3]


def test_pool_size_from_free_memory_counts_the_state():
    """Pages from free memory: the fixed-size state of all slots comes off the budget first."""
    from rustinfer_amd.engine.factory import pages_that_fit
    kv = {0: PagedKVNeed(2, 64), 1: PagedKVNeed(2, 64)}            # 2 layers: 2 * 2 * 2 * 64 * 16 * 2 B = 16 KiB a page
    free = (1 << 30) + (100 << 20)                                 # 100 MiB beyond the reserve
    assert pages_that_fit(kv, 16, 2, free, 1.0, 8, 1 << 20) == (100 << 20) // (16 << 10)
    assert pages_that_fit(kv, 16, 2, free, 0.5, 8, 1 << 20) == (50 << 20) // (16 << 10)
    assert pages_that_fit(kv, 16, 2, free, 1.0, 8, 4096) == 8 * 256                      # never more than the requests can use
    state = dict(kv)
    state[2] = StateNeed((1024, 1024), torch.float32)              # 4 MiB a slot, 9 slots
    assert pages_that_fit(state, 16, 2, free, 1.0, 8, 1 << 20) == ((100 - 36) << 20) // (16 << 10)
    assert pages_that_fit({2: StateNeed((4,))}, 16, 2, free, 1.0, 8, 4096) == 1          # no paged layers at all
    assert pages_that_fit(kv, 16, 2, 1 << 20, 1.0, 8, 4096) == 1                         # nothing free: one page, and the allocation will say so


def test_profile_forward_and_resize():
    """The largest step runs once on requests of its own, which are gone afterwards; the pool can
    then be replaced by one of another size, but not once requests are live."""
    from rustinfer_amd.cache import CacheError
    eng = engine(num_pages=12, max_requests=3, max_model_len=40, max_batch_tokens=32, page_size=4)
    assert eng.profile_forward() == 32
    ctx = eng.model.seen[-1]
    assert ctx.num_tokens == 32 and ctx.num_rows == 1 and ctx.num_want == 1
    assert not eng.cache.live_requests() and eng.cache.free_pages() == 12
    eng.cache.check()
    big = engine(num_pages=40, max_requests=3, max_model_len=16, max_batch_tokens=100, page_size=4)
    assert big.profile_forward() == 48                     # three rows of the longest request
    assert [len(x) for x in big.model.seen[-1].host_q_lens and [big.model.seen[-1].host_q_lens]] == [3]
    small = engine(num_pages=2, max_batch_tokens=32)
    assert small.profile_forward() == 0 and not small.model.seen
    eng.resize_pool(30)
    assert eng.cache.free_pages() == 30 and all(g.num_pages == 30 for g in eng.cache.groups)
    eng.step([StepEntry("a", [1] * 9, [8])])
    with pytest.raises(CacheError, match="resized"):
        eng.resize_pool(12)
