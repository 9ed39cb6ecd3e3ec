"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a caller
without torch would: its tokens are those of the entry point that takes the caller's scratch
buffer, on two calls in a row, the second with a smaller input that leaves most of the shared
array as the first call wrote it."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _argmax_both(lib, logits):
    R, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = torch.full((R,), -7, dtype=torch.int32, device="cuda")
    got = torch.full((R,), -9, dtype=torch.int32, device="cuda")
    scratch = torch.empty(2 * R * lib.ri_argmax_slices(V), dtype=torch.int32, device="cuda")
    rc = lib.ri_argmax(ctypes.c_void_p(logits.data_ptr()), R, V, logits.stride(0), ctypes.c_void_p(want.data_ptr()),
                       ctypes.c_void_p(scratch.data_ptr()), stream)
    assert rc == 0, lib.ri_last_error()
    torch.cuda.synchronize()
    # free bytes as the driver counts them (torch's own counters would not see a hipMalloc inside
    # the library); torch's allocator is at rest between the two readings
    free_before = torch.cuda.mem_get_info()[0]
    rc = lib.ri_argmax_no_alloc(ctypes.c_void_p(logits.data_ptr()), R, V, logits.stride(0),
                                ctypes.c_void_p(got.data_ptr()), stream)
    assert rc == 0, lib.ri_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    return want.cpu(), got.cpu()


def test_argmax_without_allocation_can_be_captured_in_a_graph():
    """A stream capture in the global mode refuses hipMalloc, hipFree and every call that
    synchronises: an entry point that made one would fail here or invalidate the capture.  The
    graph is replayed three times on changing logits, with eager work and a wait between the
    replays, and each replay gives the tokens of the entry point with the caller's buffer."""
    from rustinfer_amd.kernels import build
    lib = build.load()
    assert lib.ri_no_alloc_init() == 0, lib.ri_last_error()      # the address lookup happens before the capture
    gen = torch.Generator(device="cuda").manual_seed(6)
    R, V = 9, 50021
    logits = torch.randn(R, V, device="cuda", generator=gen)
    got = torch.full((R,), -9, dtype=torch.int32, device="cuda")
    want = torch.full((R,), -7, dtype=torch.int32, device="cuda")
    scratch = torch.empty(2 * R * lib.ri_argmax_slices(V), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):                                    # capture_error_mode "global"
        rc = lib.ri_argmax_no_alloc(ctypes.c_void_p(logits.data_ptr()), R, V, logits.stride(0),
                                    ctypes.c_void_p(got.data_ptr()),
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.ri_last_error()
    assert (got == -9).all()                                     # captured, not run
    for k in range(3):
        logits.copy_(torch.randn(R, V, device="cuda", generator=gen))
        logits[k, 40000 + k] = 99.0
        g.replay()
        rc = lib.ri_argmax(ctypes.c_void_p(logits.data_ptr()), R, V, logits.stride(0), ctypes.c_void_p(want.data_ptr()),
                           ctypes.c_void_p(scratch.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.ri_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, want) and got[k].item() == 40000 + k
        assert torch.equal(got.long(), logits.argmax(dim=1))


def test_argmax_without_allocation_matches_the_one_with_a_scratch_buffer():
    from rustinfer_amd.kernels import build
    lib = build.load()
    assert lib.ri_no_alloc_init() == 0, lib.ri_last_error()
    assert lib.ri_argmax_no_alloc_max_rows() == 1024
    gen = torch.Generator(device="cuda").manual_seed(5)
    # first call: many rows of a large vocabulary (64 slices a row), rows with a stride
    big = torch.randn(200, 128256 + 64, device="cuda", generator=gen)[:, :128256]
    big[3, 77] = big[3, 100000] = 50.0                       # a tie: the lower index wins
    big[5] = float("-inf")
    want, got = _argmax_both(lib, big)
    assert torch.equal(want, got) and got[3] == 77
    lib_rows = [r for r in range(200) if r not in (3, 5)]        # the library's choice on ties is its own
    assert torch.equal(got.long()[lib_rows], big.argmax(dim=1).cpu()[lib_rows]) and got[5] == 0
    # second call, smaller: fewer rows, one slice a row, then fewer rows of many slices
    for rows, V in ((3, 5000), (7, 20001)):
        small = torch.randn(rows, V, device="cuda", generator=gen)
        want, got = _argmax_both(lib, small)
        assert torch.equal(want, got)
        assert torch.equal(got.long(), small.argmax(dim=1).cpu())
    # sizes beyond the array are refused, with a message, and nothing is launched
    out = torch.zeros(1025, dtype=torch.int32, device="cuda")
    wide = torch.zeros(1025, 16, device="cuda")
    rc = lib.ri_argmax_no_alloc(ctypes.c_void_p(wide.data_ptr()), 1025, 16, 16, ctypes.c_void_p(out.data_ptr()),
                                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc != 0 and b"1025 rows exceed" in lib.ri_last_error()
