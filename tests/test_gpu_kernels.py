"""Each kernel alone against a plain PyTorch 32-bit/64-bit reference of the same op, at sizes
other than the engine tests use (widths and vocabularies that are no power of two, head sizes
in steps of 16, odd head counts and groups)."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_llama
from rustinfer_amd.engine.context import Workspace

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from rustinfer_amd.kernels import build, ops
    build.load()
    return ops


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1.6e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,d,V", [(1, 64, 50), (7, 200, 333), (33, 2056, 1001)])
def test_embed(ops, dtype, T, d, V):
    table = rnd(V, d, dtype=dtype)
    ids = torch.randint(0, V, (T,), dtype=torch.int32, device=DEV)
    out = torch.empty(T, d, device=DEV)
    ops.embed(ids, table, out)
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("T,d,eps", [(1, 64, 1e-5), (5, 200, 1e-6), (3, 4096, 1e-5), (2, 5000, 1e-3)])
def test_add_rmsnorm(ops, dtype, wdtype, T, d, eps):
    x = rnd(T, d, seed=1)
    delta = rnd(T, d, dtype=dtype, seed=2)
    w = (1 + 0.1 * rnd(d, seed=3)).to(wdtype)
    out = torch.empty(T, d, dtype=dtype, device=DEV)
    x0 = x.clone()
    ops.add_rmsnorm(x, delta, w, eps, out)
    s = x0.double() + delta.double()
    assert torch.allclose(x.double(), s, rtol=1e-6, atol=1e-6)          # residual written back in 32-bit
    ref = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps) * w.double()
    assert torch.allclose(out.double(), ref, **tol(dtype))
    # without a delta the residual is untouched
    x1 = x.clone()
    ops.add_rmsnorm(x, None, w, eps, out)
    assert torch.equal(x, x1)
    ref = x1.double() * torch.rsqrt((x1.double() ** 2).mean(-1, keepdim=True) + eps) * w.double()
    assert torch.allclose(out.double(), ref, **tol(dtype))
    # unit weight: mean square of the output is 1 (crates/infer-backend-cpu/src/lib.rs:1317-1328)
    if dtype == torch.float32:
        ops.add_rmsnorm(x, None, torch.ones(d, device=DEV), eps, out)
        assert torch.allclose((out.double() ** 2).mean(-1), torch.ones(T, dtype=torch.float64, device=DEV), atol=1e-2)


def test_add_rmsnorm_adds_up_partial_sums(ops):
    T, d, eps = 6, 2048, 1e-5
    x = rnd(T, d, seed=40)
    parts = rnd(4, T, d, seed=41)
    w = (1 + 0.1 * rnd(d, seed=42)).to(torch.bfloat16)
    out = torch.empty(T, d, dtype=torch.bfloat16, device=DEV)
    x0 = x.clone()
    ops.add_rmsnorm(x, parts, w, eps, out)
    s = x0.double() + parts.double().sum(0)
    assert torch.allclose(x.double(), s, rtol=1e-6, atol=1e-6)
    ref = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps) * w.double()
    assert torch.allclose(out.double(), ref, **tol(torch.bfloat16))


@pytest.mark.parametrize("M,N,K", [(1, 2048, 8192), (8, 2048, 2048), (20, 4096, 14336), (64, 160, 416), (3, 100, 72)])
def test_linear_delta_feeds_the_norm(ops, M, N, K):
    """A product with few rows and columns is split over K; the norm adds the slices up."""
    ws = Workspace(DEV)
    x = rnd(M, K, dtype=torch.bfloat16, seed=43)
    w = rnd(N, K, dtype=torch.bfloat16, seed=44, scale=0.02)
    delta = ops.linear_delta(x, w, ws, "t")
    wt = ops.tile_weight(w)
    ref = x.double() @ w.double().t()
    if wt is not None:
        tiled = ops.linear_delta(x, w, Workspace(DEV), "t", wt)
        if M <= 16:
            assert torch.equal(tiled, delta)          # the same kernel on a copy in another order
        else:                                         # 17..64 rows: another kernel, other slices of K
            assert tiled.dim() == 3 and tiled.dtype == torch.float32
            assert torch.allclose(tiled.double().sum(0), ref, rtol=0, atol=2e-6 * max(1.0, ref.abs().max().item()))
    got = delta.double().sum(0) if delta.dim() == 3 else delta.double()
    # split where columns are few and K is long; but a weight without its second copy goes to the
    # GEMM library from 17 rows on (or if it is large), which leaves whole sums in bfloat16
    to_library = M >= ops.UNTILED_LIBRARY_MIN_ROWS or N * K >= ops.UNTILED_LIBRARY_LARGE
    assert (delta.dim() == 3) == (N * 2 <= 8192 and K >= 2048 and not to_library)
    assert delta.dim() == 2 or delta.dtype == torch.float32
    assert torch.allclose(got, ref, rtol=0, atol=(2e-6 if delta.dim() == 3 else 1.6e-2) * max(1.0, ref.abs().max().item()))
    res = rnd(M, N, seed=45)
    res0 = res.clone()
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm(res, delta, torch.ones(N, device=DEV), 1e-5, out)
    s = res0.double() + got
    assert torch.allclose(out.double(), s * torch.rsqrt((s * s).mean(-1, keepdim=True) + 1e-5), **tol(torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm_selected_rows(ops, dtype):
    T, d, eps = 9, 328, 1e-5
    x = rnd(T, d, seed=4)
    delta = rnd(T, d, dtype=dtype, seed=5)
    w = (1 + 0.1 * rnd(d, seed=6)).to(dtype)
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32, device=DEV)
    out = torch.empty(4, d, dtype=dtype, device=DEV)
    x0 = x.clone()
    ops.add_rmsnorm(x, delta, w, eps, out, rows)
    assert torch.equal(x, x0)                       # a gather leaves the residual alone
    s = (x0.double() + delta.double())[rows.long()]
    ref = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps) * w.double()
    assert torch.allclose(out.double(), ref, **tol(dtype))
    # the sums of the gathered rows can be had as well: the residual stream cut down to those rows
    x_rows = torch.full((4, d), 7.0, device=DEV)
    out2 = torch.empty_like(out)
    ops.add_rmsnorm(x, delta, w, eps, out2, rows, x_rows)
    assert torch.equal(x, x0) and torch.equal(out2, out)
    assert torch.allclose(x_rows.double(), s, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,I", [(1, 176), (6, 1000), (3, 8192)])
def test_swiglu(ops, dtype, T, I):
    gu = rnd(T, 2 * I, dtype=dtype, seed=7, scale=2.0)
    out = torch.empty(T, I, dtype=dtype, device=DEV)
    ops.swiglu(gu, out)
    g, u = gu[:, :I].double(), gu[:, I:].double()
    assert torch.allclose(out.double(), g / (1 + torch.exp(-g)) * u, **tol(dtype))


def test_silu_values(ops):
    # silu(0) = 0, silu(1) = 0.7311 (crates/infer-backend-cpu/src/lib.rs:1387-1394)
    gu = torch.tensor([[0.0, 1.0, 1.0, 1.0]], device=DEV)
    out = torch.empty(1, 2, device=DEV)
    ops.swiglu(gu, out)
    assert abs(out[0, 0].item()) == 0.0 and abs(out[0, 1].item() - 0.731058) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 50, 64), (3, 333, 200), (8, 1000, 416), (9, 130, 72),
                                   (16, 2048, 2048), (17, 48, 8192), (33, 100, 1024), (64, 4100, 520),
                                   (70, 257, 136), (200, 96, 1000), (4, 31, 44), (70, 96, 44), (200, 31, 100), (130, 77, 36)])
def test_linear(ops, dtype, M, N, K):
    x = rnd(M, K, dtype=dtype, seed=8)
    w = rnd(N, K, dtype=dtype, seed=9, scale=0.1)
    out = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.linear(x, w, out)
    ref = x.double() @ w.double().t()
    # a 32-bit sum of K terms: rounding grows like sqrt(K) * 2^-24 * the size of the sums
    f32 = dict(rtol=0, atol=1.2e-7 * math.sqrt(K) * ref.abs().max().item())
    assert torch.allclose(out.double(), ref, **(f32 if dtype == torch.float32 else tol(dtype)))
    if dtype == torch.bfloat16:                      # 32-bit output of bfloat16 operands (logits)
        out32 = torch.empty(M, N, device=DEV)
        ops.linear(x, w, out32)
        assert torch.allclose(out32.double(), ref, **f32)
        wt = ops.tile_weight(w)                      # the tile-ordered copy gives the same bits
        assert (wt is not None) == (N % 16 == 0 and K % 32 == 0)
        if wt is not None:
            out_t = torch.empty(M, N, device=DEV)
            ops.linear(x, w, out_t, wt)
            if M < ops.UNTILED_LIBRARY_MIN_ROWS and N * K < ops.UNTILED_LIBRARY_LARGE:
                assert torch.equal(out_t, out32)     # the few-row kernel either way
            else:                                    # without the copy the GEMM library took the product
                assert torch.allclose(out_t.double(), ref, **f32)
        if M > ops.SKINNY_MAX_ROWS:
            # where the GEMM library has no kernel for a problem, the engine's own tiled kernel runs
            # it; here the library is taken to have refused, whatever it would have said
            shape = (N, K, x.stride(0), w.stride(0), N, torch.bfloat16)
            refused = shape in ops._LIBRARY_REFUSED
            ops._LIBRARY_REFUSED.add(shape)
            try:
                own = torch.full((M, N), float("nan"), dtype=dtype, device=DEV)
                ops.linear(x, w, own)
            finally:
                if not refused:
                    ops._LIBRARY_REFUSED.discard(shape)
            assert torch.allclose(own.double(), ref, **tol(dtype))
            print(f"library GEMM for M={M} N={N} K={K}: {'refused' if refused else 'took it'}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,I,K", [(1, 176, 64), (5, 416, 160), (17, 100, 72), (64, 1000, 520), (70, 96, 136), (9, 2048, 512)])
def test_linear_swiglu(ops, dtype, M, I, K):
    x = rnd(M, K, dtype=dtype, seed=20)
    w = rnd(2 * I, K, dtype=dtype, seed=21, scale=0.05)
    out = torch.empty(M, I, dtype=dtype, device=DEV)
    scratch = torch.empty(M, 2 * I, dtype=dtype, device=DEV)
    ops.linear_swiglu(x, w, out, scratch)
    wt = ops.tile_weight(w) if dtype == torch.bfloat16 else None
    g, u = x.double() @ w[:I].double().t(), x.double() @ w[I:].double().t()
    ref = g / (1 + torch.exp(-g)) * u
    if wt is not None:
        out_t = torch.empty_like(out)
        ops.linear_swiglu(x, w, out_t, scratch, wt)
        if M < ops.UNTILED_LIBRARY_MIN_ROWS:
            assert torch.equal(out_t, out)              # the few-row kernel, whichever order it reads the weight in
        else:                                            # without the second copy: the library's product, then the activation
            assert torch.allclose(out_t.double(), ref, **tol(dtype))
    f32 = dict(rtol=0, atol=5e-7 * math.sqrt(K) * max(1.0, ref.abs().max().item()))   # two 32-bit sums of K terms, multiplied
    assert torch.allclose(out.double(), ref, **(f32 if dtype == torch.float32 else tol(dtype)))


@pytest.mark.parametrize("M,N,K", [(17, 16, 32), (64, 4096, 4096), (33, 80, 96), (48, 2048, 8192), (49, 1008, 160), (20, 4096, 14336),
                                   (64, 48, 544), (40, 8192, 160), (50, 24576, 64), (40, 32896, 64)])
def test_rows_kernel_with_activations_in_lds(ops, M, N, K):
    """17..64 rows: the kernel whose blocks share their activations through LDS, as partial sums over
    slices of K, as a whole product in either output type and with the fused SwiGLU."""
    import ctypes
    lib = ops._lib()
    x = rnd(M, K, dtype=torch.bfloat16, seed=90)
    w = rnd(N, K, dtype=torch.bfloat16, seed=91, scale=0.05)
    wt = ops.tile_weight(w)
    ref = x.double() @ w.double().t()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    for nt, groups in ((1, 1), (2, 1), (1, 2), (2, 2), (1, 4), (2, 4)):
        for parts in (1, 2, 3, 16):
            stack = torch.full((parts, M, N), float("nan"), device=DEV)
            assert lib.ri_gemm_rows_bf16(P(x), K, P(wt), P(stack), N, M, N, K, 0, 0, parts, ctypes.c_longlong(M * N), nt, groups, stream) == 0, lib.ri_last_error()
            assert torch.allclose(stack.double().sum(0), ref, rtol=0, atol=2e-6 * max(1.0, ref.abs().max().item()) * math.sqrt(K / 32))
        out = torch.full((M, N + 16), float("nan"), dtype=torch.bfloat16, device=DEV)       # rows with a stride
        assert lib.ri_gemm_rows_bf16(P(x), K, P(wt), P(out), N + 16, M, N, K, 1, 0, 1, ctypes.c_longlong(0), nt, groups, stream) == 0
        assert torch.allclose(out[:, :N].double(), ref, **tol(torch.bfloat16)) and torch.isnan(out[:, N:]).all()
    # through the operations: partial sums for the norm, and SwiGLU where the columns are many
    ws = Workspace(DEV)
    delta = ops.linear_delta(x, w, ws, "t", wt)
    got = delta.double().sum(0) if delta.dim() == 3 else delta.double()
    assert torch.allclose(got, ref, **(dict(rtol=0, atol=2e-6 * max(1.0, ref.abs().max().item()) * math.sqrt(K / 32))
                                       if delta.dim() == 3 else tol(torch.bfloat16)))
    if N % 32 == 0:
        I = N // 2
        act = torch.empty(M, I, dtype=torch.bfloat16, device=DEV)
        g, u = ref[:, :I], ref[:, I:]
        want = g / (1 + torch.exp(-g)) * u
        for groups in (1, 2, 4):
            act = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
            assert lib.ri_gemm_rows_bf16(P(x), K, P(wt), P(act), I, M, I, K, 1, 1, 1, ctypes.c_longlong(0), 1, groups, stream) == 0
            assert torch.allclose(act.double(), want, **tol(torch.bfloat16))
        act = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
        # four groups at I = 4096, two at 12288, one at 16448, else the few-row kernel
        ops.linear_swiglu(x, w, act, None, wt)
        assert torch.allclose(act.double(), want, **tol(torch.bfloat16))
    bad = lib.ri_gemm_rows_bf16(P(x), K, P(wt), P(out), N, M, N, K, 1, 1, 1, ctypes.c_longlong(0), 2, 1, stream)
    assert bad != 0 and b"one gate and one up tile" in lib.ri_last_error()


def test_slices_and_groups_of_the_rows_kernel(ops):
    """The plan for products whose partial sums a norm adds up: no more blocks than run at once."""
    import ctypes
    lib = ops._lib()

    def plan(M, N, K):
        parts, groups = ctypes.c_int(), ctypes.c_int()
        assert lib.ri_gemm_rows_plan(M, N, K, 1, ctypes.byref(parts), ctypes.byref(groups)) == 0
        return parts.value, groups.value

    assert plan(64, 4096, 4096) == (4, 2) and plan(64, 4096, 14336) == (8, 1)
    assert plan(64, 8192, 8192) == (4, 1) and plan(64, 8192, 28672) == (4, 1)
    assert plan(64, 5120, 5120) == (4, 1) and plan(32, 5120, 5120) == (8, 1)     # 80 blocks of columns: 640 at 64 rows would not
    assert plan(64, 2048, 8192) == (8, 2) and plan(20, 64, 64) == (1, 1)
    assert ops._swiglu_groups(8192) == 4 and ops._swiglu_groups(14336) == 2 and ops._swiglu_groups(11008) == 2
    assert ops._swiglu_groups(28672) == 1 and ops._swiglu_groups(9000) == 0 and ops._swiglu_groups(2048) == 0
    # the product that adds to the residual stream itself: not beyond eight rows against a large
    # weight, nor where its blocks of 16 columns fill the chip badly
    shape = lambda N, K: torch.empty(N, K, device="meta")
    pays = ops.linear_residual_pays
    assert pays(8, shape(4096, 14336)) and not pays(9, shape(4096, 14336)) and pays(16, shape(4096, 4096))
    assert not pays(1, shape(5120, 13824)) and pays(16, shape(5120, 5120)) and pays(16, shape(3072, 8192))
    assert pays(8, shape(8192, 8192)) and not pays(16, shape(8192, 8192)) and pays(16, shape(2048, 8192))


def test_library_gemm_with_a_tuned_kernel(ops, tmp_path):
    """With tuning on, a product of more than 64 rows times the library's kernels once for its row
    bucket, keeps the choice in a file, and gives the same result (to bfloat16 rounding) as before."""
    M, N, K = 96, 320, 256
    x = rnd(M, K, dtype=torch.bfloat16, seed=80)
    w = rnd(N, K, dtype=torch.bfloat16, seed=81, scale=0.05)
    ref = x.double() @ w.double().t()
    plain = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(x, w, plain)
    file = tmp_path / "tuned.txt"
    before = ops.gemm_tuned_shapes()
    try:
        ops.set_gemm_tuning(True, str(file))
        out = torch.empty(M + 3, N, dtype=torch.bfloat16, device=DEV)          # other row counts of the bucket (81..96)
        for rows in (M - 3, M, 85):
            ops.linear(torch.cat([x, x[:3]])[:rows], w, out[:rows])
            assert torch.allclose(out[:min(rows, M)].double(), ref[:min(rows, M)], **tol(torch.bfloat16))
        assert ops.gemm_tuned_shapes() == before + 1                             # one bucket, tuned once
        lines = file.read_text().split("\n")
        assert len([l for l in lines if l.strip()]) == 1 and lines[0].split()[:4] == ["96", str(N), str(K), "0"]
    finally:
        ops.set_gemm_tuning(False)
    assert torch.allclose(plain.double(), ref, **tol(torch.bfloat16))


def test_library_gemm_asks_for_a_kernel_once_a_row_bucket(ops):
    """Prompt portions of changing length: the library is asked to choose a kernel once for a
    (row bucket, N, K), not once for every row count, and every row count gives the right product."""
    N, K = 448, 352
    w = rnd(N, K, dtype=torch.bfloat16, seed=83, scale=0.05)
    x = rnd(1100, K, dtype=torch.bfloat16, seed=82)
    ref = x.double() @ w.double().t()
    _, asked0 = ops.gemm_library_stats()
    rows = [129, 200, 131, 255, 256, 300, 511, 257, 600, 1000, 1024, 513, 130, 1100]      # buckets 144, 208, 256, 320, 512, 288, 640, 1024, 1152
    for M in rows:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops.linear(x[:M], w, out)
        assert torch.allclose(out.double(), ref[:M], **tol(torch.bfloat16)), M
    plans, asked = ops.gemm_library_stats()
    assert asked - asked0 <= 9 + 2, (asked0, asked)      # one question a bucket (one more where a bucket's kernel refuses a row count)
    assert plans >= len(set(rows))


def test_library_gemm_does_not_depend_on_what_was_served_before(ops):
    """Which of the library's kernels a row count gets depends on its bucket and on itself, not on
    the row counts that came earlier: the same product has the same bits whether a shorter or a
    longer portion of its bucket was served first."""
    N, K = 704, 480
    w = rnd(N, K, dtype=torch.bfloat16, seed=85, scale=0.05)
    x = rnd(512, K, dtype=torch.bfloat16, seed=84)
    got = {}
    for order in ((130, 250, 400, 512), (512, 400, 250, 130), (250, 512, 130, 400)):
        ops.gemm_library_reset()
        for M in order:
            out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            ops.linear(x[:M], w, out)
            got.setdefault(M, []).append(out)
    ref = x.double() @ w.double().t()
    for M, outs in got.items():
        assert torch.allclose(outs[0].double(), ref[:M], **tol(torch.bfloat16))
        assert all(torch.equal(outs[0], o) for o in outs[1:]), M


def test_linear_identity_and_strided_output(ops):
    # identity weight returns the input; a strided output view leaves its padding untouched
    # (crates/infer-backend-cpu/src/lib.rs:1330-1352)
    x = rnd(5, 48, seed=10)
    eye = torch.eye(48, device=DEV)
    buf = torch.full((5, 64), 7.0, device=DEV)
    ops.linear(x, eye, buf[:, :48])
    assert torch.equal(buf[:, :48], x) and torch.all(buf[:, 48:] == 7.0)


def test_linear_rows_do_not_depend_on_the_batch(ops):
    # the exact path: a row's result is the same bits whatever else is in the batch
    x = rnd(70, 136, seed=11)
    w = rnd(257, 136, seed=12)
    full = torch.empty(70, 257, device=DEV)
    ops.linear(x, w, full)
    one = torch.empty(1, 257, device=DEV)
    for r in (0, 33, 69):
        ops.linear(x[r:r + 1], w, one)
        # one row goes to the few-row kernel, 70 to the tiled one: both keep 64-bit sums, so the 32-bit
        # results agree to the last bit but for a sum that lies on a rounding boundary to 1e-16
        assert torch.equal(one[0], full[r])
    # the few-row kernel alone: 1, 5, 8, 13 and 16 rows
    x2, w2 = rnd(16, 1352, seed=13), rnd(1001, 1352, seed=14)
    all16 = torch.empty(16, 1001, device=DEV)
    ops.linear(x2, w2, all16)
    ref = x2.double() @ w2.double().t()
    assert torch.allclose(all16.double(), ref, rtol=0, atol=6e-8 * ref.abs().max().item())    # half a unit of the last place
    for rows in ([3], [0, 1, 2, 3, 4], list(range(4, 12)), list(range(13)), list(range(15, -1, -1))):
        sub = torch.empty(len(rows), 1001, device=DEV)
        ops.linear(x2[rows].contiguous(), w2, sub)
        assert torch.equal(sub, all16[rows])
    # 17..64 rows: the same kernel, 16 rows a pass
    x3 = rnd(64, 1352, seed=15)
    x3[20] = x2[3]
    for M in (17, 37, 64):
        out = torch.full((M, 1001), float("nan"), device=DEV)
        ops.linear(x3[:M].contiguous(), w2, out)
        ref = x3[:M].double() @ w2.double().t()
        assert torch.allclose(out.double(), ref, rtol=0, atol=6e-8 * ref.abs().max().item())
        if M > 20:
            assert torch.equal(out[20], all16[3])


def _paged_setup(dtype, B, H, Hkv, hd, page, q_lens, starts, seed=0, num_pages=128, shuffle=True):
    """A cache with random pages for each request, the step's q/k/v, and contiguous copies."""
    g = torch.Generator().manual_seed(seed)
    max_blocks = max(80, max(s + q for s, q in zip(starts, q_lens)) // page + 2)
    perm = torch.randperm(num_pages, generator=g).tolist() if shuffle else list(range(num_pages))
    table = torch.full((B, max_blocks), -1, dtype=torch.int32)
    kv_lens = [s + q for s, q in zip(starts, q_lens)]
    used = 0
    for b in range(B):
        n = (kv_lens[b] + page - 1) // page
        table[b, :n] = torch.tensor(perm[used:used + n], dtype=torch.int32)
        used += n
    T = sum(q_lens)
    positions, rows = [], []
    for b in range(B):
        positions += list(range(starts[b], kv_lens[b]))
        rows += [b] * q_lens[b]
    qkv_dim = (H + 2 * Hkv) * hd
    qkv = (torch.randn(T, qkv_dim, generator=g)).to(dtype).to(DEV)
    # pages are never cleared in the engine: what was not written may hold anything
    kc = torch.full((num_pages, Hkv, page, hd), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((num_pages, Hkv, hd, page), float("nan"), dtype=dtype, device=DEV)
    # history: random keys/values at positions [0, start)
    hist_k = [torch.randn(kv_lens[b], Hkv, hd, generator=g).to(dtype) for b in range(B)]
    hist_v = [torch.randn(kv_lens[b], Hkv, hd, generator=g).to(dtype) for b in range(B)]
    for b in range(B):
        for lo in range(0, starts[b], page):
            hi = min(starts[b], lo + page)
            blk = int(table[b, lo // page])
            kc[blk, :, :hi - lo] = hist_k[b][lo:hi].permute(1, 0, 2).to(DEV)
            vc[blk, :, :, :hi - lo] = hist_v[b][lo:hi].permute(1, 2, 0).to(DEV)
    ctx = SimpleNamespace(
        num_tokens=T, num_rows=B,
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
        row_of_token=torch.tensor(rows, dtype=torch.int32, device=DEV),
        kv_lens=torch.tensor(kv_lens, dtype=torch.int32, device=DEV),
        q_start=torch.tensor(starts, dtype=torch.int32, device=DEV),
        cu_q=torch.tensor(np.concatenate([[0], np.cumsum(q_lens)]), dtype=torch.int32, device=DEV),
        max_q_len=max(q_lens), max_kv_len=max(kv_lens), decode_only=max(q_lens) == 1,
        host_q_lens=q_lens, host_q_start=starts, host_kv_lens=kv_lens, workspace=Workspace(DEV))
    # as the engine's steps do: the tokens of the rows of one token, then -1
    singles = [int(t) for t, q in zip(np.concatenate([[0], np.cumsum(q_lens)])[:-1], q_lens) if q == 1]
    ctx.num_single = len(singles)
    ctx.single_tokens = torch.tensor(singles + [-1] * (B - len(singles)), dtype=torch.int32, device=DEV)
    longer = [b for b, q in enumerate(q_lens) if q > 1]
    ctx.num_portion = len(longer)
    ctx.portion_rows = torch.tensor(longer + [-1] * (B - len(longer)), dtype=torch.int32, device=DEV)
    return qkv, kc, vc, table.to(DEV), ctx, hist_k, hist_v


ATT_CASES = [
    # B, H, Hkv, hd, page, q_lens, starts
    (1, 4, 2, 16, 16, [33], [0]),
    (3, 5, 1, 32, 8, [1, 7, 20], [40, 0, 13]),
    (2, 6, 3, 48, 16, [1, 1], [15, 16]),
    (2, 8, 2, 64, 16, [17, 1], [3, 99]),
    (1, 3, 3, 80, 4, [9], [22]),
    (2, 4, 1, 128, 16, [40, 2], [0, 130]),
    (1, 2, 2, 256, 16, [5], [11]),
    # single tokens at sizes the split-key matrix-core kernel takes (head 64 / 128, page 16 / 32)
    (3, 8, 2, 64, 16, [1, 1, 1], [0, 127, 300]),
    (2, 12, 4, 128, 16, [1, 1], [128, 515]),
    (2, 16, 1, 64, 32, [1, 1], [255, 256]),
    (4, 4, 4, 128, 16, [1, 1, 1, 1], [15, 16, 17, 1000]),
    # portions of prompts at sizes the tiled matrix-core kernel takes, alone and beside single tokens
    (2, 8, 2, 64, 16, [70, 33], [0, 50]),
    (3, 12, 4, 128, 16, [17, 1, 40], [100, 200, 0]),
    (1, 16, 1, 64, 32, [100], [29]),
    (2, 6, 2, 128, 16, [5, 64], [250, 3]),
    (3, 3, 3, 64, 16, [2, 16, 31], [0, 16, 1]),
    # portions whose blocks share keys and values through LDS and take the steps below the diagonal
    # two at a time (64 queries with 64 keys or more before them): one, three and no such double steps
    (2, 8, 2, 64, 16, [200, 130], [70, 0]),
    (2, 4, 2, 128, 16, [150, 64], [300, 5]),
    # head size 128 with so many tiles and heads that the tiled kernel runs two waves per SIMD
    (2, 128, 16, 128, 16, [1100, 100], [0, 37]),
    # single tokens over contexts so long that a wave of the split-key kernel takes several chunks
    (8, 8, 4, 64, 16, [1] * 8, [4500, 4099, 64, 1, 3000, 4351, 2047, 4496]),
    (8, 8, 4, 128, 32, [1] * 8, [4200, 63, 4159, 0, 1024, 4223, 17, 4100]),
    # single tokens of so many requests and kv heads that one block takes all chunks of a (token, kv head)
    (16, 16, 8, 64, 16, [1] * 16, [700, 0, 63, 64, 1023, 1024, 2500, 15, 16, 17, 300, 1, 2, 999, 48, 47]),
    (16, 24, 8, 128, 16, [1] * 16, [2047, 5, 1300, 128, 127, 64, 1000, 0, 1, 15, 16, 31, 32, 500, 63, 65]),
    (32, 20, 4, 64, 32, [1] * 32, [100, 1, 0, 500, 31, 32, 33, 2000, 64, 65, 1500, 7] + [(53 * i) % 400 for i in range(20)]),
    # ... and so many pairs that it does so whatever the number of chunks (here 9 and more a wave)
    (32, 16, 16, 64, 16, [1] * 32, [8300] + [(37 * i) % 200 for i in range(1, 32)]),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATT_CASES)
@pytest.mark.parametrize("window", [0, 11])
def test_rope_write_and_attention(ops, dtype, case, window):
    """rope_kv_write then paged_attention equal rotation + causal attention computed plainly
    over each request's whole sequence."""
    _check_rope_write_and_attention(ops, dtype, case, window)


def test_attention_of_a_long_portion_at_head_size_64(ops):
    """So many tiles and heads (128 over 32 kv heads, 2,100 tokens) that the tiled kernel takes
    four heads per wave with the keys and values shared through LDS and two waves per SIMD;
    three kv heads' groups are compared with the plain computation."""
    _check_rope_write_and_attention(ops, torch.bfloat16, (1, 128, 32, 64, 16, [2100], [0]), 0, kv_heads=(0, 13, 31))


RANGE_CASES = [
    # B, H, Hkv, hd, page, q_lens, starts; ranges of keys asked for (0: the kernel's own choice)
    ((1, 8, 2, 128, 16, [16], [2040]), 0),                       # a short portion behind many keys: six ranges of 384
    ((1, 8, 2, 128, 16, [16], [2040]), 16),                      # ranges of 129 -> 256 keys
    ((3, 8, 2, 64, 16, [200, 1, 70], [700, 300, 0]), 0),         # beside a single token; the third row ends inside the first range
    ((3, 8, 2, 64, 16, [200, 1, 70], [700, 300, 0]), 3),
    ((2, 4, 1, 128, 16, [130, 64], [1000, 129]), 5),             # a tile of queries that begins in one range and ends in the next
    ((2, 4, 1, 128, 16, [130, 64], [1000, 129]), 2),
    ((1, 8, 8, 64, 16, [1000], [0]), 4),                         # from the first token: ranges that the early tiles never reach
    ((2, 6, 2, 128, 16, [3, 259], [381, 250]), 2),               # a range's edge (256) inside a portion, odd lengths
]


@pytest.mark.parametrize("case,ranges", RANGE_CASES)
def test_attention_of_a_portion_with_the_keys_divided_between_blocks(ops, monkeypatch, case, ranges):
    """Short portions behind many cached keys: blocks take ranges of keys and a second kernel
    puts a query's ranges together; the result is the plain attention whatever the ranges."""
    import ctypes
    B, H, Hkv, hd, page, q_lens, starts = case
    lib = ops._lib()
    lib.ri_attention_prefill_workspace.restype = ctypes.c_size_t
    # the case does divide the keys (else it would test nothing new)
    portions = [(s, q) for s, q in zip(starts, q_lens) if q > 1]
    assert lib.ri_attention_prefill_workspace(H, Hkv, hd, page, 0, sum(q_lens), max(s for s, _ in portions),
                                              max(s + q for s, q in portions), ranges) > 0
    monkeypatch.setattr(ops, "PREFILL_KEY_RANGES", ranges)
    _check_rope_write_and_attention(ops, torch.bfloat16, case, 0)


@pytest.mark.parametrize("blocks", [2, 3, 8])
@pytest.mark.parametrize("window", [0, 700])
@pytest.mark.parametrize("case", [
    (8, 8, 4, 64, 16, [1] * 8, [4500, 4099, 64, 1, 3000, 4351, 2047, 4496]),
    (8, 8, 4, 128, 32, [1] * 8, [4200, 63, 4159, 0, 1024, 4223, 17, 4100]),
    (16, 24, 8, 128, 16, [1] * 16, [2047, 5, 1300, 128, 127, 64, 1000, 0, 1, 15, 16, 31, 32, 500, 63, 65]),
    (3, 12, 4, 128, 16, [17, 1, 40], [100, 1200, 0]),            # beside prompt portions
])
def test_single_token_attention_with_several_blocks_a_pair(ops, monkeypatch, case, window, blocks):
    """Single tokens whose (kv head, token) pairs are too few to fill the chip with a block each:
    several blocks of several waves a pair, each leaving one partial result.  Rows shorter than a
    block's first chunk leave that block's slot unwritten, and with a window a block may find every
    chunk of its own passed; the result is the plain attention all the same."""
    monkeypatch.setattr(ops, "DECODE_PAIR_BLOCKS", blocks)
    _check_rope_write_and_attention(ops, torch.bfloat16, case, window)


def _check_rope_write_and_attention(ops, dtype, case, window, kv_heads=None):
    B, H, Hkv, hd, page, q_lens, starts = case
    need = sum((s + q + page - 1) // page for s, q in zip(starts, q_lens))
    qkv, kc, vc, table, ctx, hist_k, hist_v = _paged_setup(dtype, B, H, Hkv, hd, page, q_lens, starts, seed=hd + B,
                                                           num_pages=max(128, need + 16))
    freqs = plain_llama.rope_frequencies(hd, 10000.0, None)
    maxpos = max(1100, max(starts) + max(q_lens) + 1)
    ang = np.arange(maxpos)[:, None] * freqs[None, :]
    cos = torch.tensor(np.cos(ang), dtype=torch.float32, device=DEV)
    sin = torch.tensor(np.sin(ang), dtype=torch.float32, device=DEV)
    qkv0 = qkv.clone()
    ops.rope_kv_write(qkv, H, Hkv, hd, (cos, sin, hd), ctx.positions, ctx.row_of_token, kc, vc, table, page)
    out = torch.empty(ctx.num_tokens, H * hd, dtype=dtype, device=DEV)
    scale = 1.0 / math.sqrt(hd)
    ops.paged_attention(qkv, out, H, Hkv, hd, kc, vc, table, page, ctx, scale, window)
    if 1 in q_lens and max(q_lens) > 1:
        # single tokens beside portions: the same without the lists of them (a context that brings none)
        ctx.single_tokens = ctx.portion_rows = None
        again = torch.empty_like(out)
        ops.paged_attention(qkv, again, H, Hkv, hd, kc, vc, table, page, ctx, scale, window)
        assert torch.equal(out, again)
    t0 = 0
    for b in range(B):
        q_len, s = q_lens[b], starts[b]
        rows = qkv0[t0:t0 + q_len].double().cpu().numpy()
        q = rows[:, :H * hd].reshape(q_len, H, hd)
        k_new = rows[:, H * hd:(H + Hkv) * hd].reshape(q_len, Hkv, hd)
        v_new = rows[:, (H + Hkv) * hd:].reshape(q_len, Hkv, hd)
        pos = np.arange(s, s + q_len)
        q_rot = plain_llama.rope(q, pos, freqs)
        k_rot = plain_llama.rope(k_new, pos, freqs)
        if dtype == torch.bfloat16:                  # the cache holds rounded keys; q is rounded in place
            k_rot = torch.tensor(k_rot).to(torch.bfloat16).double().numpy()
            q_rot = torch.tensor(q_rot).to(torch.bfloat16).double().numpy()
        k_all = np.concatenate([hist_k[b][:s].double().numpy(), k_rot])
        v_all = np.concatenate([hist_v[b][:s].double().numpy(), v_new])
        # whole-sequence attention with dummy queries for the cached part
        q_all = np.concatenate([np.zeros((s, H, hd)), q_rot])
        got = out[t0:t0 + q_len].double().cpu().numpy().reshape(q_len, H, hd)
        lim = 1e-5 if dtype == torch.float32 else 2e-2
        if kv_heads is None:
            ref = plain_llama.attention(q_all, k_all, v_all, scale, window or None)[s:]
            assert np.max(np.abs(got - ref)) < lim, (case, window, np.max(np.abs(got - ref)))
        else:
            G = H // Hkv
            for g in kv_heads:                       # a kv head with its group of query heads
                ref = plain_llama.attention(q_all[:, g * G:(g + 1) * G], k_all[:, g:g + 1], v_all[:, g:g + 1], scale, window or None)[s:]
                err = np.max(np.abs(got[:, g * G:(g + 1) * G] - ref))
                assert err < lim, (case, window, g, err)
        # q was rotated in place
        got_q = qkv[t0:t0 + q_len, :H * hd].double().cpu().numpy().reshape(q_len, H, hd)
        assert np.max(np.abs(got_q - q_rot)) < (1e-5 if dtype == torch.float32 else 1e-6 + 2e-2)
        t0 += q_len


@pytest.mark.parametrize("B,H,Hkv,hd,page,K", [(1, 4, 2, 16, 16, 64), (5, 5, 1, 32, 8, 160), (8, 32, 8, 64, 16, 2048),
                                                (33, 6, 2, 128, 16, 96), (64, 3, 3, 48, 16, 224),
                                                # 33..64 tokens: the kernel that shares the activations through LDS
                                                (40, 32, 8, 128, 16, 4096), (64, 32, 8, 64, 16, 2048), (49, 12, 4, 128, 32, 544),
                                                (32, 8, 2, 64, 16, 512)])
def test_fused_projection_rotation_and_cache_write(ops, monkeypatch, B, H, Hkv, hd, page, K):
    """The one-kernel form for single tokens equals projection, then rope_kv_write.  (33 tokens and
    more: the kernel with the activations in LDS, here whatever the number of columns.)"""
    monkeypatch.setattr(ops, "QKV_ROPE_LDS_MIN_COLUMNS", 0)
    _check_fused_projection(ops, B, H, Hkv, hd, page, K)


@pytest.mark.parametrize("B,H,Hkv,hd,page,K", [
    (17, 8, 2, 64, 16, 512), (20, 5, 5, 48, 8, 224), (32, 32, 8, 128, 16, 1024),     # blocks of 32 columns
    (24, 96, 24, 128, 16, 128),                                                      # 18432 columns: blocks of 64
    (64, 48, 12, 128, 16, 256), (40, 40, 40, 80, 16, 96)])                           # more than 32 rows: 64 from 8208 columns on
def test_fused_projection_through_lds_from_17_tokens_and_in_wider_blocks(ops, monkeypatch, B, H, Hkv, hd, page, K):
    """The kernel with the activations in LDS, as it is taken for large weights from 17 tokens on,
    and with blocks of 64 columns where those of 32 would not all run at once."""
    monkeypatch.setattr(ops, "QKV_ROPE_LDS_MIN_COLUMNS", 0)
    monkeypatch.setattr(ops, "QKV_ROPE_LDS_LARGE", 0)
    lib, taken = ops._lib(), []
    entry = lib.ri_gemm_rows_qkv_rope
    monkeypatch.setattr(lib, "ri_gemm_rows_qkv_rope", lambda *a: taken.append(1) or entry(*a))
    _check_fused_projection(ops, B, H, Hkv, hd, page, K)
    assert taken


def _check_fused_projection(ops, B, H, Hkv, hd, page, K):
    q_lens, starts = [1] * B, [(7 * i + 3) % 60 for i in range(B)]
    qkv, kc, vc, table, ctx, _, _ = _paged_setup(torch.bfloat16, B, H, Hkv, hd, page, q_lens, starts, seed=K, num_pages=640)
    ctx.row_of_token[B // 2] = -1 if B > 2 else ctx.row_of_token[B // 2]      # a padding row touches nothing
    x = rnd(B, K, dtype=torch.bfloat16, seed=50)
    w = rnd((H + 2 * Hkv) * hd, K, dtype=torch.bfloat16, seed=51, scale=0.05)
    freqs = plain_llama.rope_frequencies(hd, 10000.0, None)
    ang = np.arange(128)[:, None] * freqs[None, :]
    rotary = (torch.tensor(np.cos(ang), dtype=torch.float32, device=DEV), torch.tensor(np.sin(ang), dtype=torch.float32, device=DEV), hd)
    wf = ops.qkv_rope_weight(w, hd)
    assert wf is not None
    kc1, vc1, kc2, vc2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
    ref = torch.zeros_like(qkv)
    ops.linear(x, w, ref)
    ops.rope_kv_write(ref, H, Hkv, hd, rotary, ctx.positions, ctx.row_of_token, kc1, vc1, table, page)
    got = torch.zeros_like(qkv)
    assert ops.qkv_rope_fused(x, wf, got, H, Hkv, hd, rotary, ctx.positions, ctx.row_of_token, kc2, vc2, table, page)
    live = (ctx.row_of_token >= 0).cpu()
    nn = torch.nan_to_num
    # the separate kernels round the projection to bfloat16 before rotating; the fused one does not:
    # two roundings of values up to the largest sum against one
    big = max(1.0, ref[live].float().abs().max().item() / 2)
    assert torch.allclose(got[live, :H * hd].float(), ref[live, :H * hd].float(), atol=2e-2 * big, rtol=2e-2)
    assert torch.allclose(nn(kc2).float(), nn(kc1).float(), atol=2e-2 * big, rtol=2e-2)
    assert torch.allclose(nn(vc2).float(), nn(vc1).float(), atol=1e-2, rtol=1e-2)
    # and against the product in 64-bit, rotated: one rounding to bfloat16
    full = x.double() @ w.double().t()
    q = full[:, :H * hd].view(B, H, hd)
    c, sn = rotary[0][ctx.positions.long()].double()[:, None, :], rotary[1][ctx.positions.long()].double()[:, None, :]
    a, b = q[..., :hd // 2], q[..., hd // 2:]
    want = torch.cat([a * c - b * sn, a * sn + b * c], -1).reshape(B, H * hd)
    assert torch.allclose(got[live, :H * hd].double(), want[live], atol=1e-3, rtol=2.0 ** -8)
    assert torch.equal(torch.isnan(kc2), torch.isnan(kc1)) and torch.equal(torch.isnan(vc2), torch.isnan(vc1))
    # against 64-bit arithmetic the fused form is the closer one
    x64, w64 = x.double().cpu().numpy(), w.double().cpu().numpy()
    qf = (x64 @ w64.T)[:, :H * hd].reshape(B, H, hd)
    for b in np.nonzero(live.numpy())[0][:4]:
        want = plain_llama.rope(qf[b:b + 1], np.array([starts[b]]), freqs)[0].reshape(-1)
        # one bfloat16 rounding: half a unit in the 8th bit of each value
        assert np.all(np.abs(got[b, :H * hd].double().cpu().numpy() - want) <= 2.0 ** -8 * np.maximum(1.0, np.abs(want)))


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,I,eps", [(1, 64, 64, 176, 1e-5), (5, 384, 1056, 416, 1e-6), (8, 2048, 8192, 1024, 1e-5),
                                         (16, 4096, 14336, 512, 1e-5), (13, 160, 416, 48, 1e-5), (2, 2304, 2304, 1184, 1e-6)])
def test_a_norm_done_by_the_products_around_it(ops, wdtype, M, N, K, I, eps):
    """Few rows: the product before a norm adds its sums to the residual stream and leaves
    x * w and partial sums of x^2; the products after it (plain, SwiGLU) multiply their sums by
    rsqrt(mean(x^2) + eps).  Against 64-bit arithmetic, and against the norm's own kernel."""
    act = rnd(M, K, dtype=torch.bfloat16, seed=60)
    w = rnd(N, K, dtype=torch.bfloat16, seed=61, scale=0.05)
    wt = ops.tile_weight(w)
    x = rnd(M, N, seed=62, scale=2.0)
    wn = (1.0 + rnd(N, seed=63, scale=0.1)).to(wdtype)
    assert ops.linear_residual_ok(M, w, wt, wn) and not ops.linear_residual_ok(ops.DEFERRED_NORM_MAX_ROWS + 1, w, wt, wn)
    ws = Workspace(DEV)
    x0 = x.clone()
    a, ssq = ops.linear_residual(act, w, wt, x, wn, ws, "t")
    want_x = x0.double() + act.double() @ w.double().t()
    assert a.dtype == torch.bfloat16 and tuple(a.shape) == (M, N) and ssq.shape[0] == M
    assert torch.allclose(x.double(), want_x, rtol=0, atol=2e-5 * max(1.0, want_x.abs().max().item()))
    assert torch.equal(a, (x * wn.float()).to(torch.bfloat16))                    # rounded once, from the 32-bit sum
    assert torch.allclose(ssq.double().sum(1), (x.double() ** 2).sum(1), rtol=1e-5)
    # the products behind the norm
    n64 = want_x * torch.rsqrt((want_x ** 2).mean(-1, keepdim=True) + eps) * wn.double()
    w2 = rnd(2 * I, N, dtype=torch.bfloat16, seed=64, scale=0.05)
    w2t = ops.tile_weight(w2)
    out = torch.empty(M, I, dtype=torch.bfloat16, device=DEV)
    ops.linear_swiglu(a, w2, out, None, w2t, scale=(ssq, eps))
    g, u = n64 @ w2[:I].double().t(), n64 @ w2[I:].double().t()
    ref = g / (1 + torch.exp(-g)) * u
    assert torch.allclose(out.double(), ref, rtol=1.6e-2, atol=1.6e-2 * max(1.0, ref.abs().max().item()) / 4)
    for odt, tiled in ((torch.float32, w2t), (torch.bfloat16, None)):
        lin = torch.empty(M, 2 * I, dtype=odt, device=DEV)
        ops.linear(a, w2, lin, tiled, scale=(ssq, eps))
        ref = n64 @ w2.double().t()
        assert torch.allclose(lin.double(), ref, rtol=1.6e-2, atol=1.6e-2 * max(1.0, ref.abs().max().item()) / 4)
    # the same through the norm's own kernel: rows rounded after the factor instead of before it
    normed = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    xr = x0.clone()
    delta = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops.linear(act, w, delta, wt)
    ops.add_rmsnorm(xr, delta, wn, eps, normed)
    assert torch.allclose(xr, x, rtol=0, atol=1e-5 * max(1.0, x.abs().max().item()))
    lin2 = torch.empty(M, 2 * I, dtype=torch.float32, device=DEV)
    ops.linear(normed, w2, lin2, w2t)
    lin = torch.empty(M, 2 * I, dtype=torch.float32, device=DEV)
    ops.linear(a, w2, lin, w2t, scale=(ssq, eps))
    assert torch.allclose(lin, lin2, rtol=2e-2, atol=2e-2 * max(1.0, lin2.abs().max().item()) / 4)
    # more rows than the few-row kernel takes: the factors have no product to go with
    big = rnd(80, N, dtype=torch.bfloat16, seed=65)
    with pytest.raises(ops.KernelError, match="deferred norm"):
        ops.linear(big, w2, torch.empty(80, 2 * I, dtype=torch.float32, device=DEV), w2t,
                   scale=(torch.ones(80, 4, device=DEV), eps))


@pytest.mark.parametrize("B,H,Hkv,hd,K", [(1, 4, 2, 64, 256), (2, 6, 2, 128, 384), (8, 32, 8, 64, 2048), (16, 3, 3, 48, 96),
                                          (13, 5, 1, 32, 160)])
def test_fused_projection_finishes_a_deferred_norm(ops, B, H, Hkv, hd, K):
    """Single tokens: the fused projection, rotation and cache write on rows x * w with the factor
    rsqrt(mean(x^2) + eps) applied to its sums equals the same kernel on rows normalised before."""
    page, eps = 16, 1e-5
    q_lens, starts = [1] * B, [(11 * i + 5) % 60 for i in range(B)]
    qkv, kc, vc, table, ctx, _, _ = _paged_setup(torch.bfloat16, B, H, Hkv, hd, page, q_lens, starts, seed=K, num_pages=64)
    x = rnd(B, K, seed=70, scale=2.0)
    wn = (1.0 + rnd(K, seed=72, scale=0.1)).to(torch.bfloat16)
    w = rnd((H + 2 * Hkv) * hd, K, dtype=torch.bfloat16, seed=73, scale=0.05)
    freqs = plain_llama.rope_frequencies(hd, 10000.0, None)
    ang = np.arange(128)[:, None] * freqs[None, :]
    rotary = (torch.tensor(np.cos(ang), dtype=torch.float32, device=DEV), torch.tensor(np.sin(ang), dtype=torch.float32, device=DEV), hd)
    wf = ops.qkv_rope_weight(w, hd)
    kc1, vc1, kc2, vc2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
    normed = torch.empty(B, K, dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm(x.clone(), None, wn, eps, normed)
    ref = torch.zeros_like(qkv)
    assert ops.qkv_rope_fused(normed, wf, ref, H, Hkv, hd, rotary, ctx.positions, ctx.row_of_token, kc1, vc1, table, page)
    # the deferred form: rows x * w, sums of squares in 7 uneven parts
    a = (x * wn.float()).to(torch.bfloat16)
    sq = x * x
    cuts = [0, 1, K // 7, K // 3, K // 2, K - 9, K - 1, K]
    ssq = torch.stack([sq[:, lo:hi].sum(1) for lo, hi in zip(cuts[:-1], cuts[1:])], dim=1).contiguous()
    got = torch.zeros_like(qkv)
    assert ops.qkv_rope_fused(a, wf, got, H, Hkv, hd, rotary, ctx.positions, ctx.row_of_token, kc2, vc2, table, page,
                              scale=(ssq, eps))
    nn = torch.nan_to_num
    assert torch.allclose(got[:, :H * hd].float(), ref[:, :H * hd].float(), atol=3e-2, rtol=3e-2)
    assert torch.allclose(nn(kc2).float(), nn(kc1).float(), atol=3e-2, rtol=3e-2)
    assert torch.allclose(nn(vc2).float(), nn(vc1).float(), atol=3e-2, rtol=3e-2)
    assert torch.equal(torch.isnan(kc2), torch.isnan(kc1)) and torch.equal(torch.isnan(vc2), torch.isnan(vc1))
    # against 64-bit arithmetic
    x64 = x.double()
    n = x64 * torch.rsqrt((x64 * x64).mean(-1, keepdim=True) + eps) * wn.double()
    qf = (n.cpu().numpy() @ w.double().cpu().numpy().T)[:, :H * hd].reshape(B, H, hd)
    for b in range(B):
        want = plain_llama.rope(qf[b:b + 1], np.array([starts[b]]), freqs)[0].reshape(-1)
        assert np.all(np.abs(got[b, :H * hd].double().cpu().numpy() - want) <= 1.6e-2 * np.maximum(1.0, np.abs(want)))


@pytest.mark.parametrize("q_len", [1, 5, 40])
def test_attention_finds_a_far_key(ops, q_len):
    """One key among hundreds is made to stand out for the last query: the output must be that
    key's value (a fault at a page edge, in the split of long histories or in a tile's key order
    would miss it).  q_len 1 takes the split-key kernel, longer portions the tiled one."""
    B, H, Hkv, hd, page = 1, 4, 2, 64, 16
    start = 512 - (q_len - 1)
    for far in (0, 3, 4, 7, 8, 15, 16, 31, 32, 127, 128, 255, 256, 300, 383, 384, 511):
        qkv, kc, vc, table, ctx, hk, hv = _paged_setup(torch.bfloat16, B, H, Hkv, hd, page, [q_len], [start], seed=far)
        ops.rope_kv_write(qkv, H, Hkv, hd, None, ctx.positions, ctx.row_of_token, kc, vc, table, page)
        blk = int(table[0, far // page])
        q = qkv[q_len - 1, :H * hd].view(H, hd)
        for g in range(Hkv):
            kc[blk, g, far % page] = (q[g * (H // Hkv)] * 4.0)
        out = torch.empty(q_len, H * hd, dtype=torch.bfloat16, device=DEV)
        ops.paged_attention(qkv, out, H, Hkv, hd, kc, vc, table, page, ctx, 1.0, 0)
        for g in range(Hkv):
            h = g * (H // Hkv)
            assert torch.allclose(out[q_len - 1, h * hd:(h + 1) * hd].float(), vc[blk, g, :, far % page].float(), atol=2e-2), far


@pytest.mark.parametrize("H,Hkv,hd,page,window", [(8, 2, 64, 16, 0), (6, 1, 128, 16, 0), (5, 5, 48, 8, 70), (16, 2, 80, 16, 0)])
def test_exact_attention_of_a_portion_does_not_depend_on_the_cut(ops, H, Hkv, hd, page, window):
    """The tiled kernel of the 32-bit path: a token's output is the same bits whether its portion
    is the whole prompt's tail or cut in two (key blocks are aligned to absolute positions, a
    row's sums go in a fixed order), it agrees with the generic kernel to rounding, and it finds
    one far key that is made to stand out."""
    from types import SimpleNamespace
    start, n = 200, 37
    qkv, kc, vc, table, ctx, hk, hv = _paged_setup(torch.float32, 1, H, Hkv, hd, page, [n], [start], seed=hd)
    ops.rope_kv_write(qkv, H, Hkv, hd, None, ctx.positions, ctx.row_of_token, kc, vc, table, page)
    scale = 1.0 / math.sqrt(hd)

    def portion(lo, hi):
        c = SimpleNamespace(num_tokens=hi - lo, num_rows=1, positions=ctx.positions[lo:hi].contiguous(),
                            row_of_token=ctx.row_of_token[lo:hi].contiguous(),
                            kv_lens=torch.tensor([start + hi], dtype=torch.int32, device=DEV),
                            q_start=torch.tensor([start + lo], dtype=torch.int32, device=DEV),
                            cu_q=torch.tensor([0, hi - lo], dtype=torch.int32, device=DEV),
                            max_q_len=hi - lo, max_kv_len=start + hi, decode_only=False,
                            host_q_lens=[hi - lo], host_q_start=[start + lo], host_kv_lens=[start + hi], workspace=ctx.workspace)
        o = torch.full((hi - lo, H * hd), float("nan"), device=DEV)
        ops.paged_attention(qkv[lo:hi], o, H, Hkv, hd, kc, vc, table, page, c, scale, window)
        return o

    if window:
        # pages that lie below the window of the portion's first token have been given back
        table[0, :(start + 1 - window) // page] = -1
    whole = portion(0, n)
    assert torch.equal(torch.cat([portion(0, 20), portion(20, n)]), whole)
    assert torch.equal(torch.cat([portion(0, 2), portion(2, 35), portion(35, n)]), whole)
    # single tokens take the split-key kernel: the same bits again, alone or several in a step
    for i in (0, 1, 19, n - 1):
        assert torch.equal(portion(i, i + 1), whole[i:i + 1]), i
    rows = [3, 30, 11]
    c = SimpleNamespace(num_tokens=3, num_rows=3, positions=ctx.positions[rows].contiguous(),
                        row_of_token=torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV),
                        kv_lens=torch.tensor([start + r + 1 for r in rows], dtype=torch.int32, device=DEV),
                        max_q_len=1, max_kv_len=start + n, decode_only=True, workspace=ctx.workspace)
    o = torch.full((3, H * hd), float("nan"), device=DEV)
    ops.paged_attention(qkv[rows].contiguous(), o, H, Hkv, hd, kc, vc, table[[0, 0, 0]].contiguous(), page, c, scale, window)
    assert torch.equal(o, whole[rows])
    generic = torch.empty_like(whole)
    lib = ops._lib()
    import ctypes
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    assert lib.ri_attention_generic(P(qkv), qkv.stride(0), P(generic), generic.stride(0), 0, P(kc), P(vc), kc.shape[0], page,
                                    H, Hkv, hd, P(table), table.shape[1], P(ctx.row_of_token), P(ctx.positions), P(ctx.kv_lens),
                                    n, ctypes.c_float(scale), window, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    assert torch.allclose(whole, generic, rtol=0, atol=2e-6)
    # a far key for the last query (inside the window where there is one)
    G = H // Hkv
    for far in (0, 63, 64, 127, 199, 200, 235):
        if window and far < start + n - window:
            continue
        blk = int(table[0, far // page])
        saved = kc[blk, :, far % page].clone()
        q = qkv[n - 1, :H * hd].view(H, hd)
        for g in range(Hkv):
            kc[blk, g, far % page] = q[g * G] * (40.0 / float(q[g * G].norm()) ** 2) / scale
        o = portion(0, n)
        for g in range(Hkv):
            assert torch.allclose(o[n - 1, g * G * hd:(g * G + 1) * hd], vc[blk, g, :, far % page], atol=1e-4), far
        kc[blk, :, far % page] = saved


def test_attention_padding_rows_touch_nothing(ops):
    qkv, kc, vc, table, ctx, _, _ = _paged_setup(torch.float32, 2, 4, 2, 16, 16, [1, 1], [5, 9])
    kc0, vc0 = kc.clone(), vc.clone()
    ctx.row_of_token = torch.tensor([0, -1], dtype=torch.int32, device=DEV)
    ops.rope_kv_write(qkv, 4, 2, 16, None, ctx.positions, ctx.row_of_token, kc, vc, table, 16)
    blk = int(table[0, 0])
    nn = torch.nan_to_num
    assert not torch.equal(nn(kc[blk]), nn(kc0[blk]))
    kc0[blk], vc0[blk] = kc[blk], vc[blk]
    assert torch.equal(nn(kc), nn(kc0)) and torch.equal(nn(vc), nn(vc0))
    out = torch.full((2, 64), 3.0, device=DEV)
    ops.paged_attention(qkv, out, 4, 2, 16, kc, vc, table, 16, ctx, 0.25, 0)
    assert torch.all(out[1] == 0)


@pytest.mark.parametrize("R,V", [(1, 50), (3, 333), (5, 128256)])
def test_argmax_lowest_index_on_ties(ops, R, V):
    logits = rnd(R, V, seed=13)
    ref = logits.argmax(-1)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.argmax(logits, out)
    assert torch.equal(out.long(), ref)
    logits[:, V // 2] = 100.0
    logits[:, V // 3] = 100.0
    ops.argmax(logits, out)
    assert torch.all(out == V // 3)


def _plain_sample(logits, temperature, top_k, top_p, min_p, u):
    order, w = plain_llama.filtered_distribution(logits, temperature, top_k, top_p, min_p)
    return plain_llama.sample_from(order, w, u), set(order.tolist())


@pytest.mark.parametrize("V", [7, 50, 1000, 32003, 140001])
def test_sample_matches_plain(ops, V):
    """Same token as the plain sorted walk for the same uniform number, under every filter.
    (32,003 tokens: four slices of the vocabulary, each with a list of its tokens ordered by bin;
    140,001: slices longer than such a list can be, the kernel reads the row instead.)"""
    rng = np.random.default_rng(V)
    cases = []
    for temperature in (0.7, 1.0, 1.5):
        for top_k, top_p, min_p in ((0, 1.0, 0.0), (5, 1.0, 0.0), (0, 0.9, 0.0), (0, 1.0, 0.05),
                                    (20, 0.8, 0.01), (1000000, 0.5, 0.0), (3, 0.3, 0.2)):
            for _ in range(6):
                cases.append((temperature, top_k, top_p, min_p, float(rng.random())))
    R = len(cases)
    logits = torch.tensor(rng.normal(0, 2.0, (R, V)), dtype=torch.float32)
    logits[::3, : min(V, 4)] = 3.0                   # ties among the largest
    dl = logits.to(DEV)
    f = lambda i, dt: torch.tensor([c[i] for c in cases], dtype=dt, device=DEV)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.sample(dl, f(0, torch.float32), f(1, torch.int32).clamp(max=2**31 - 1), f(2, torch.float32),
               f(3, torch.float32), f(4, torch.float64), out)
    got = out.tolist()
    bad = 0
    for r, (temperature, top_k, top_p, min_p, u) in enumerate(cases):
        want, kept = _plain_sample(logits[r].numpy(), temperature, top_k, top_p, min_p, u)
        assert got[r] in kept, (r, cases[r], got[r])          # never outside the kept set
        bad += got[r] != want
    assert bad <= max(1, R // 100), f"{bad} of {R} draws differ from the plain walk"


def test_sample_rows_with_many_equal_or_far_logits(ops):
    """Rows the bins of the kernel do not separate: thousands of equal logits (more than it sorts
    in one go, so the descent over key digits answers) and a peaked row whose tokens nearly all
    lie far below the largest (weight 0 in fixed point)."""
    V = 9000
    rng = np.random.default_rng(5)
    flat = np.full(V, 1.0, dtype=np.float32)
    flat[[17, 4000, 8999]] = [2.5, 2.5, 0.5]
    peaked = np.full(V, -60.0, dtype=np.float32) + rng.normal(0, 3.0, V).astype(np.float32)
    peaked[[3, 77, 5000, 8000]] = [4.0, 3.5, 3.5, 1.0]
    cases = []
    for row in (flat, peaked):
        for top_k, top_p, min_p in ((0, 1.0, 0.0), (5000, 1.0, 0.0), (0, 0.7, 0.0), (6000, 0.9, 0.0), (0, 1.0, 0.3)):
            for u in (0.0, 0.013, 0.35, 0.5, 0.77, 0.999999):
                cases.append((row, 1.0, top_k, top_p, min_p, u))
    R = len(cases)
    dl = torch.tensor(np.stack([c[0] for c in cases]), device=DEV)
    f = lambda i, dt: torch.tensor([c[i] for c in cases], dtype=dt, device=DEV)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.sample(dl, f(1, torch.float32), f(2, torch.int32), f(3, torch.float32), f(4, torch.float32),
               f(5, torch.float64), out)
    got = out.tolist()
    bad = 0
    for r, (row, temperature, top_k, top_p, min_p, u) in enumerate(cases):
        want, kept = _plain_sample(row, temperature, top_k, top_p, min_p, u)
        assert got[r] in kept, (r, cases[r][1:], got[r])
        bad += got[r] != want
    assert bad <= 1, f"{bad} of {R} draws differ from the plain walk"


def test_sample_reference_vectors(ops):
    """The reference's own sampler cases (crates/infer-worker/src/application/sampler_stack.rs:421-446):
    logits [3, 2, 1] with top_p 0.5 and draw 0.99 give token 0; top-k never leaves its set."""
    logits = torch.tensor([[3.0, 2.0, 1.0]], device=DEV)
    out = torch.empty(1, dtype=torch.int32, device=DEV)
    one = lambda v, dt: torch.tensor([v], dtype=dt, device=DEV)
    ops.sample(logits, one(1.0, torch.float32), one(0, torch.int32), one(0.5, torch.float32),
               one(0.0, torch.float32), one(0.99, torch.float64), out)
    assert out.item() == 0
    logits = torch.tensor([[0.1, 5.0, 4.9, -1.0, 4.8]], device=DEV)
    for u in np.linspace(0, 0.999999, 50):
        ops.sample(logits, one(1.0, torch.float32), one(2, torch.int32), one(1.0, torch.float32),
                   one(0.0, torch.float32), one(float(u), torch.float64), out)
        assert out.item() in (1, 2)


def test_sample_frequencies_and_greedy_rows(ops):
    """Over many draws the frequencies follow softmax(logits / T); temperature 0 rows are greedy."""
    V, R, T = 11, 20000, 0.8
    rng = np.random.default_rng(5)
    row = rng.normal(0, 1.5, V).astype(np.float32)
    logits = torch.tensor(row, device=DEV).repeat(R, 1)
    temp = torch.full((R,), T, device=DEV)
    temp[:10] = 0.0
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    u = torch.tensor(rng.random(R), dtype=torch.float64, device=DEV)
    ops.sample(logits, temp, torch.zeros(R, dtype=torch.int32, device=DEV), torch.ones(R, device=DEV),
               torch.zeros(R, device=DEV), u, out)
    got = out.cpu().numpy()
    assert np.all(got[:10] == int(np.argmax(row)))
    p = plain_llama.softmax(row.astype(np.float64) / T)
    freq = np.bincount(got[10:], minlength=V) / (R - 10)
    assert np.max(np.abs(freq - p)) < 0.015


def test_sample_log_probabilities(ops):
    """ln p of the chosen token and of the five most probable kept tokens equal the plain
    computation, for greedy rows, plain temperature, and every filter; the tokens are the same
    with and without asking for them."""
    V, rng = 3001, np.random.default_rng(5)
    cases = [(0.0, 0, 1.0, 0.0), (1.0, 0, 1.0, 0.0), (0.7, 40, 1.0, 0.0), (1.3, 0, 0.8, 0.0),
             (0.9, 0, 1.0, 0.05), (0.5, 3, 0.9, 0.01), (1.0, 1, 1.0, 0.0), (2.0, 0, 0.3, 0.0)]
    R = len(cases)
    logits = torch.tensor(rng.normal(0, 3, (R, V)), dtype=torch.float32)
    logits[2, 5] = logits[2, 9] = logits[2].max() + 1                       # a tie at the top
    u = rng.random(R)
    dev = lambda a, dt: torch.tensor(a, dtype=dt, device=DEV)
    temp = dev([c[0] for c in cases], torch.float32)
    tk = dev([c[1] for c in cases], torch.int32)
    tp = dev([c[2] for c in cases], torch.float32)
    mp = dev([c[3] for c in cases], torch.float32)
    draws = dev(u, torch.float64)
    out0 = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), temp, tk, tp, mp, draws, out0)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    lp = torch.empty(R, dtype=torch.float32, device=DEV)
    ids = torch.empty(R, 5, dtype=torch.int32, device=DEV)
    tlp = torch.empty(R, 5, dtype=torch.float32, device=DEV)
    want = dev([1] * (R - 1) + [0], torch.int32)
    ops.sample(logits.to(DEV), temp, tk, tp, mp, draws, out, lp, ids, tlp, want)
    assert torch.equal(out, out0)
    for r, (t, k, p, m) in enumerate(cases):
        greedy_row = t <= 0 or k == 1 or p <= 0
        tok, chosen, top = plain_llama.sample_with_logprobs(logits[r].numpy(), t if t > 0 else 1.0, k, p, m, u[r], greedy_row)
        assert out[r].item() == tok
        assert abs(lp[r].item() - chosen) < 1e-3, (r, lp[r].item(), chosen)
        got = [(i, x) for i, x in zip(ids[r].tolist(), tlp[r].tolist()) if i >= 0]
        if greedy_row or r == R - 1:                 # no list for greedy rows and for rows that did not ask
            assert got == []
        else:
            assert [i for i, _ in got] == [i for i, _ in top], (r, got, top)
            assert all(abs(a - b) < 1e-3 for (_, a), (_, b) in zip(got, top)), (r, got, top)
