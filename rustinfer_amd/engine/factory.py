"""From a model folder to a running engine: config.json chooses the architecture, the
registry builds the model, the loader fills it, and the cache is sized.
(reference start-up: crates/infer-worker/src/application/serve_loop.rs:184-510.)"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import load_model_config
from ..parts.base import Runtime
from ..weights.loader import load_weights
from .step import Engine

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32}


def make_runtime(dtype="bfloat16", device="cuda:0", ops=None, tiled_weight_copy: bool = True) -> Runtime:
    if isinstance(dtype, str):
        if dtype not in _DTYPES:
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
        dtype = _DTYPES[dtype]
    device = torch.device(device)
    if ops is None:
        if device.type != "cuda":
            raise RuntimeError("the engine runs on a GPU only: its kernels are HIP kernels and "
                               "there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible to this process")
        from ..kernels import build, ops as hip_ops
        build.load()            # fails loudly if the kernel library cannot be built or loaded
        ops = hip_ops
        # products of the exact path never run in a reduced-precision matrix mode
        torch.backends.cuda.matmul.allow_tf32 = False
    return Runtime(device=device, dtype=dtype, ops=ops, tiled_weight_copy=bool(tiled_weight_copy))


def pages_that_fit(needs, page_size: int, element_size: int, free_bytes: int, mem_fraction: float,
                   max_requests: int, max_model_len: int) -> int:
    """Pages for ``mem_fraction`` of ``free_bytes`` less 1 GiB, after the fixed-size state of
    ``max_requests`` requests (and the scratch slot) has been taken from it; at most what
    ``max_requests`` full-length requests can use.  ``needs``: what ``DecoderModel.cache_needs``
    returns (serve_loop.rs:391-501)."""
    from ..parts.base import PagedKVNeed, StateNeed
    per_page = state = 0
    for need in needs.values():
        if isinstance(need, PagedKVNeed):
            per_page += 2 * need.num_kv_heads * need.head_dim * page_size * element_size
        elif isinstance(need, StateNeed):
            n = 1
            for d in need.shape:
                n *= int(d)
            state += (max_requests + 1) * n * torch.empty((), dtype=need.dtype).element_size()
    if per_page == 0:
        return 1
    budget = max(0, int((free_bytes - (1 << 30)) * mem_fraction) - state)
    cap = max_requests * ((max_model_len + page_size - 1) // page_size)
    return max(1, min(budget // per_page, cap))


def auto_num_pages(model, rt: Runtime, page_size: int, mem_fraction: float,
                   max_requests: int, max_model_len: int, held_bytes: int = 0) -> int:
    """``held_bytes``: device memory that will be given back before the pool is allocated (a
    bootstrap pool) and so counts as free."""
    free, _total = torch.cuda.mem_get_info(rt.device)
    return pages_that_fit(model.cache_needs(), page_size, 2 if rt.dtype == torch.bfloat16 else 4, free + held_bytes,
                          mem_fraction, max_requests, max_model_len)


TILE_MARGIN_BYTES = 8 << 30       # left beside weights, their second copies and the cache: workspaces, graphs, the GEMM library


def second_copy_budget(model, rt: Runtime, page_size: int, num_pages: int, max_requests: int,
                       reserve: float) -> Optional[int]:
    """Bytes the second, tile-ordered copies of the weights may take on ``rt.device``: what is
    free now, less the weights themselves, less the cache (``num_pages`` pages if that is given,
    else the share ``reserve`` of the device's memory) and a margin.  None off a GPU."""
    if rt.device.type != "cuda" or not torch.cuda.is_available():
        return None
    from ..parts.base import PagedKVNeed
    el = 2 if rt.dtype == torch.bfloat16 else 4
    weights = 0
    for spec in model.param_specs().values():
        n = 1
        for d in spec.shape:
            n *= int(d)
        weights += n * (4 if spec.kind == "int" else el)
    free, total = torch.cuda.mem_get_info(rt.device)
    # what the allocator holds and does not use is free to it as well
    free += max(0, torch.cuda.memory_reserved(rt.device) - torch.cuda.memory_allocated(rt.device))
    if num_pages > 0:
        cache = sum(2 * need.num_kv_heads * need.head_dim * page_size * el * (num_pages + 1)
                    for need in model.cache_needs().values() if isinstance(need, PagedKVNeed))
    else:
        cache = int(reserve * total)
    return max(0, free - weights - cache - TILE_MARGIN_BYTES)


def build_engine(model_dir: str, dtype="bfloat16", device="cuda:0", page_size: int = 16,
                 num_pages: int = 0, max_requests: int = 32, max_model_len: int = 4096,
                 max_batch_tokens: int = 8192, mem_fraction: float = 0.9, ops=None,
                 random_weights_seed: Optional[int] = None, tiled_weight_copy: bool = True,
                 tiled_weight_reserve: float = 0.25, tile_budget_bytes: Optional[int] = None) -> Engine:
    """``random_weights_seed``: do not read a checkpoint; draw the weights from this seed (the
    folder then needs config.json only).  ``tiled_weight_copy``: see ``parts.base.Runtime``; the
    second copies take what the device has left beside the weights and the cache (of an explicit
    ``num_pages``, else the share ``tiled_weight_reserve`` of its memory), or ``tile_budget_bytes``
    if that is given: a model that fills most of the device keeps second copies of the weights that
    are loaded first only."""
    rt = make_runtime(dtype, device, ops, tiled_weight_copy)
    entry, config = load_model_config(model_dir)
    model = entry.builder(config)
    if tiled_weight_copy:
        rt.tile_budget = int(tile_budget_bytes) if tile_budget_bytes is not None else \
            second_copy_budget(model, rt, page_size, num_pages, max_requests, tiled_weight_reserve)
    if random_weights_seed is not None and random_weights_seed >= 0:
        from ..weights.random_init import init_random_weights
        init_random_weights(model, random_weights_seed, rt, norm_noise=True)
    else:
        load_weights(model, model_dir, rt)
    if num_pages > 0:
        return Engine(model, rt, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                      max_model_len=max_model_len, max_batch_tokens=max_batch_tokens)
    # The pool takes what is free once everything else exists: a bootstrap pool that just holds the
    # largest step, one such step run eagerly (workspace, the GEMM library's buffers), then the
    # real pool in place of the bootstrap one (serve_loop.rs:391-510).
    worst = min(max_batch_tokens, max_requests * max_model_len)
    rows = -(-worst // max_model_len)
    bootstrap = -(-worst // page_size) + rows
    engine = Engine(model, rt, page_size=page_size, num_pages=bootstrap, max_requests=max_requests,
                    max_model_len=max_model_len, max_batch_tokens=max_batch_tokens)
    engine.profile_forward()
    held = sum(g.k_pool.numel() * g.k_pool.element_size() * 2 for g in engine.cache.groups) + engine.cache.state_bytes()
    # the state tensors are part of what auto_num_pages subtracts; the bootstrap's own go back with its pool
    num_pages = auto_num_pages(model, rt, page_size, mem_fraction, max_requests, max_model_len, held_bytes=held)
    engine.resize_pool(num_pages)
    return engine
