"""Grouped-query attention over a paged key/value cache.

Per token: fused q/k/v projection (rows of q, then k, then v:
crates/infer-worker/src/models/loader.rs:419-454), rotation of q and k by absolute
position, write of k and v into the request's pages, attention of every query over
the positions it may see (``j <= p``, and ``j > p - window`` if a window is set;
bottom-right causal rule of crates/infer-core/src/ports/fused_ops.rs:430-535), and the
output projection (crates/infer-worker/src/components/attention.rs:44-181).
Query head ``h`` reads key/value head ``h // (H / Hkv)``; the scale is
``1/sqrt(head_dim)`` unless given (crates/infer-worker/src/models/decoder.rs:276).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import DeferredNorm, Mixer, PagedKVNeed, ParamSpec, PositionEncoding, Runtime, split_normed
from .linear import Linear


class PagedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 pos_enc: Optional[PositionEncoding] = None, scale: Optional[float] = None,
                 window: Optional[int] = None, own_kv: bool = True, qk_transform=None):
        """``qk_transform``: what a variant of this mixer does between the projection and the
        rotation (a norm or a scale per head on q and k, a bias): called as
        ``qk_transform(ctx, qkv, self)`` on the projected rows ``qkv [T, q_dim + 2 kv_dim]`` (queries
        first, then keys, then values; ``own_kv=False``: queries only), which it changes in place.
        It may be a part of its own: ``param_specs()`` / ``load(tensors, rt)`` are then used under
        the mixer's names, and ``graph_safe`` is honoured.  With a transform the projection, the
        rotation and the cache write run as separate kernels (the fused kernel has no place for it)."""
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.pos_enc = pos_enc
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.window = int(window) if window else None
        self.own_kv = bool(own_kv)       # False: no k/v projection, reads another layer's cache
        self.q_dim = self.num_heads * self.head_dim
        self.kv_dim = self.num_kv_heads * self.head_dim
        self.qkv_dim = self.q_dim + (2 * self.kv_dim if self.own_kv else 0)
        self.qkv = Linear(self.hidden_size, self.qkv_dim)
        self.o = Linear(self.q_dim, self.hidden_size)
        self.qkv_fused = None
        self.qk_transform = qk_transform

    @property
    def graph_safe(self) -> bool:
        return getattr(self.qk_transform, "graph_safe", True)

    def param_specs(self) -> Dict[str, ParamSpec]:
        h = self.hidden_size
        specs = {"q_proj.weight": ParamSpec((self.q_dim, h))}
        if self.own_kv:
            specs["k_proj.weight"] = ParamSpec((self.kv_dim, h))
            specs["v_proj.weight"] = ParamSpec((self.kv_dim, h))
        specs["o_proj.weight"] = ParamSpec((h, self.q_dim))
        if hasattr(self.qk_transform, "param_specs"):
            specs.update(self.qk_transform.param_specs())
        return specs

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        names = ["q_proj.weight"] + (["k_proj.weight", "v_proj.weight"] if self.own_kv else [])
        parts = [tensors[n].to(device=rt.device, dtype=rt.dtype) for n in names]
        # for steps of few single tokens: projection, rotation and cache write in one kernel, which
        # reads its own copy of the weight (rows ordered so that rotary partners meet in a tile);
        # the plain tile-ordered copy would never be read beside it
        make = getattr(rt.ops, "qkv_rope_weight", None)
        fuse = make is not None and rt.tiled_weight_copy and self.own_kv and self.qk_transform is None
        w = torch.cat(parts, dim=0) if len(parts) > 1 else parts[0]
        del parts
        self.qkv.set_weight(w, rt, tile=not fuse)
        self.qkv_fused = None
        if fuse and rt.take_tile_budget(w.numel() * w.element_size()):
            self.qkv_fused = make(self.qkv.weight, self.head_dim)
            if self.qkv_fused is None:           # no such copy for these sizes: the plain one, if any
                rt.give_tile_budget_back(w.numel() * w.element_size())
                self.qkv.weight_tiled = rt.tile(self.qkv.weight)
        self.o.set_weight(tensors["o_proj.weight"], rt)
        if hasattr(self.qk_transform, "load"):
            own = self.qk_transform.param_specs() if hasattr(self.qk_transform, "param_specs") else {}
            self.qk_transform.load({n: tensors[n] for n in own}, rt)

    takes_deferred_norm = True

    def _project(self, ctx, normed, cache):
        """Rotated queries in ``qkv`` (and this step's keys and values in the cache) from the input
        rows, be they normalised or a ``DeferredNorm``."""
        rows, scale = split_normed(normed)
        T = rows.shape[0]
        ws, ops = ctx.workspace, self.rt.ops
        qkv = ws.get("attn.qkv", T, self.qkv_dim, self.rt.dtype)
        rotary = self.pos_enc.rotary() if self.pos_enc is not None else None
        table = ctx.block_tables[cache.group]
        kw = {} if scale is None else {"scale": scale}
        fused = (self.qkv_fused is not None and cache.write and ctx.max_q_len == 1
                 and ops.qkv_rope_fused(rows, self.qkv_fused, qkv, self.num_heads, self.num_kv_heads,
                                        self.head_dim, rotary, ctx.positions, ctx.row_of_token,
                                        cache.k, cache.v, table, cache.page_size, **kw))
        if not fused:
            self.qkv.forward(rows, qkv, scale)
            if self.qk_transform is not None:
                self.qk_transform(ctx, qkv, self)
            ops.rope_kv_write(qkv, self.num_heads, self.num_kv_heads, self.head_dim, rotary,
                              ctx.positions, ctx.row_of_token, cache.k, cache.v, table,
                              cache.page_size, write_kv=self.own_kv and cache.write)
        return qkv, table

    def forward(self, ctx, normed, cache) -> torch.Tensor:
        qkv, table = self._project(ctx, normed, cache)
        attn = self._attend(ctx, qkv, cache, table)
        return self.rt.ops.linear_delta(attn, self.o.weight, ctx.workspace, "mixer.out", self.o.weight_tiled)

    def update_cache(self, ctx, normed, cache) -> None:
        """What a step leaves behind for later ones, and nothing else: this step's keys and values
        in the cache.  For the last block of a step whose logits nobody wants."""
        if self.own_kv and cache.write:
            self._project(ctx, normed, cache)

    def forward_into(self, ctx, normed, cache, x: torch.Tensor, next_norm):
        """Few rows: the output projection adds its sums to ``x`` itself and prepares the input behind
        ``next_norm`` (see parts/base.py).  None, and nothing done, where that form does not apply."""
        ops = self.rt.ops
        ok = getattr(ops, "linear_residual_ok", None)
        if ok is None or not ok(x.shape[0], self.o.weight, self.o.weight_tiled, next_norm.weight):
            return None
        pays = getattr(ops, "linear_residual_pays", None)
        if pays is not None and not pays(x.shape[0], self.o.weight):
            return None
        qkv, table = self._project(ctx, normed, cache)
        attn = self._attend(ctx, qkv, cache, table)
        a, ssq = ops.linear_residual(attn, self.o.weight, self.o.weight_tiled, x, next_norm.weight,
                                     ctx.workspace, "deferred")
        return DeferredNorm(a, ssq, next_norm.eps)

    def _attend(self, ctx, qkv: torch.Tensor, cache, table) -> torch.Tensor:
        """Attention over the cache with the rotated queries in ``qkv``."""
        ws, ops = ctx.workspace, self.rt.ops
        attn = ws.get("attn.out", qkv.shape[0], self.q_dim, self.rt.dtype)
        ops.paged_attention(qkv, attn, self.num_heads, self.num_kv_heads, self.head_dim,
                            cache.k, cache.v, table, cache.page_size, ctx, self.scale,
                            self.window or 0)
        return attn
