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

from .base import Mixer, PagedKVNeed, ParamSpec, PositionEncoding, Runtime
from .linear import Linear


class PagedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 pos_enc: Optional[PositionEncoding] = None, scale: Optional[float] = None,
                 window: Optional[int] = None, own_kv: bool = True):
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

    def param_specs(self) -> Dict[str, ParamSpec]:
        h = self.hidden_size
        specs = {"q_proj.weight": ParamSpec((self.q_dim, h))}
        if self.own_kv:
            specs["k_proj.weight"] = ParamSpec((self.kv_dim, h))
            specs["v_proj.weight"] = ParamSpec((self.kv_dim, h))
        specs["o_proj.weight"] = ParamSpec((h, self.q_dim))
        return specs

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        names = ["q_proj.weight"] + (["k_proj.weight", "v_proj.weight"] if self.own_kv else [])
        parts = [tensors[n].to(device=rt.device, dtype=rt.dtype) for n in names]
        self.qkv.set_weight(torch.cat(parts, dim=0) if len(parts) > 1 else parts[0], rt)
        self.o.set_weight(tensors["o_proj.weight"], rt)
        # for steps of few single tokens: projection, rotation and cache write in one kernel, which
        # reads its own copy of the weight (rows ordered so that rotary partners meet in a tile)
        make = getattr(rt.ops, "qkv_rope_weight", None)
        self.qkv_fused = make(self.qkv.weight, self.head_dim) if (make is not None and self.own_kv) else None
        if self.qkv_fused is not None:
            self.qkv.weight_tiled = None         # the plain tile-ordered copy would never be read

    def forward_prenorm(self, ctx, x: torch.Tensor, pending, norm, x_out: torch.Tensor, cache):
        """A few single tokens: the norm before this layer half is made inside the fused
        projection's kernel (see PreNormBlock._prenorm).  None where that form does not apply."""
        ops = self.rt.ops
        fold = getattr(ops, "qkv_rope_fused_norm", None)
        if fold is None or self.qkv_fused is None or not cache.write or ctx.max_q_len != 1:
            return None
        T = x.shape[0]
        qkv = ctx.workspace.get("attn.qkv", T, self.qkv_dim, self.rt.dtype)
        rotary = self.pos_enc.rotary() if self.pos_enc is not None else None
        table = ctx.block_tables[cache.group]
        if not fold(x, pending, norm.weight, norm.eps, x_out, self.qkv_fused, qkv, self.num_heads,
                    self.num_kv_heads, self.head_dim, rotary, ctx.positions, ctx.row_of_token,
                    cache.k, cache.v, table, cache.page_size):
            return None
        return self._attend(ctx, qkv, cache, table)

    def forward(self, ctx, normed: torch.Tensor, cache) -> torch.Tensor:
        T = normed.shape[0]
        ws, ops = ctx.workspace, self.rt.ops
        qkv = ws.get("attn.qkv", T, self.qkv_dim, self.rt.dtype)
        rotary = self.pos_enc.rotary() if self.pos_enc is not None else None
        table = ctx.block_tables[cache.group]
        fused = (self.qkv_fused is not None and cache.write and ctx.max_q_len == 1
                 and ops.qkv_rope_fused(normed, self.qkv_fused, qkv, self.num_heads, self.num_kv_heads,
                                        self.head_dim, rotary, ctx.positions, ctx.row_of_token,
                                        cache.k, cache.v, table, cache.page_size))
        if not fused:
            self.qkv.forward(normed, qkv)
            ops.rope_kv_write(qkv, self.num_heads, self.num_kv_heads, self.head_dim, rotary,
                              ctx.positions, ctx.row_of_token, cache.k, cache.v, table,
                              cache.page_size, write_kv=self.own_kv and cache.write)
        return self._attend(ctx, qkv, cache, table)

    def _attend(self, ctx, qkv: torch.Tensor, cache, table) -> torch.Tensor:
        """Attention over the cache with the rotated queries in ``qkv``, then the output projection."""
        ws, ops = ctx.workspace, self.rt.ops
        attn = ws.get("attn.out", qkv.shape[0], self.q_dim, self.rt.dtype)
        ops.paged_attention(qkv, attn, self.num_heads, self.num_kv_heads, self.head_dim,
                            cache.k, cache.v, table, cache.page_size, ctx, self.scale,
                            self.window or 0)
        return ops.linear_delta(attn, self.o.weight, ws, "mixer.out", self.o.weight_tiled)
