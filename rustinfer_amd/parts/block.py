"""The arrangement of parts in one layer: pre-norm residual.

``x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x))``.  A sub-layer's output is not
added at once: it stays *pending* and the next norm adds it while it normalises
(crates/infer-worker/src/components/attention.rs:83-95,179,
crates/infer-worker/src/components/ffn_dense.rs:97-113).  Either half may be absent.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import FeedForward, Mixer, Norm, ParamSpec, Part, Runtime


class Hidden:
    """Residual stream ``x`` (32-bit, [T, hidden]) and a delta not yet added to it."""

    __slots__ = ("x", "pending")

    def __init__(self, x: torch.Tensor):
        self.x = x
        self.pending = None


class PreNormBlock(Part):
    def __init__(self, hidden_size: int,
                 mixer_norm: Optional[Norm], mixer: Optional[Mixer],
                 ffn_norm: Optional[Norm], ffn: Optional[FeedForward],
                 names: Optional[Dict[str, str]] = None):
        self.hidden_size = int(hidden_size)
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.ffn_norm, self.ffn = ffn_norm, ffn
        if (mixer is None) != (mixer_norm is None) or (ffn is None) != (ffn_norm is None):
            raise ValueError("a sub-layer and its norm come together")
        self.names = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                      "ffn_norm": "post_attention_layernorm", "ffn": "mlp"}
        if names:
            self.names.update(names)

    def _children(self):
        for key in ("mixer_norm", "mixer", "ffn_norm", "ffn"):
            part = getattr(self, key)
            if part is not None:
                yield self.names[key], part

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[f"{prefix}.{name}"] = spec
        return specs

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        for prefix, part in self._children():
            sub = {n[len(prefix) + 1:]: t for n, t in tensors.items() if n.startswith(prefix + ".")}
            part.load(sub, rt)

    def cache_need(self):
        return self.mixer.cache_need() if self.mixer is not None else None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", True) for _, part in self._children())

    def can_cut_rows(self) -> bool:
        """Whether forward() can leave the residual stream with a subset of its rows."""
        return self.ffn is not None and getattr(self.ffn_norm, "cuts_rows", False)

    def forward(self, ctx, hidden: Hidden, cache, out_rows: Optional[torch.Tensor] = None) -> None:
        """``out_rows`` (row indices on the device): nothing after this block needs the other
        rows.  The mixer still sees every token (it fills the cache), but the feed-forward half
        runs on those rows only, and ``hidden`` leaves with them alone."""
        T = hidden.x.shape[0]
        normed = ctx.workspace.get("block.normed", T, self.hidden_size, self.rt.dtype)
        if self.mixer is not None and not self._prenorm(self.mixer, self.mixer_norm, ctx, hidden, cache):
            self.mixer_norm.forward(ctx, hidden.x, hidden.pending, normed)
            hidden.pending = self.mixer.forward(ctx, normed, cache)
        if self.ffn is not None and out_rows is None and self._prenorm(self.ffn, self.ffn_norm, ctx, hidden):
            return
        if self.ffn is not None:
            if out_rows is not None:
                W = out_rows.numel()
                x_rows = ctx.workspace.get("block.x_rows", W, self.hidden_size, torch.float32)
                normed = ctx.workspace.get("block.normed_rows", W, self.hidden_size, self.rt.dtype)
                self.ffn_norm.forward(ctx, hidden.x, hidden.pending, normed, rows=out_rows, x_rows=x_rows)
                hidden.x = x_rows
            else:
                self.ffn_norm.forward(ctx, hidden.x, hidden.pending, normed)
            hidden.pending = self.ffn.forward(ctx, normed)

    def _prenorm(self, part, norm, ctx, hidden: Hidden, *cache) -> bool:
        """A sub-layer that has ``forward_prenorm(ctx, x, pending, norm, x_out, [cache])`` may take the
        residual stream and the pending delta as they are and fold the norm into its own first
        kernel (worth it for a few tokens, where the norm's kernel is as long as a product).
        It returns its delta, having written ``x + pending`` to ``x_out``, or None if it cannot
        this time; then the norm runs as a kernel of its own."""
        fused = getattr(part, "forward_prenorm", None)
        if fused is None or not getattr(norm, "plain_rms", False):
            return False
        T = hidden.x.shape[0]
        x_out = ctx.workspace.get("block.x_a", T, self.hidden_size, torch.float32)
        if x_out.data_ptr() == hidden.x.data_ptr():
            x_out = ctx.workspace.get("block.x_b", T, self.hidden_size, torch.float32)
        delta = fused(ctx, hidden.x, hidden.pending, norm, x_out, *cache)
        if delta is None:
            return False
        hidden.x, hidden.pending = x_out, delta
        return True
