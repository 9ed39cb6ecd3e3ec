"""The arrangement of parts in one layer: pre-norm residual.

``x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x))``.  A sub-layer's output is not
added at once: it stays *pending* and the next norm adds it while it normalises
(crates/infer-worker/src/components/attention.rs:83-95,179,
crates/infer-worker/src/components/ffn_dense.rs:97-113).  Either half may be absent.

With few tokens in a step a norm's kernel takes as long as a product, so a sub-layer that
can (``forward_into``) adds its output to the residual stream itself and hands the next
sub-layer a ``DeferredNorm``: the norm between them is done by the two products around it.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import FeedForward, Mixer, Norm, ParamSpec, Part, Runtime, narrow_tensors


class Hidden:
    """Residual stream ``x`` (32-bit, [T, hidden]) and either a delta not yet added to it
    (``pending``) or, with ``x`` complete, the input that a sub-layer has already prepared for
    the sub-layer behind a given norm (``deferred = (that norm, DeferredNorm)``)."""

    __slots__ = ("x", "pending", "deferred")

    def __init__(self, x: torch.Tensor):
        self.x = x
        self.pending = None
        self.deferred = None

    def input_behind(self, ctx, norm, out: torch.Tensor):
        """What the sub-layer behind ``norm`` reads: the prepared input if there is one for this
        norm, else ``norm`` run into ``out`` (adding the pending delta)."""
        if self.deferred is not None:
            made_for, prepared = self.deferred
            self.deferred = None
            if made_for is norm:
                return prepared
        norm.forward(ctx, self.x, self.pending, out)
        self.pending = None
        return out


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
            sub = narrow_tensors(tensors, prefix)
            part.load(sub, rt)

    def cache_need(self):
        return self.mixer.cache_need() if self.mixer is not None else None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(part, "graph_safe", True) for _, part in self._children())

    def can_cut_rows(self) -> bool:
        """Whether forward() can leave the residual stream with a subset of its rows."""
        return self.ffn is not None and getattr(self.ffn_norm, "cuts_rows", False)

    takes_follow = True          # forward() accepts ``follow``

    def entry(self):
        """(norm, sub-layer) that a step enters this block through."""
        return (self.mixer_norm, self.mixer) if self.mixer is not None else (self.ffn_norm, self.ffn)

    def forward(self, ctx, hidden: Hidden, cache, out_rows: Optional[torch.Tensor] = None, follow=None) -> None:
        """``out_rows`` (row indices on the device): nothing after this block needs the other
        rows.  The mixer still sees every token (it fills the cache), but the feed-forward half
        runs on those rows only, and ``hidden`` leaves with them alone.
        ``follow``: (norm, sub-layer) that come after this block (the next block's ``entry()``, or
        the final norm and the head), if the caller allows the last sub-layer here to prepare
        that sub-layer's input."""
        T = hidden.x.shape[0]
        normed = ctx.workspace.get("block.normed", T, self.hidden_size, self.rt.dtype)
        if self.mixer is not None:
            inp = hidden.input_behind(ctx, self.mixer_norm, normed)
            after = (self.ffn_norm, self.ffn) if self.ffn is not None else follow
            self._run(self.mixer, ctx, hidden, inp, after if out_rows is None or self.ffn is None else None, cache)
        if self.ffn is not None:
            if out_rows is not None:
                W = out_rows.numel()
                x_rows = ctx.workspace.get("block.x_rows", W, self.hidden_size, torch.float32)
                normed = ctx.workspace.get("block.normed_rows", W, self.hidden_size, self.rt.dtype)
                self.ffn_norm.forward(ctx, hidden.x, hidden.pending, normed, rows=out_rows, x_rows=x_rows)
                hidden.x, hidden.pending, hidden.deferred = x_rows, None, None
                hidden.pending = self.ffn.forward(ctx, normed)
            else:
                inp = hidden.input_behind(ctx, self.ffn_norm, normed)
                self._run(self.ffn, ctx, hidden, inp, follow)

    def update_cache_only(self, ctx, hidden: Hidden, cache) -> None:
        """The last block of a step whose logits nobody wants (a prompt portion before the last):
        only what later steps read is made.  A mixer that has ``update_cache`` fills its cache and
        computes no output; any other mixer runs whole (its state must move on); the feed-forward
        half is left out.  ``hidden`` is not meaningful afterwards."""
        if self.mixer is None:
            return
        normed = ctx.workspace.get("block.normed", hidden.x.shape[0], self.hidden_size, self.rt.dtype)
        inp = hidden.input_behind(ctx, self.mixer_norm, normed)
        update = getattr(self.mixer, "update_cache", None)
        if update is not None:
            update(ctx, inp, cache)
        else:
            self.mixer.forward(ctx, inp, cache)

    def _run(self, part, ctx, hidden: Hidden, inp, after, *cache) -> None:
        """Run a sub-layer.  If it can (``forward_into``), the norm after it is a plain RMS norm and the
        sub-layer behind that norm takes a ``DeferredNorm``, it adds its output to the residual stream
        itself and prepares that sub-layer's input; else its output stays pending."""
        into = getattr(part, "forward_into", None)
        if into is not None and after is not None:
            norm, consumer = after
            if getattr(norm, "plain_rms", False) and getattr(consumer, "takes_deferred_norm", False):
                prepared = into(ctx, inp, *cache, hidden.x, norm)
                if prepared is not None:
                    hidden.pending, hidden.deferred = None, (norm, prepared)
                    return
        hidden.pending, hidden.deferred = part.forward(ctx, inp, *cache), None
