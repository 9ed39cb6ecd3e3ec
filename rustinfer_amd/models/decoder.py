"""A decoder-only model as data: an embedding, a list of blocks, the order in which
they run, a final norm and an output head.

The run order is a list of ``LayerCall``.  A call names the block to run and the
cache it uses, so a block may run twice (shared weights) and a block may read the
cache another call writes.  The reference's decoder is a homogeneous stage list
(crates/infer-worker/src/models/decoder.rs:57-200); selection of rows before the final
norm and head follows its ``finalize`` (:118-199): only the rows whose logits are
wanted are normalised and projected.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from ..parts.base import ParamSpec, Part, PositionEncoding, Runtime, narrow_tensors
from ..parts.block import Hidden
from ..parts.embed import Embedding, LMHead


@dataclass(frozen=True)
class LayerCall:
    layer: int                   # index into DecoderModel.layers
    cache: Optional[int] = None  # cache id; None = this call's own position in the run order
    write: bool = True           # False: read the cache, do not write it


class DecoderModel(Part):
    def __init__(self, config, embed: Embedding, layers: Sequence[Part],
                 final_norm, lm_head: LMHead,
                 position_encodings: Sequence[PositionEncoding] = (),
                 schedule: Optional[Sequence[LayerCall]] = None,
                 names: Optional[Dict[str, str]] = None):
        self.config = config
        self.embed = embed
        self.layers = list(layers)
        self.final_norm = final_norm
        self.lm_head = lm_head
        self.position_encodings = list(position_encodings)
        if schedule is None:
            schedule = [LayerCall(i) for i in range(len(self.layers))]
        self.schedule: List[LayerCall] = [
            LayerCall(c.layer, c.cache if c.cache is not None else pos, c.write)
            for pos, c in enumerate(schedule)]
        for c in self.schedule:
            if not (0 <= c.layer < len(self.layers)):
                raise ValueError(f"run order names layer {c.layer}, the model has {len(self.layers)}")
        self.names = {"embed": "model.embed_tokens", "layer": "model.layers.{i}",
                      "final_norm": "model.norm", "lm_head": "lm_head"}
        if names:
            self.names.update(names)
        self.hidden_size = embed.dim
        self.vocab_size = lm_head.vocab_size

    # -- weights ---------------------------------------------------------
    def _children(self):
        yield self.names["embed"], self.embed
        for i, layer in enumerate(self.layers):
            yield self.names["layer"].format(i=i), layer
        yield self.names["final_norm"], self.final_norm
        yield self.names["lm_head"], self.lm_head

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs: Dict[str, ParamSpec] = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[f"{prefix}.{name}"] = spec
        return specs

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        for prefix, part in self._children():
            sub = narrow_tensors(tensors, prefix)
            part.load(sub, rt)

    @property
    def graph_safe(self) -> bool:
        """Whether a step of this model may be captured as a graph: every part must allow it."""
        return all(getattr(part, "graph_safe", True) for _, part in self._children()) \
            and all(getattr(pe, "graph_safe", True) for pe in self.position_encodings)

    def prepare(self, rt: Runtime, max_positions: int) -> None:
        for pe in self.position_encodings:
            pe.prepare(rt, max_positions)

    # -- cache needs -------------------------------------------------------
    def cache_needs(self) -> Dict[int, object]:
        """cache id -> need, for every cache a call of the run order uses."""
        needs: Dict[int, object] = {}
        for call in self.schedule:
            need = self.layers[call.layer].cache_need()
            if need is None:
                continue
            if call.cache in needs and needs[call.cache] != need:
                raise ValueError(f"cache {call.cache} is used with two different needs")
            needs[call.cache] = need
        return needs

    # -- one step ------------------------------------------------------------
    def forward(self, ctx, caches) -> torch.Tensor:
        """Run the tokens of ``ctx`` and return 32-bit logits [len(ctx.want_rows), vocab]."""
        rt, ws = self.rt, ctx.workspace
        T = ctx.num_tokens
        x = ws.get("model.x", T, self.hidden_size, torch.float32)
        self.embed.forward(ctx, ctx.token_ids, x)
        for pe in self.position_encodings:
            pe.on_embedding(ctx, x)
        hidden = Hidden(x)
        W = ctx.num_want
        # Only the rows whose logits are wanted matter after the last block's mixer: a long prompt
        # portion that wants one row (or none) runs that block's feed-forward on that row alone.
        last = self.layers[self.schedule[-1].layer] if self.schedule else None
        cut = 0 < W < T and last is not None and getattr(last, "can_cut_rows", lambda: False)()
        # What comes after each call, for blocks that can prepare the next sub-layer's input
        # themselves: the next block's first norm and sub-layer; after the last block the final norm
        # and the head, if every row is wanted, in order (no gather between them).
        all_rows = W == T and bool(getattr(ctx, "want_all_in_order", False))
        for n, call in enumerate(self.schedule):
            cache = caches.view(call.cache, call.write) if call.cache in caches else None
            layer = self.layers[call.layer]
            if n + 1 < len(self.schedule):
                nxt = self.layers[self.schedule[n + 1].layer]
                follow = nxt.entry() if hasattr(nxt, "entry") else None
            else:
                follow = (self.final_norm, self.lm_head) if all_rows else None
            kw = {"follow": follow} if follow is not None and getattr(layer, "takes_follow", False) else {}
            if W == 0 and n == len(self.schedule) - 1 and hasattr(layer, "update_cache_only"):
                layer.update_cache_only(ctx, hidden, cache)      # nobody reads what this block would add
            elif cut and n == len(self.schedule) - 1:
                layer.forward(ctx, hidden, cache, out_rows=ctx.want_rows)
            else:
                layer.forward(ctx, hidden, cache, **kw)
        if W == 0:
            return ws.get("model.logits", 0, self.vocab_size, torch.float32)
        logits = ws.get("model.logits", W, self.vocab_size, torch.float32)
        normed = ws.get("model.final_normed", W, self.hidden_size, rt.dtype)
        if all_rows and not cut:
            inp = hidden.input_behind(ctx, self.final_norm, normed)
        else:
            self.final_norm.forward(ctx, hidden.x, hidden.pending, normed, rows=None if cut else ctx.want_rows)
            inp = normed
        self.lm_head.forward(ctx, inp, logits)
        return logits
