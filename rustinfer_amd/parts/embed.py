"""Token embedding and output head.

``x[t, :] = E[id_t, :]`` with no scale (crates/infer-worker/src/components/embed.rs:63-137);
the head is a projection onto the vocabulary that shares the embedding table when the
model ties them (crates/infer-worker/src/models/decoder.rs:245-262,
crates/infer-worker/src/components/lm_head.rs:13-20).  Logits leave in 32-bit.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import ParamSpec, Part, Runtime, split_normed, stored_to


class Embedding(Part):
    def __init__(self, vocab_size: int, dim: int):
        self.vocab_size = int(vocab_size)
        self.dim = int(dim)
        self.weight = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab_size, self.dim), "matrix")}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = stored_to(tensors["weight"], rt)

    def forward(self, ctx, ids: torch.Tensor, out_x: torch.Tensor) -> torch.Tensor:
        self.rt.ops.embed(ids, self.weight, out_x, getattr(ctx, "device_tokens", None))
        return out_x


class LMHead(Part):
    def __init__(self, vocab_size: int, dim: int, tied_to: Optional[Embedding] = None):
        self.vocab_size = int(vocab_size)
        self.dim = int(dim)
        self.tied_to = tied_to
        self.weight = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.tied_to is not None:
            return {}
        return {"weight": ParamSpec((self.vocab_size, self.dim), "matrix")}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        if self.tied_to is not None:
            self.weight = self.tied_to.weight      # same storage, no copy
        else:
            self.weight = stored_to(tensors["weight"], rt)
        self.weight_tiled = rt.tile(self.weight)

    takes_deferred_norm = True

    def forward(self, ctx, normed, logits: torch.Tensor) -> torch.Tensor:
        rows, scale = split_normed(normed)
        if scale is None:
            self.rt.ops.linear(rows, self.weight, logits, self.weight_tiled)
        else:
            self.rt.ops.linear(rows, self.weight, logits, self.weight_tiled, scale=scale)
        return logits
