"""A dense projection ``out = x @ W^T`` with ``W`` stored ``[out, in]`` as in the
checkpoint (crates/infer-worker/src/components/linear.rs:172-212; no bias in this
architecture)."""
from __future__ import annotations

import torch

from .base import Runtime


class Linear:
    def __init__(self, in_features: int, out_features: int):
        self.in_features = int(in_features)
        self.out_features = int(out_features)
        self.weight = None
        self.weight_tiled = None

    def set_weight(self, w: torch.Tensor, rt: Runtime, tile: bool = True) -> None:
        """``tile=False``: the caller keeps a copy of its own for the few-row kernels."""
        if tuple(w.shape) != (self.out_features, self.in_features):
            raise ValueError(f"linear weight {tuple(w.shape)} != {(self.out_features, self.in_features)}")
        self.rt = rt
        self.weight = w.to(device=rt.device, dtype=rt.dtype).contiguous()
        # a second copy in the order the few-row kernel streams it (memory is plentiful, bandwidth is not)
        self.weight_tiled = rt.tile(self.weight) if tile else None

    def forward(self, x: torch.Tensor, out: torch.Tensor, scale=None) -> torch.Tensor:
        """``scale``: the row factors of a norm this product finishes (``DeferredNorm.scale``)."""
        if scale is None:
            self.rt.ops.linear(x, self.weight, out, self.weight_tiled)
        else:
            self.rt.ops.linear(x, self.weight, out, self.weight_tiled, scale=scale)
        return out
