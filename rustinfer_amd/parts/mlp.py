"""Dense SwiGLU feed-forward: ``down( silu(gate(x)) * up(x) )``.

Gate and up weights are stacked row-wise (gate first) so one product makes both
(crates/infer-worker/src/models/loader.rs:543-571); ``silu(z) = z / (1 + exp(-z))``
in 32-bit (crates/infer-worker/src/components/ffn_dense.rs:39-68,
crates/infer-backend-cuda/src/kernels/swiglu/swiglu.cu:294-343).
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import FeedForward, ParamSpec, Runtime
from .linear import Linear


class SwiGLUMLP(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up = Linear(self.hidden_size, 2 * self.intermediate_size)
        self.down = Linear(self.intermediate_size, self.hidden_size)

    def param_specs(self) -> Dict[str, ParamSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_proj.weight": ParamSpec((i, h)),
            "up_proj.weight": ParamSpec((i, h)),
            "down_proj.weight": ParamSpec((h, i)),
        }

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        gate = tensors["gate_proj.weight"].to(device=rt.device, dtype=rt.dtype)
        up = tensors["up_proj.weight"].to(device=rt.device, dtype=rt.dtype)
        self.gate_up.set_weight(torch.cat([gate, up], dim=0), rt)
        self.down.set_weight(tensors["down_proj.weight"], rt)

    def forward_prenorm(self, ctx, x: torch.Tensor, pending, norm, x_out: torch.Tensor):
        """A few rows: the norm before the feed-forward is made inside the gate/up product's
        kernel (see PreNormBlock._prenorm).  None where that form does not apply."""
        fold = getattr(self.rt.ops, "linear_swiglu_norm", None)
        if fold is None:
            return None
        ws = ctx.workspace
        act = ws.get("ffn.act", x.shape[0], self.intermediate_size, self.rt.dtype)
        if not fold(x, pending, norm.weight, norm.eps, x_out, self.gate_up.weight, self.gate_up.weight_tiled, act):
            return None
        return self.rt.ops.linear_delta(act, self.down.weight, ws, "ffn.out", self.down.weight_tiled)

    def forward(self, ctx, normed: torch.Tensor) -> torch.Tensor:
        T = normed.shape[0]
        ws = ctx.workspace
        gate_up = ws.get("ffn.gate_up", T, 2 * self.intermediate_size, self.rt.dtype)
        act = ws.get("ffn.act", T, self.intermediate_size, self.rt.dtype)
        self.rt.ops.linear_swiglu(normed, self.gate_up.weight, act, gate_up, self.gate_up.weight_tiled)
        return self.rt.ops.linear_delta(act, self.down.weight, ws, "ffn.out", self.down.weight_tiled)
