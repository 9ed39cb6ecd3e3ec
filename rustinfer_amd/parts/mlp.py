"""Dense SwiGLU feed-forward: ``down( silu(gate(x)) * up(x) )``.

Gate and up weights are stacked row-wise (gate first) so one product makes both
(crates/infer-worker/src/models/loader.rs:543-571); ``silu(z) = z / (1 + exp(-z))``
in 32-bit (crates/infer-worker/src/components/ffn_dense.rs:39-68,
crates/infer-backend-cuda/src/kernels/swiglu/swiglu.cu:294-343).
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import DeferredNorm, FeedForward, ParamSpec, Runtime, split_normed
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

    takes_deferred_norm = True

    def _activation(self, ctx, normed) -> torch.Tensor:
        """silu(gate) * up of the input rows (normalised, or with the norm's factor still to apply)."""
        rows, scale = split_normed(normed)
        T = rows.shape[0]
        ws = ctx.workspace
        act = ws.get("ffn.act", T, self.intermediate_size, self.rt.dtype)
        if scale is not None:
            self.rt.ops.linear_swiglu(rows, self.gate_up.weight, act, None, self.gate_up.weight_tiled, scale=scale)
        else:
            gate_up = ws.get("ffn.gate_up", T, 2 * self.intermediate_size, self.rt.dtype)
            self.rt.ops.linear_swiglu(rows, self.gate_up.weight, act, gate_up, self.gate_up.weight_tiled)
        return act

    def forward(self, ctx, normed) -> torch.Tensor:
        act = self._activation(ctx, normed)
        return self.rt.ops.linear_delta(act, self.down.weight, ctx.workspace, "ffn.out", self.down.weight_tiled)

    def forward_into(self, ctx, normed, x: torch.Tensor, next_norm):
        """Few rows: the down projection adds its sums to ``x`` itself and prepares the input behind
        ``next_norm`` (see parts/base.py).  None, and nothing done, where that form does not apply."""
        ops = self.rt.ops
        ok = getattr(ops, "linear_residual_ok", None)
        if ok is None or not ok(x.shape[0], self.down.weight, self.down.weight_tiled, next_norm.weight):
            return None
        pays = getattr(ops, "linear_residual_pays", None)
        if pays is not None and not pays(x.shape[0], self.down.weight):
            return None
        act = self._activation(ctx, normed)
        a, ssq = ops.linear_residual(act, self.down.weight, self.down.weight_tiled, x, next_norm.weight,
                                     ctx.workspace, "deferred")
        return DeferredNorm(a, ssq, next_norm.eps)
