"""RMSNorm with the residual add folded in.

``y = x * rsqrt(mean(x^2) + eps) * w``; the weight multiplies directly
(crates/infer-worker/src/components/norm.rs:19-26,
crates/infer-backend-cuda/src/kernels/rmsnorm/rmsnorm.cu:52-113).  The fused
form ``x += delta; out = norm(x)`` is the reference's ``fused_add_rmsnorm``
(crates/infer-core/src/ports/fused_ops.rs:42-52); here the residual ``x`` is kept
in 32-bit, so the sum is rounded once, into ``out``.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import Norm, ParamSpec, Runtime, stored_to


class RMSNorm(Norm):
    def __init__(self, dim: int, eps: float):
        self.dim = int(dim)
        self.eps = float(eps)
        self.weight = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.dim,), "norm")}

    def load(self, tensors, rt: Runtime) -> None:
        self.rt = rt
        self.weight = stored_to(tensors["weight"], rt, keep_fp32=True)

    cuts_rows = True          # forward() takes x_rows (see PreNormBlock.forward)
    # nothing but ``weight`` and ``eps``: the sub-layers around this norm may do it between them
    # (``forward_into`` and ``DeferredNorm``, see PreNormBlock.forward)
    plain_rms = True

    def forward(self, ctx, x, delta, out, rows=None, x_rows=None):
        self.rt.ops.add_rmsnorm(x, delta, self.weight, self.eps, out, rows, x_rows)
        return out
