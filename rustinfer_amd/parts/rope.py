"""Rotary position encoding with the llama3 frequency rescale.

Frequencies ``f_i = theta^(-2i/rot_dim)``; llama3 scaling keeps wavelengths
shorter than ``O/high``, divides those longer than ``O/low`` by ``factor`` and
blends in between; angles ``pos * f_i`` are formed in 64-bit and the sin/cos
tables kept in 32-bit (crates/infer-worker/src/models/loader.rs:1533-1590; the
reference rounds the tables to the model dtype, this engine does not).  The
rotation itself pairs element ``i`` with ``i + rot_dim/2``
(crates/infer-backend-cuda/src/kernels/rope/rope.cu:84-133) and is done by the
kernel that also writes keys and values into the cache.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..config.model_config import RopeScaling
from .base import PositionEncoding, Runtime


def rotary_frequencies(rot_dim: int, theta: float, scaling: Optional[RopeScaling]) -> torch.Tensor:
    half = rot_dim // 2
    freqs = [1.0 / (theta ** (2.0 * i / rot_dim)) for i in range(half)]
    if scaling is not None:
        orig = float(scaling.original_max_position_embeddings)
        lam_low = orig / scaling.low_freq_factor
        lam_high = orig / scaling.high_freq_factor
        for i, f in enumerate(freqs):
            lam = 2.0 * math.pi / f
            if lam < lam_high:
                continue
            if lam > lam_low:
                freqs[i] = f / scaling.factor
            else:
                s = (orig / lam - scaling.low_freq_factor) / (
                    scaling.high_freq_factor - scaling.low_freq_factor)
                freqs[i] = (1.0 - s) * (f / scaling.factor) + s * f
    return torch.tensor(freqs, dtype=torch.float64)


class RotaryEmbedding(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, scaling: Optional[RopeScaling] = None,
                 rot_dim: Optional[int] = None):
        self.head_dim = int(head_dim)
        self.rot_dim = int(rot_dim if rot_dim is not None else head_dim)
        if self.rot_dim % 2 or not (0 < self.rot_dim <= self.head_dim):
            raise ValueError(f"rot_dim {self.rot_dim} must be even and within head_dim {self.head_dim}")
        self.theta = float(theta)
        self.scaling = scaling
        self.cos = self.sin = None
        self.max_positions = 0

    def prepare(self, rt: Runtime, max_positions: int) -> None:
        self.rt = rt
        if self.cos is not None and self.max_positions >= max_positions:
            return
        freqs = rotary_frequencies(self.rot_dim, self.theta, self.scaling)
        pos = torch.arange(max_positions, dtype=torch.float64)
        ang = pos[:, None] * freqs[None, :]
        self.cos = ang.cos().to(torch.float32).to(rt.device).contiguous()
        self.sin = ang.sin().to(torch.float32).to(rt.device).contiguous()
        self.max_positions = max_positions

    def rotary(self):
        return self.cos, self.sin, self.rot_dim
