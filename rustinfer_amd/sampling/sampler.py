"""Choosing the next token from logits on the device.

Greedy rows take the largest logit (lowest id on ties).  Other rows draw from the softmax
of ``logits / temperature`` after the top-k, min-p and top-p filters, with one uniform
number per row.  The number is a function of the request's seed and of the position of the
token it produces, not of the row's place in the batch (the reference also mixes in the row
index, crates/infer-worker/src/application/sampler_stack.rs:71-85), so a request draws the
same tokens however it is batched or cut into steps.
"""
from __future__ import annotations

import os
from typing import List, Sequence

import numpy as np
import torch

from .params import SamplingParams

_MASK = (1 << 64) - 1


def splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform_draw(seed: int, position: int) -> float:
    """A number in [0, 1) for the token at ``position`` of a request seeded with ``seed``."""
    h = splitmix64((seed & _MASK) ^ ((position * 0x9E3779B97F4A7C15) & _MASK))
    return (h >> 11) * (1.0 / (1 << 53))


def fresh_seed() -> int:
    return int.from_bytes(os.urandom(8), "little")


class Sampler:
    def __init__(self, rt, max_rows: int = 64):
        self.rt = rt
        self._cap = 0
        self._grow(max_rows)

    def _grow(self, rows: int) -> None:
        dev = self.rt.device
        self._cap = rows
        self._out = torch.empty(rows, dtype=torch.int32, device=dev)
        self._f = torch.empty((3, rows), dtype=torch.float32, device=dev)
        self._k = torch.empty(rows, dtype=torch.int32, device=dev)
        self._u = torch.empty(rows, dtype=torch.float64, device=dev)

    def greedy_device(self, logits: torch.Tensor) -> torch.Tensor:
        """Argmax of every row, left on the device (int32 [rows])."""
        R = logits.shape[0]
        if R > self._cap:
            self._grow(max(R, 2 * self._cap))
        self.rt.ops.argmax(logits, self._out[:R])
        return self._out[:R]

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               positions: Sequence[int]) -> List[int]:
        """One token for each row; ``positions[i]`` is the position the new token will take."""
        R = logits.shape[0]
        if R == 0:
            return []
        if R > self._cap:
            self._grow(max(R, 2 * self._cap))
        self.sample_into(logits, params, seeds, positions, self._out[:R])
        return self._out[:R].tolist()

    def sample_into(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
                    positions: Sequence[int], out: torch.Tensor) -> None:
        """As ``sample``, but the tokens are left in ``out`` (int32, on the device): nothing waits."""
        R = logits.shape[0]
        if not (len(params) == len(seeds) == len(positions) == R):
            raise ValueError("sample: one params, seed and position for each row of logits")
        if R == 0:
            return
        if R > self._cap:
            self._grow(max(R, 2 * self._cap))
        if all(p.is_greedy for p in params):
            self.rt.ops.argmax(logits, out)
            return
        f = np.empty((3, R), dtype=np.float32)
        k = np.empty(R, dtype=np.int32)
        u = np.empty(R, dtype=np.float64)
        for i, (p, s, pos) in enumerate(zip(params, seeds, positions)):
            f[0, i] = 0.0 if p.is_greedy else p.temperature
            f[1, i], f[2, i] = p.top_p, p.min_p
            k[i] = max(0, p.top_k)
            u[i] = uniform_draw(s, pos)
        self._f[:, :R].copy_(torch.from_numpy(f))
        self._k[:R].copy_(torch.from_numpy(k))
        self._u[:R].copy_(torch.from_numpy(u))
        self.rt.ops.sample(logits, self._f[0, :R], self._k[:R], self._f[1, :R], self._f[2, :R],
                           self._u[:R], out)
