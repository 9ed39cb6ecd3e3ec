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


def uniform_draws(seeds: Sequence[int], positions: Sequence[int]) -> np.ndarray:
    """``uniform_draw`` for many rows at once (64-bit arithmetic that wraps, as in the scalar form)."""
    with np.errstate(over="ignore"):
        x = np.array([s & _MASK for s in seeds], dtype=np.uint64) \
            ^ (np.array(positions, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15))
        x = x + np.uint64(0x9E3779B97F4A7C15)
        x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        x = x ^ (x >> np.uint64(31))
    return (x >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


class Sampler:
    """Per-row parameters travel to the device through a ring of pinned buffers and one
    asynchronous copy a step, so that sampling never makes the host wait for the GPU."""

    RING = 4

    def __init__(self, rt, max_rows: int = 64):
        self.rt = rt
        self._cap = 0
        self._turn = 0
        self._grow(max_rows)

    def _grow(self, rows: int) -> None:
        dev = self.rt.device
        if self._cap and dev.type == "cuda":
            torch.cuda.synchronize(dev)                      # copies from the old buffers may be in flight
        rows = (rows + 7) // 8 * 8
        self._cap = rows
        self._out = torch.empty(rows, dtype=torch.int32, device=dev)
        # one block of bytes: float32 [3][rows] (temperature, top_p, min_p) | int32 [rows] (top_k) |
        # float64 [rows] (draws) | int32 [rows] (who wants the five most probable tokens)
        nbytes = rows * 28
        pin = dev.type == "cuda"
        self._host = [torch.empty(nbytes, dtype=torch.uint8, pin_memory=pin) for _ in range(self.RING)]
        self._events = [None] * self.RING
        self._dev = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        self._f = self._dev[:rows * 12].view(torch.float32).view(3, rows)
        self._k = self._dev[rows * 12:rows * 16].view(torch.int32)
        self._u = self._dev[rows * 16:rows * 24].view(torch.float64)
        self._want = self._dev[rows * 24:].view(torch.int32)
        self._lp = torch.empty(rows, dtype=torch.float32, device=dev)
        self._top_ids = torch.empty(rows, 5, dtype=torch.int32, device=dev)
        self._top_lp = torch.empty(rows, 5, dtype=torch.float32, device=dev)

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
                    positions: Sequence[int], out: torch.Tensor):
        """As ``sample``, but the tokens are left in ``out`` (int32, on the device): nothing waits.
        If some row's parameters ask for log-probabilities, returns device tensors
        ``(logprobs [R], top_ids [R, 5], top_logprobs [R, 5])`` (rows that did not ask have no
        list: ids -1), else None."""
        R = logits.shape[0]
        if not (len(params) == len(seeds) == len(positions) == R):
            raise ValueError("sample: one params, seed and position for each row of logits")
        if R == 0:
            return
        if R > self._cap:
            self._grow(max(R, 2 * self._cap))
        with_lp = any(p.logprobs for p in params)
        if not with_lp and all(p.is_greedy for p in params):
            self.rt.ops.argmax(logits, out)
            return None
        cap = self._cap
        i = self._turn
        self._turn = (i + 1) % self.RING
        if self._events[i] is not None:
            self._events[i].synchronize()                    # the copy that last used this buffer is done
        host = self._host[i].numpy()
        f = host[:cap * 12].view(np.float32).reshape(3, cap)
        k = host[cap * 12:cap * 16].view(np.int32)
        u = host[cap * 16:cap * 24].view(np.float64)
        want = host[cap * 24:].view(np.int32)
        f[0, :R] = [0.0 if p.is_greedy else p.temperature for p in params]
        f[1, :R] = [p.top_p for p in params]
        f[2, :R] = [p.min_p for p in params]
        k[:R] = [max(0, p.top_k) for p in params]
        u[:R] = uniform_draws(seeds, positions)
        want[:R] = [1 if p.logprobs else 0 for p in params]
        self._dev.copy_(self._host[i], non_blocking=True)
        if self._dev.device.type == "cuda":
            ev = torch.cuda.Event()
            ev.record()
            self._events[i] = ev
        if not with_lp:
            self.rt.ops.sample(logits, self._f[0, :R], self._k[:R], self._f[1, :R], self._f[2, :R],
                               self._u[:R], out)
            return None
        self.rt.ops.sample(logits, self._f[0, :R], self._k[:R], self._f[1, :R], self._f[2, :R],
                           self._u[:R], out, self._lp[:R], self._top_ids[:R], self._top_lp[:R], self._want[:R])
        return self._lp[:R], self._top_ids[:R], self._top_lp[:R]
