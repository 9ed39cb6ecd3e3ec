"""Interfaces of the parts a model is put together from.

A model is a list of blocks and a run order.  A block arranges a *mixer*
(something that moves information between positions: attention here) and a
*feed-forward* around *norms*; a *position encoding* is handed to the parts that
use it.  Every part takes its sizes and constants as constructor arguments and
never learns which model it sits in (reference seam: ``Component::run`` on a
``Hidden`` with a deferred delta, crates/infer-core/src/component.rs:8-84,
crates/infer-worker/src/components/decoder_block.rs:9-31).

What a part must provide
------------------------
``param_specs()``   checkpoint tensors it reads, by name relative to the part:
                    ``{name: ParamSpec(shape, kind)}``.
``load(tensors, rt)``  take those tensors (CPU or device, stored dtype) and keep
                    what the kernels need on ``rt.device`` in ``rt.dtype``.  ``tensors``
                    is indexed by name; it may make a tensor when it is asked for
                    (``LazyTensors``), so a part asks for each once and hands the names
                    of a part of its own on with ``narrow_tensors``.  Second copies in
                    another order come from ``rt.tile`` / ``rt.take_tile_budget``.
``forward(...)``    run on the tokens of one step, described by a ``StepContext``.

Mixer:        ``cache_need()`` -> ``PagedKVNeed`` | ``StateNeed`` | ``None`` and
              ``forward(ctx, normed, cache) -> delta [T, hidden]``.
FeedForward:  ``forward(ctx, normed) -> delta [T, hidden]``.
Norm:         ``forward(ctx, x, delta, out, rows=None)``: ``x += delta`` (if any),
              ``out = norm(x)``; with ``rows`` only those rows are read and ``out``
              has one row for each of them.
PositionEncoding: ``prepare(rt, max_positions)``; ``rotary()`` -> ``(cos, sin,
              rot_dim)`` or ``None``; ``on_embedding(ctx, x)`` for encodings that
              add to the embedded tokens.

Optional, for a mixer or a feed-forward (and the output head), so that a plain RMS norm
between two sub-layers needs no kernel of its own when a step has few tokens:
``takes_deferred_norm = True``: ``forward`` also accepts a ``DeferredNorm`` in place of
              the normalised rows: rows ``x * w`` that still lack the factor
              ``rsqrt(mean(x^2) + eps)``, which the part applies to the result of its
              first product (a product commutes with a factor per row).
``forward_into(ctx, normed, [cache,] x, next_norm)`` -> ``DeferredNorm`` or ``None``:
              as ``forward``, but the part adds its output to the residual stream ``x``
              itself and returns the input of the sub-layer behind ``next_norm``;
              ``None`` (and nothing done) where it cannot this time.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSpec:
    """A checkpoint tensor a part reads: its shape, and how the random-weights mode draws it.
    ``kind`` names one of the usual distributions; a part whose parameter needs another one (a
    decay in (0, 1), a bias around some value) gives ``mean``/``std`` of a normal distribution, or
    ``init(generator, shape, device) -> float32 tensor`` for anything else."""
    shape: Tuple[int, ...]
    kind: str = "matrix"      # "matrix": N(0, 0.02);  "norm": 1 (+ noise);  "int": int32 table
    int_high: int = 0         # for kind "int": values in [0, int_high)
    mean: Optional[float] = None
    std: Optional[float] = None
    init: Optional[Callable[..., torch.Tensor]] = None


@dataclass(frozen=True)
class PagedKVNeed:
    """Keys and values of every position (or of the last ``window`` positions)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """A fixed-size state for each live request, ``shape`` elements of ``dtype``."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class DeferredNorm:
    """The input of a sub-layer whose norm is not finished: ``rows = x * w`` in the run dtype and
    partial sums of squares ``ssq [T, P]`` (32-bit) with ``sum(ssq[t]) = sum(x[t]^2)``; the
    normalised rows would be ``rows * rsqrt(sum(ssq[t]) / dim + eps)``."""
    rows: torch.Tensor
    ssq: torch.Tensor
    eps: float

    @property
    def scale(self):
        return (self.ssq, self.eps)


def split_normed(normed):
    """(rows, scale) of a sub-layer's input, be it normalised rows or a ``DeferredNorm``."""
    if isinstance(normed, DeferredNorm):
        return normed.rows, normed.scale
    return normed, None


class LazyTensors:
    """name -> tensor for ``load``: a tensor is made when it is asked for and not kept, so that a
    model can be filled part by part without all of its tensors existing at once beside it."""

    def __init__(self, names, make: Callable[[str], torch.Tensor], prefix: str = ""):
        self._names, self._make, self._prefix = names, make, prefix

    def __getitem__(self, name: str) -> torch.Tensor:
        full = self._prefix + name
        if full not in self._names:
            raise KeyError(name)
        return self._make(full)

    def __contains__(self, name) -> bool:
        return self._prefix + str(name) in self._names

    def keys(self):
        return [n[len(self._prefix):] for n in self._names if n.startswith(self._prefix)]

    def __iter__(self):
        return iter(self.keys())

    def __len__(self) -> int:
        return len(self.keys())

    def items(self):
        return ((n, self[n]) for n in self.keys())

    def narrow(self, prefix: str) -> "LazyTensors":
        return LazyTensors(self._names, self._make, self._prefix + prefix + ".")


def narrow_tensors(tensors, prefix: str):
    """The tensors whose names begin with ``prefix.``, under the rest of their names."""
    if hasattr(tensors, "narrow"):
        return tensors.narrow(prefix)
    return {n[len(prefix) + 1:]: t for n, t in tensors.items() if n.startswith(prefix + ".")}


@dataclass
class Runtime:
    """Where and in which precision a model runs."""
    device: torch.device
    dtype: torch.dtype            # torch.bfloat16 (serving) or torch.float32 (exact path)
    ops: Any                      # the kernel module (rustinfer_amd.kernels.ops)
    # A second copy of every projection weight in the order the few-row kernels stream it (and a
    # third, row-permuted one of the q/k/v weight for the fused projection).  False: one copy, as
    # the checkpoint has it; single-token steps then read row-major weights, more slowly, and the
    # weights take half the memory.
    tiled_weight_copy: bool = True
    # Bytes the second copies may still take (None: as much as they like).  A model whose weights
    # fill most of the device keeps second copies of the weights that are loaded first and reads the
    # others as the checkpoint has them.
    tile_budget: Optional[int] = None
    tiled_bytes: int = 0          # what the second copies have taken so far

    def take_tile_budget(self, nbytes: int) -> bool:
        """Whether a second copy of ``nbytes`` may be made; if so it is taken off the budget."""
        if not self.tiled_weight_copy:
            return False
        if self.tile_budget is not None:
            if nbytes > self.tile_budget:
                return False
            self.tile_budget -= int(nbytes)
        self.tiled_bytes += int(nbytes)
        return True

    def give_tile_budget_back(self, nbytes: int) -> None:
        """A copy that was allowed and not made after all (its shape has no such form)."""
        self.tiled_bytes -= int(nbytes)
        if self.tile_budget is not None:
            self.tile_budget += int(nbytes)

    def tile(self, w):
        """The tile-ordered copy of ``w`` if this runtime keeps such copies, the shape has one and
        the budget allows it."""
        make = getattr(self.ops, "tile_weight", None)
        if make is None or not self.tiled_weight_copy:
            return None
        if not self.take_tile_budget(w.numel() * w.element_size()):
            return None
        t = make(w)
        if t is None:
            self.give_tile_budget_back(w.numel() * w.element_size())
        return t


class Part:
    # A step of single tokens is captured once per batch shape as a HIP graph, on rows that belong
    # to no request, and replayed for the real rows.  A part whose ``forward`` launches the same
    # kernels with the same arguments whatever the rows hold (it reads the step's device tensors
    # only, keeps its temporaries in ``ctx.workspace``, and never waits for the GPU) may be
    # captured.  A part that looks at the host copies in the context (``host_q_lens``,
    # ``host_q_start``, ``host_slots``, ``request_ids``), allocates, or synchronises says
    # ``graph_safe = False``; a model that holds one runs every step eagerly.
    graph_safe = True

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt


class Norm(Part):
    def forward(self, ctx, x, delta, out, rows=None):
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        return None

    def forward(self, ctx, normed, cache):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, normed):
        raise NotImplementedError


class PositionEncoding(Part):
    def prepare(self, rt: Runtime, max_positions: int) -> None:
        self.rt = rt

    def rotary(self):
        return None

    def on_embedding(self, ctx, x) -> None:
        return None


def stored_to(t: torch.Tensor, rt: Runtime, keep_fp32: bool = False) -> torch.Tensor:
    """Bring a checkpoint tensor to the device.  Floating tensors go to the run
    dtype, except that with ``keep_fp32`` a tensor stored in 32-bit stays 32-bit."""
    if t.dtype in (torch.int32, torch.int64, torch.uint8, torch.int8):
        return t.to(device=rt.device, dtype=torch.int32).contiguous()
    if keep_fp32 and t.dtype == torch.float32:
        return t.to(device=rt.device).contiguous()
    return t.to(device=rt.device, dtype=rt.dtype).contiguous()
