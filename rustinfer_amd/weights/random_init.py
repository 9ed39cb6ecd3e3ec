"""Random-weights mode: a model folder (config.json + model.safetensors) from a
configuration and a seed.

Each tensor has its own stream, seeded by the seed and the tensor's checkpoint name,
so values do not depend on the order of creation.  Matrices are N(0, 0.02); norm
weights are 1 + N(0, 0.02) (or exactly 1 with ``norm_noise=False``); integer tables
are uniform; a spec may instead give the mean and deviation of a normal distribution or a
function that draws the tensor (``ParamSpec.mean/std/init``).  The reference only has a
generic seeded ``randn`` (crates/infer-core/src/tensor.rs:553-606) and never builds a model
from it.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterator, Tuple

import torch

from .safetensors_io import write_safetensors


def tensor_seed(seed: int, name: str) -> int:
    h = hashlib.blake2b(f"{seed}:{name}".encode("utf-8"), digest_size=8).digest()
    return int.from_bytes(h, "little") & ((1 << 63) - 1)


def random_tensor(name: str, spec, seed: int, dtype: torch.dtype, device="cpu",
                  norm_noise: bool = True, std: float = 0.02) -> torch.Tensor:
    g = torch.Generator(device=device)
    g.manual_seed(tensor_seed(seed, name))
    if spec.init is not None:
        t = spec.init(g, tuple(spec.shape), device)
        if tuple(t.shape) != tuple(spec.shape):
            raise ValueError(f"{name}: init returned shape {tuple(t.shape)}, the spec says {tuple(spec.shape)}")
        return t if not t.is_floating_point() else t.to(dtype)
    if spec.mean is not None or spec.std is not None:
        t = torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32)
        return (t * (std if spec.std is None else spec.std) + (spec.mean or 0.0)).to(dtype)
    if spec.kind == "int":
        return torch.randint(0, max(1, spec.int_high), spec.shape, generator=g,
                             device=device, dtype=torch.int32)
    if spec.kind not in ("matrix", "norm"):
        raise ValueError(f"{name}: unknown kind {spec.kind!r} (matrix, norm, int; or give mean/std or init)")
    t = torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32) * std
    if spec.kind == "norm":
        t = t + 1.0 if norm_noise else torch.ones_like(t)
    return t.to(dtype)


def random_tensors(model, seed: int, dtype: torch.dtype = torch.bfloat16, device="cpu",
                   norm_noise: bool = True) -> Iterator[Tuple[str, torch.Tensor]]:
    for name, spec in sorted(model.param_specs().items()):
        yield name, random_tensor(name, spec, seed, dtype, device, norm_noise)


def write_random_model(config, seed: int, out_dir: str, dtype: torch.dtype = torch.bfloat16,
                       norm_noise: bool = True) -> str:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors`` and return ``out_dir``."""
    from ..config.registry import resolve_architecture
    entry = resolve_architecture(config.to_dict())
    model = entry.builder(config)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=2)
    tensors = dict(random_tensors(model, seed, dtype, "cpu", norm_noise))
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return out_dir


def init_random_weights(model, seed: int, rt, norm_noise: bool = False) -> None:
    """Fill ``model`` with random weights on ``rt.device`` without a file (benchmarks, the
    ``random_weights_seed`` option).  Tensors are drawn one by one, so that no full 32-bit copy
    of the model ever exists, and by the generator of ``rt.device``: on a GPU eight billion
    values take a second, but they are not the values ``write_random_model`` draws on the CPU
    for the same seed and name.  Both are reproducible; a run that must agree with a written
    folder loads that folder."""
    from ..parts.base import LazyTensors
    specs = model.param_specs()
    # each tensor is drawn when its part asks for it: beside the model only the tensors of the
    # part that is being filled exist, so a model that fills most of the device can be drawn
    model.load(LazyTensors(specs, lambda name: random_tensor(name, specs[name], seed, rt.dtype, rt.device, norm_noise)), rt)
