"""Weights by tensor name.

The model says which tensors it reads (``param_specs``); the loader checks the
checkpoint against that list before anything is copied and reports every missing
tensor, every tensor nobody reads and every wrong shape in ONE error.  (The
reference fails on the first missing tensor or bad shape and ignores extras:
crates/infer-worker/src/models/loader.rs:191-201, :1038-1052.)

Tensors reach the parts in the dtype they are stored in (16-bit floats of either kind,
32-bit; 64-bit floats as 32-bit), and each part casts once, from the stored dtype to the
run dtype (bfloat16 or float32), as the reference casts source to target directly
(crates/infer-worker/src/models/loader.rs:1398-1516): a float16 checkpoint is exact in a
float32 run.  Integer tables go to int32, and a vector that is stored in 32-bit and used in
32-bit arithmetic (norm weights) stays 32-bit.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..parts.base import Runtime
from .safetensors_io import SafetensorsReader, WeightError


def check_checkpoint(model, reader, tie_note: str = "") -> None:
    specs = model.param_specs()
    have = set(reader.names())
    missing = sorted(n for n in specs if n not in have)
    unexpected = sorted(n for n in have if n not in specs)
    wrong = []
    for name, spec in specs.items():
        if name in have:
            dtype, shape = reader.info(name)
            if tuple(shape) != tuple(spec.shape):
                wrong.append(f"{name}: expected {list(spec.shape)}, got {list(shape)}")
            elif spec.kind == "int" and dtype.is_floating_point:
                wrong.append(f"{name}: expected an integer table, got {dtype}")
            elif spec.kind != "int" and not dtype.is_floating_point:
                wrong.append(f"{name}: expected floating point, got {dtype}")
    if not (missing or unexpected or wrong):
        return
    lines = ["checkpoint does not fit the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shapes or types ({len(wrong)}): " + "; ".join(wrong))
    head = model.names.get("lm_head", "lm_head") + ".weight" if hasattr(model, "names") else None
    if head is not None:
        if head in unexpected:
            lines.append(f"  note: config says tie_word_embeddings=true but the checkpoint holds {head}")
        if head in missing:
            lines.append(f"  note: config says tie_word_embeddings=false but the checkpoint has no {head}")
    raise WeightError("\n".join(lines))


def load_weights(model, model_dir: str, rt: Runtime) -> None:
    """Check ``model_dir``'s checkpoint against ``model`` and load it onto ``rt.device``."""
    reader = SafetensorsReader(model_dir)
    check_checkpoint(model, reader)
    specs = model.param_specs()
    tensors: Dict[str, torch.Tensor] = {}
    for name in specs:
        t = reader.tensor(name)
        if t.dtype == torch.float64:
            t = t.to(torch.float32)
        tensors[name] = t
    model.load(tensors, rt)
