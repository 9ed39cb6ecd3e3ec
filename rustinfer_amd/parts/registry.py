"""Names for the kinds of part, so that a configuration can choose them layer by
layer (``layer_types``-like lists) and a new kind can be added from outside."""
from __future__ import annotations

from typing import Callable, Dict

from .attention import PagedAttention
from .mlp import SwiGLUMLP
from .norm import RMSNorm
from .rope import RotaryEmbedding

MIXERS: Dict[str, Callable] = {"attention": PagedAttention}
FEED_FORWARDS: Dict[str, Callable] = {"swiglu": SwiGLUMLP}
NORMS: Dict[str, Callable] = {"rmsnorm": RMSNorm}
POSITION_ENCODINGS: Dict[str, Callable] = {"rope": RotaryEmbedding}

_TABLES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS,
           "position_encoding": POSITION_ENCODINGS}


def _register(table: Dict[str, Callable], name: str, factory: Callable, replace: bool) -> None:
    if name in table and not replace:
        raise ValueError(f"{name!r} is already registered")
    table[name] = factory


def register_mixer(name, factory, replace=False):
    _register(MIXERS, name, factory, replace)


def register_feed_forward(name, factory, replace=False):
    _register(FEED_FORWARDS, name, factory, replace)


def register_norm(name, factory, replace=False):
    _register(NORMS, name, factory, replace)


def register_position_encoding(name, factory, replace=False):
    _register(POSITION_ENCODINGS, name, factory, replace)


def make_part(kind: str, name: str, **kwargs):
    """Build the part registered as ``name`` of ``kind`` ('mixer', 'feed_forward', 'norm',
    'position_encoding') with its sizes and constants as keyword arguments."""
    table = _TABLES[kind]
    if name not in table:
        raise KeyError(f"no {kind} named {name!r}; registered: {', '.join(sorted(table))}")
    return table[name](**kwargs)
