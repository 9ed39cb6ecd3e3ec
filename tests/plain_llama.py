"""A plain, slow implementation of the dense Llama-3 decoder, written from the reference's
formulas: whole sequences, no cache, one function for each part, 64-bit arithmetic, and no
code shared with ``rustinfer_amd``.  The reference was read, not run.

Each function cites where the reference computes the same thing.  Paths are relative to
the reference's root; ``W/`` = crates/infer-worker/src, ``C/`` = crates/infer-core/src,
``CU/`` = crates/infer-backend-cuda/src, ``CPU`` = crates/infer-backend-cpu/src/lib.rs.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np


# ---------------------------------------------------------------------------
# reading a model folder (own reader: nothing of the engine's loader is used)
# ---------------------------------------------------------------------------
def read_safetensors(path: str) -> Dict[str, np.ndarray]:
    """All tensors of a .safetensors file as float64 / int64 arrays.
    Container format as parsed in W/infrastructure/io/safetensors.rs:47-213."""
    with open(path, "rb") as f:
        (hlen,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hlen))
        data = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        raw = data[b:e]
        dt = info["dtype"]
        if dt == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif dt == "BF16":
            u = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            arr = u.view(np.float32).astype(np.float64)
        elif dt == "F16":
            arr = np.frombuffer(raw, dtype="<f2").astype(np.float64)
        elif dt == "I32":
            arr = np.frombuffer(raw, dtype="<i4").astype(np.int64)
        elif dt == "I64":
            arr = np.frombuffer(raw, dtype="<i8").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {dt}")
        out[name] = arr.reshape(info["shape"])
    return out


def read_model(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(model_dir, "model.safetensors"))


# ---------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------
def embedding(table: np.ndarray, ids) -> np.ndarray:
    """x[t, :] = E[id_t, :], no scale.  W/components/embed.rs:78-81, CPU:533-559."""
    return table[np.asarray(ids, dtype=np.int64)]


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """y = x * w / sqrt(mean(x^2) + eps); the weight multiplies directly (no 1 + w).
    W/components/norm.rs:19-26, CPU:701-728."""
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return x * w / np.sqrt(ms + eps)


def rope_frequencies(head_dim: int, theta: float, scaling: Optional[dict]) -> np.ndarray:
    """f_i = theta^(-2i/head_dim), i < head_dim/2, then the llama3 rescale by wavelength:
    shorter than O/high: kept; longer than O/low: divided by factor; between: blended with
    s = (O/lambda - low) / (high - low).  W/models/loader.rs:1543-1571.  Scaling applies
    only for rope_type 'llama3' (W/bin/worker_main.rs:393-404)."""
    half = head_dim // 2
    f = np.array([theta ** (-2.0 * i / head_dim) for i in range(half)], dtype=np.float64)
    if scaling is not None and scaling.get("rope_type", scaling.get("type")) == "llama3":
        F = float(scaling["factor"])
        lo = float(scaling["low_freq_factor"])
        hi = float(scaling["high_freq_factor"])
        O = float(scaling["original_max_position_embeddings"])
        for i in range(half):
            lam = 2.0 * math.pi / f[i]
            if lam < O / hi:
                pass
            elif lam > O / lo:
                f[i] = f[i] / F
            else:
                s = (O / lam - lo) / (hi - lo)
                f[i] = (1.0 - s) * f[i] / F + s * f[i]
    return f


def rope(x: np.ndarray, positions: np.ndarray, freqs: np.ndarray) -> np.ndarray:
    """Rotate [T, heads, head_dim] by absolute position, pairing element i with i + head_dim/2:
    x[i] <- a cos - b sin, x[i + hd/2] <- a sin + b cos with a = x[i], b = x[i + hd/2].
    CU/kernels/rope/rope.cu:107-119 (the production kernel; the CPU backend's interleaved
    pairing, CPU:843-868, disagrees with the loader's tables and is not followed)."""
    half = x.shape[-1] // 2
    ang = positions.astype(np.float64)[:, None] * freqs[None, :]       # [T, half]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return np.concatenate([a * c - b * s, a * s + b * c], axis=-1)


def softmax(s: np.ndarray) -> np.ndarray:
    """Along the last axis, with the maximum subtracted.  CPU:501-531."""
    m = np.max(s, axis=-1, keepdims=True)
    e = np.exp(s - m)
    return e / np.sum(e, axis=-1, keepdims=True)


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
              window: Optional[int] = None) -> np.ndarray:
    """Causal grouped-query attention of one whole sequence.
    q [T, H, hd], k, v [T, Hkv, hd] -> [T, H, hd].  Query head h reads kv head
    h * Hkv // H; position t sees keys j <= t (and j > t - window if a window is given);
    s = (q . k) * scale, softmax, weighted sum of v.  C/ports/fused_ops.rs:486-530."""
    T, H, hd = q.shape
    Hkv = k.shape[1]
    out = np.zeros_like(q)
    j = np.arange(T)
    mask = j[None, :] <= j[:, None]
    if window is not None:
        mask &= j[None, :] > j[:, None] - window
    for h in range(H):
        g = h * Hkv // H
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = np.where(mask, s, -np.inf)
        out[:, h, :] = softmax(s) @ v[:, g, :]
    return out


def silu(z: np.ndarray) -> np.ndarray:
    """z / (1 + exp(-z)).  CPU:762-771."""
    return z / (1.0 + np.exp(-z))


def swiglu_mlp(x: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray) -> np.ndarray:
    """down( silu(gate(x)) * up(x) ), every projection x @ W^T.
    W/components/ffn_dense.rs:39-68."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def attention_block(x, w, prefix, cfg, positions, freqs):
    """q/k/v projections, rotation of q and k, attention, output projection.
    W/components/attention.rs:96-179; scale 1/sqrt(head_dim), W/models/decoder.rs:276."""
    H, Hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or cfg["hidden_size"] // H
    T = x.shape[0]
    q = (x @ w[prefix + "q_proj.weight"].T).reshape(T, H, hd)
    k = (x @ w[prefix + "k_proj.weight"].T).reshape(T, Hkv, hd)
    v = (x @ w[prefix + "v_proj.weight"].T).reshape(T, Hkv, hd)
    q, k = rope(q, positions, freqs), rope(k, positions, freqs)
    o = attention(q, k, v, 1.0 / math.sqrt(hd))
    return o.reshape(T, H * hd) @ w[prefix + "o_proj.weight"].T


def forward(cfg: dict, w: Dict[str, np.ndarray], ids, start_position: int = 0) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence.
    x <- x + attn(norm1(x)); x <- x + mlp(norm2(x)) per layer, then the final norm and the
    head (the embedding table when no lm_head.weight exists).
    W/models/decoder.rs:57-200 (order), :245-262 (tied head)."""
    H = cfg["num_attention_heads"]
    hd = cfg.get("head_dim") or cfg["hidden_size"] // H
    eps = cfg.get("rms_norm_eps", 1e-5)
    freqs = rope_frequencies(hd, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    T = len(ids)
    positions = np.arange(start_position, start_position + T)
    x = embedding(w["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        n = rmsnorm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_block(n, w, p + "self_attn.", cfg, positions, freqs)
        n = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu_mlp(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"])
    x = rmsnorm(x, w["model.norm.weight"], eps)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return x @ head.T


# ---------------------------------------------------------------------------
# sampling
# ---------------------------------------------------------------------------
def greedy(logits: np.ndarray) -> int:
    """Index of the largest logit, the lowest index on ties (CU/kernels/sampler/sampler.cu:65-78)."""
    return int(np.argmax(logits))


def filtered_distribution(logits: np.ndarray, temperature: float, top_k: int = 0,
                          top_p: float = 1.0, min_p: float = 0.0):
    """(token ids in order of descending logit, their weights) after the filters, as
    W/application/sampler_stack.rs:259-321: logits / T, sort descending, keep top_k,
    w = exp(l - max), drop w < w0 * min_p, keep the shortest prefix whose share of the total
    reaches top_p (at least one)."""
    l = np.asarray(logits, dtype=np.float64) / temperature
    l = np.where(np.isnan(l), -np.inf, l)
    order = np.argsort(-l, kind="stable")
    if top_k > 0:
        order = order[:min(top_k, len(order))]
    w = np.exp(l[order] - l[order[0]])
    if min_p > 0:
        keep = w >= w[0] * min_p
        order, w = order[keep], w[keep]
    if top_p < 1.0:
        c = np.cumsum(w / w.sum())
        n = int(np.searchsorted(c, top_p, side="left")) + 1
        n = max(1, min(n, len(w)))
        order, w = order[:n], w[:n]
    return order, w


def sample_from(order: np.ndarray, w: np.ndarray, u: float) -> int:
    """Walk the kept tokens with target u * sum(w).  sampler_stack.rs:323-334."""
    target = min(max(u, 0.0), 1.0 - 2.0 ** -52) * w.sum()
    sel = order[0]
    for tok, wt in zip(order, w):
        sel = tok
        if target < wt:
            break
        target -= wt
    return int(sel)


def sample_with_logprobs(logits: np.ndarray, temperature: float, top_k: int, top_p: float, min_p: float,
                         u: float, greedy_row: bool):
    """(token, ln p of it, [(token, ln p)] of the five most probable kept tokens).
    Greedy rows: argmax and the log-softmax of the raw logits there, no list
    (sampler_stack.rs:248-256, :353-365).  Else p = w / sum of the kept weights, and the list is
    the first five kept tokens in their order (sampler_stack.rs:335-350)."""
    if greedy_row:
        l = np.asarray(logits, dtype=np.float64)
        tok = greedy(l)
        return tok, float(l[tok] - l.max() - np.log(np.exp(l - l.max()).sum())), []
    order, w = filtered_distribution(logits, temperature, top_k, top_p, min_p)
    tok = sample_from(order, w, u)
    lp = np.log(w / w.sum())
    chosen = float(lp[list(order).index(tok)])
    return tok, chosen, [(int(t), float(x)) for t, x in zip(order[:5], lp[:5])]
