"""What one step looks like to the parts: the tokens of the batch, where each stands in
its request, and the tables that lead to its cache.

Counterpart of the reference's ``BatchPlan`` + ``KvIndexTensors``
(crates/infer-core/src/plan.rs:27-67, crates/infer-core/src/kv.rs:22-39), written to
the device once a step (crates/infer-worker/src/application/runtime/plan.rs:293-369).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch


class Workspace:
    """Named scratch buffers, allocated once at the largest row count seen and handed out
    as ``[rows, cols]`` views.  Buffers of one name are shared by all layers (the reference
    aliases eight logical buffers onto two slots, crates/infer-worker/src/domain/forward_scratch.rs:41-209;
    here each name has its own allocation)."""

    def __init__(self, device, min_rows: int = 0):
        self.device = device
        self.min_rows = int(min_rows)
        self._bufs: Dict[Tuple[str, int, torch.dtype], torch.Tensor] = {}
        self._frozen = False
        self._captured = False       # a graph has been captured at some time
        self._retired = []

    @property
    def frozen(self) -> bool:
        """Set while captured graphs rely on the buffers handed out so far."""
        return self._frozen

    @frozen.setter
    def frozen(self, on: bool) -> None:
        self._frozen = bool(on)
        self._captured = self._captured or self._frozen

    def get(self, name: str, rows: int, cols: int, dtype: torch.dtype) -> torch.Tensor:
        key = (name, cols, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.shape[0] < rows:
            cap = max(rows, self.min_rows, 1)
            if buf is not None:
                # A captured graph may still point into the old buffer: then it is kept, not freed
                # (else the allocator takes it back; work queued on it is ordered before any reuse).
                # Buffers grow by half at least, so that steps of slowly growing sizes do not
                # allocate, and with graphs keep, a buffer each.
                if self._captured:
                    self._retired.append(buf)
                cap = max(cap, buf.shape[0] + buf.shape[0] // 2)
            buf = torch.empty((cap, cols), device=self.device, dtype=dtype)
            self._bufs[key] = buf
        return buf[:rows]

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._bufs.values())


class StepContext:
    """Device tensors (int32) and host numbers of one step.

    token_ids[T]      the tokens, request after request; -(k+1) stands for device_tokens[k]
    positions[T]      absolute position of each token in its request (= where its key goes)
    row_of_token[T]   which request row a token belongs to (-1: padding, touches nothing)
    cu_q[B+1]         token offsets of the rows
    q_start[B]        position of a row's first token (= tokens already cached)
    kv_lens[B]        length of the request after this step
    state_slots[B]    the request's slot in state tensors
    want_rows[W]      flat token indices whose logits are wanted
    want_all_in_order (host) every token's logits are wanted, in the tokens' order
    single_tokens[B]  flat token indices of the rows of exactly one token, then -1 (steps with longer rows beside them)
    portion_rows[B]   the rows of several tokens, then -1
    num_portion       (host) their number, or an upper bound of it
    num_single        (host) rows of exactly one token, or an upper bound of their number
    portion_prefix    (host) no row of several tokens has more tokens cached before the step
    portion_kv_len    (host) no row of several tokens is longer than this after the step
    block_tables[g]   [B, max_blocks_g] page ids of group g (-1: given back)
    """

    __slots__ = ("num_tokens", "num_rows", "num_want", "token_ids", "positions", "row_of_token",
                 "cu_q", "q_start", "kv_lens", "state_slots", "want_rows", "block_tables",
                 "workspace", "max_q_len", "max_kv_len", "host_q_lens", "host_q_start",
                 "host_kv_lens", "host_slots", "request_ids", "decode_only", "device_tokens",
                 "want_all_in_order", "num_single", "portion_prefix", "portion_kv_len", "single_tokens", "portion_rows", "num_portion")

    def __init__(self):
        self.block_tables: List[torch.Tensor] = []
