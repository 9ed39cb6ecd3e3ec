"""Per-request sampling parameters; names, defaults and the greedy rule follow the
reference's ``SamplingParams`` (crates/infer-core/src/ports/sampler.rs:17-47) and its checks
(crates/infer-worker/src/application/sampler_stack.rs:221-240)."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0            # 0 = greedy
    top_k: int = 0                      # 0 (or negative) = off
    top_p: float = 1.0                  # 1 = off
    min_p: float = 0.0                  # 0 = off
    repetition_penalty: float = 1.0     # anything else is refused, as in the reference
    seed: Optional[int] = None          # None = a fresh seed for each request
    max_tokens: int = 2048              # crates/infer-protocol/src/server_to_scheduler.rs:126-137
    ignore_eos: bool = False
    # token sequences that end a request when its output ends with one of them; the matched tokens
    # are taken off the output (crates/infer-scheduler/src/domain/inference_session/table.rs:541-560)
    stop_sequences: Tuple[Tuple[int, ...], ...] = ()
    logprobs: bool = False              # ln p of each generated token and of the five most probable (the reference's want_logprobs)

    @property
    def is_greedy(self) -> bool:
        return self.temperature <= 0.0 or self.top_k == 1 or self.top_p <= 0.0

    def validate(self) -> None:
        if not math.isfinite(self.temperature) or self.temperature < 0.0:
            raise ValueError("sampling temperature must be finite and non-negative")
        if not math.isfinite(self.top_p) or not (0.0 <= self.top_p <= 1.0):
            raise ValueError("sampling top_p must be in [0, 1]")
        if not math.isfinite(self.min_p) or not (0.0 <= self.min_p <= 1.0):
            raise ValueError("sampling min_p must be in [0, 1]")
        if self.repetition_penalty != 1.0:
            raise ValueError("repetition-penalty sampling is not supported")
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be > 0")
        for stop in self.stop_sequences:
            if isinstance(stop, (str, bytes)) or not all(isinstance(t, int) for t in stop):
                raise ValueError("stop_sequences are sequences of token ids")
