"""Launch configuration: one TOML file, every field defaulted, unknown keys refused.

Names and meanings follow the reference's ``RustInferConfig``
(crates/infer-protocol/src/config.rs:53-195, defaults :197-262, checks :281-344).
Fields that only its HTTP server, its scheduler process or tensor parallelism read
are accepted and ignored so that an existing launch file still loads.
"""
from __future__ import annotations

from dataclasses import dataclass, field, fields
from typing import Any, Dict, List, Tuple

from .model_config import ConfigError

# Keys of the reference's file that have no meaning in a single-process engine.
_IGNORED_KEYS = {
    "model_name", "cluster_id", "host", "port", "request_timeout_secs",
    "tp_operation_timeout_secs", "tp_startup_timeout_secs",
    "worker_heartbeat_timeout_secs", "max_inflight_requests", "batch_wait_ms",
    "worker_id", "cuda_memory",
}


@dataclass
class EngineConfig:
    model: str = ""                          # model folder (config.json + model.safetensors)
    device: str = "cuda:0"
    dtype: str = "bfloat16"                  # "bfloat16" | "float32" (not in the reference: it is bf16 only)
    max_batch_tokens: int = 8192             # tokens per step
    max_batch_seqs: int = 32                 # live requests
    max_model_len: int = 4096                # prompt + generation
    paged_block_size: int = 16               # tokens per KV page (the reference only runs 1)
    chunked_prefill_size: int = 0            # 0 = prompts are cut only by the token budget
    max_prefill_seqs_per_iter: int = 0       # 0 = unlimited
    prefill_sjf: bool = False                # shortest prompt first instead of FCFS
    enable_prefix_caching: bool = False      # must stay false: no prefix cache here
    mem_fraction_static: float = 0.9
    num_blocks: int = 0                      # KV pages; 0 = size from free memory
    ignore_eos: bool = False
    mode: str = "llm"
    tensor_parallel_size: int = 1
    log_level: str = "info"
    capture_sizes: Tuple[int, ...] = (1, 2, 4, 8, 16, 24, 32, 40, 48, 56, 64)
    random_weights_seed: int = -1            # >= 0: `model` needs only config.json, weights are drawn from this seed
    gemm_tune: bool = False                  # time the GEMM library's kernels for each shape of many rows once and keep the fastest
    mixed_graph_tokens: int = -1             # steps with prompt portions of up to this many tokens replay graphs too (0: they launch eagerly;
                                             # -1: up to 1024 where launching a step costs the host more time than its kernels take, else 0;
                                             # the reference's switch is RUSTINFER_MIXED_GRAPH, crates/infer-worker/src/application/runtime/mod.rs:426-440)
    mixed_graph_after: int = 2               # a shape of such a step is captured the n-th time it is met (a capture costs ten such steps)
    tiled_weight_copy: bool = True           # a second copy of every projection weight in the order the few-row kernels stream it
                                             # (false: half the memory for weights, slower single-token steps); not in the reference
    tiled_weight_reserve: float = 0.25       # with `num_blocks = 0`: the share of the device's memory that the second copies leave to the
                                             # cache; a model that fills most of the device keeps second copies of its first layers only
    step_token_align: int = 256              # a step up to an eighth of this over a multiple of it gives the tokens over back to a prompt
                                             # portion that is not its prompt's last (0: never); not in the reference
    prewarm_graphs: bool = False             # capture the graphs of every capture size and key-length bucket at start-up
                                             # (crates/infer-worker/src/application/runtime/graph_exec.rs:149-247) instead of when first met

    def validate(self) -> None:
        if not self.model.strip():
            raise ConfigError("`model` is required")
        if self.tensor_parallel_size != 1:
            raise ConfigError("`tensor_parallel_size` must be 1: this engine runs on one GPU")
        if not (0.0 < self.mem_fraction_static <= 1.0):
            raise ConfigError(f"`mem_fraction_static` must be in (0, 1], got {self.mem_fraction_static}")
        for key in ("max_model_len", "max_batch_tokens", "max_batch_seqs", "paged_block_size"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"`{key}` must be > 0")
        if self.random_weights_seed < -1:
            raise ConfigError("`random_weights_seed` must be >= 0 (or -1: load the checkpoint)")
        for key in ("chunked_prefill_size", "max_prefill_seqs_per_iter", "num_blocks", "step_token_align"):
            if getattr(self, key) < 0:
                raise ConfigError(f"`{key}` must be >= 0")
        if not (0.0 <= self.tiled_weight_reserve < 1.0):
            raise ConfigError(f"`tiled_weight_reserve` must be in [0, 1), got {self.tiled_weight_reserve}")
        if self.mixed_graph_after < 1:
            raise ConfigError("`mixed_graph_after` must be >= 1")
        if self.mixed_graph_tokens < -1:
            raise ConfigError("`mixed_graph_tokens` must be >= 0 (or -1: decided from the model's size)")
        if self.mode != "llm":
            raise ConfigError(f"`mode` must be \"llm\", got {self.mode!r}")
        if self.enable_prefix_caching:
            raise ConfigError("`enable_prefix_caching` must be false: there is no prefix cache")
        if self.dtype not in ("bfloat16", "float32"):
            raise ConfigError(f"`dtype` must be \"bfloat16\" or \"float32\", got {self.dtype!r}")
        if not self.device.startswith("cuda"):
            raise ConfigError(f"`device` must name a GPU as \"cuda:N\", got {self.device!r}")
        if any((not isinstance(c, int)) or c <= 0 for c in self.capture_sizes):
            raise ConfigError("`capture_sizes` must hold positive integers")

    @staticmethod
    def from_dict(d: Dict[str, Any], where: str = "config") -> "EngineConfig":
        known = {f.name: f for f in fields(EngineConfig)}
        kwargs: Dict[str, Any] = {}
        unknown = []
        for key, value in d.items():
            if key in _IGNORED_KEYS:
                continue
            if key not in known:
                unknown.append(key)
                continue
            default = known[key].default
            if isinstance(default, bool):
                ok = isinstance(value, bool)
            elif isinstance(default, int):
                ok = isinstance(value, int) and not isinstance(value, bool)
            elif isinstance(default, float):
                ok = isinstance(value, (int, float)) and not isinstance(value, bool)
                value = float(value) if ok else value
            elif isinstance(default, str):
                ok = isinstance(value, str)
            else:  # capture_sizes
                ok = isinstance(value, (list, tuple))
                value = tuple(value) if ok else value
            if not ok:
                raise ConfigError(f"{where}: `{key}` has the wrong type: {value!r}")
            kwargs[key] = value
        if unknown:
            raise ConfigError(f"{where}: unknown keys: {', '.join(sorted(unknown))}")
        cfg = EngineConfig(**kwargs)
        try:
            cfg.validate()
        except ConfigError as e:
            raise ConfigError(f"{where}: {e}") from None
        return cfg


def load_engine_config(path: str) -> EngineConfig:
    try:
        with open(path, "r", encoding="utf-8") as f:
            text = f.read()
    except OSError as e:
        raise ConfigError(f"read config {path}: {e}") from None
    return EngineConfig.from_dict(parse_toml(text, path), where=f"config {path}")


# ---------------------------------------------------------------------------
# The subset of TOML that launch files use: `key = value` lines, [table]
# headers, strings, integers, floats, booleans and flat arrays, # comments.
# ---------------------------------------------------------------------------

def _strip_comment(line: str) -> str:
    out, quote = [], None
    for ch in line:
        if quote:
            out.append(ch)
            if ch == quote:
                quote = None
        elif ch in "\"'":
            quote = ch
            out.append(ch)
        elif ch == "#":
            break
        else:
            out.append(ch)
    return "".join(out).strip()


def _parse_value(text: str, where: str):
    text = text.strip()
    if not text:
        raise ConfigError(f"{where}: missing value")
    if text[0] in "\"'":
        if len(text) < 2 or text[-1] != text[0]:
            raise ConfigError(f"{where}: unterminated string {text!r}")
        body = text[1:-1]
        if text[0] == '"':
            body = body.replace('\\"', '"').replace("\\\\", "\\").replace("\\n", "\n").replace("\\t", "\t")
        return body
    if text == "true":
        return True
    if text == "false":
        return False
    if text[0] == "[":
        if text[-1] != "]":
            raise ConfigError(f"{where}: unterminated array {text!r}")
        inner = text[1:-1].strip()
        if not inner:
            return []
        parts, depth, quote, cur = [], 0, None, []
        for ch in inner:
            if quote:
                cur.append(ch)
                if ch == quote:
                    quote = None
            elif ch in "\"'":
                quote = ch
                cur.append(ch)
            elif ch == "[":
                depth += 1
                cur.append(ch)
            elif ch == "]":
                depth -= 1
                cur.append(ch)
            elif ch == "," and depth == 0:
                parts.append("".join(cur))
                cur = []
            else:
                cur.append(ch)
        if "".join(cur).strip():
            parts.append("".join(cur))
        return [_parse_value(p, where) for p in parts]
    num = text.replace("_", "")
    try:
        return int(num, 0) if not any(c in num for c in ".eE") or num.lower().startswith("0x") else float(num)
    except ValueError:
        try:
            return float(num)
        except ValueError:
            raise ConfigError(f"{where}: cannot parse value {text!r}") from None


def parse_toml(text: str, where: str = "toml") -> Dict[str, Any]:
    root: Dict[str, Any] = {}
    table = root
    pending = None  # (key, text so far) of an array that spans several lines
    for lineno, raw in enumerate(text.splitlines(), 1):
        line = _strip_comment(raw)
        if not line:
            continue
        loc = f"{where}:{lineno}"
        if pending is not None:
            pending = (pending[0], pending[1] + " " + line)
            if pending[1].count("[") == pending[1].count("]"):
                table[pending[0]] = _parse_value(pending[1], loc)
                pending = None
            continue
        if line.startswith("["):
            if not line.endswith("]") or line.startswith("[["):
                raise ConfigError(f"{loc}: unsupported table header {line!r}")
            table = root
            for name in line[1:-1].strip().split("."):
                name = name.strip()
                if not name:
                    raise ConfigError(f"{loc}: empty table name")
                table = table.setdefault(name, {})
                if not isinstance(table, dict):
                    raise ConfigError(f"{loc}: {name!r} is both a value and a table")
            continue
        if "=" not in line:
            raise ConfigError(f"{loc}: expected `key = value`, got {line!r}")
        key, value = line.split("=", 1)
        key = key.strip().strip('"')
        if not key:
            raise ConfigError(f"{loc}: empty key")
        if key in table:
            raise ConfigError(f"{loc}: duplicate key {key!r}")
        value = value.strip()
        if value.startswith("[") and value.count("[") != value.count("]"):
            pending = (key, value)
            continue
        table[key] = _parse_value(value, loc)
    if pending is not None:
        raise ConfigError(f"{where}: unterminated array for key {pending[0]!r}")
    return root
