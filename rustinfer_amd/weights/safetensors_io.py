"""Reader and writer for the safetensors container: 8-byte little-endian header
length, a JSON header ``{name: {dtype, shape, data_offsets}}``, then raw
little-endian data.  The reader memory-maps the file and hands out views by
tensor name (reference: crates/infer-worker/src/infrastructure/io/safetensors.rs:47-213).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch


class WeightError(ValueError):
    """A checkpoint that does not fit the model, or a file that is not readable."""


_DTYPES = {
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
    "U8": (torch.uint8, 1),
    "I8": (torch.int8, 1),
    "F64": (torch.float64, 8),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One memory-mapped ``.safetensors`` file."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except OSError as e:
            raise WeightError(f"{path}: cannot open: {e}") from None
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise WeightError(f"{path}: too short to be a safetensors file ({size} bytes)")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise WeightError(f"{path}: header length {hlen} exceeds the file size {size}")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightError(f"{path}: header is not valid JSON: {e}") from None
        self._data_start = 8 + hlen
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        self.metadata = header.pop("__metadata__", {}) or {}
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        data_size = size - self._data_start
        for name, info in header.items():
            try:
                dtype, shape = info["dtype"], tuple(int(s) for s in info["shape"])
                begin, end = (int(v) for v in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightError(f"{path}: malformed header entry for tensor '{name}'") from None
            if dtype not in _DTYPES:
                raise WeightError(f"{path}: tensor '{name}' has unsupported dtype {dtype}")
            numel = 1
            for s in shape:
                numel *= s
            want = numel * _DTYPES[dtype][1]
            if begin < 0 or end < begin or end > data_size or end - begin != want:
                raise WeightError(
                    f"{path}: tensor '{name}': byte range [{begin}, {end}) does not match "
                    f"shape {list(shape)} of {dtype} ({want} bytes) within {data_size} data bytes")
            self.entries[name] = (dtype, shape, begin, end)

    def names(self) -> List[str]:
        return list(self.entries)

    def __contains__(self, name: str) -> bool:
        return name in self.entries

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        dtype, shape, _, _ = self.entries[name]
        return _DTYPES[dtype][0], shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped bytes (read-only: clone before writing)."""
        if name not in self.entries:
            raise WeightError(f"{self.path}: tensor '{name}' not found")
        dtype, shape, begin, end = self.entries[name]
        tdtype = _DTYPES[dtype][0]
        if end == begin:
            return torch.empty(shape, dtype=tdtype)
        buf = memoryview(self._mm)[self._data_start + begin:self._data_start + end]
        raw = np.frombuffer(buf, dtype=np.uint8)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")       # numpy view is read-only; we never write
            t = torch.from_numpy(raw)
        return t.view(tdtype).reshape(shape)

    def close(self) -> None:
        # Views handed out keep the map alive through the buffer protocol.
        try:
            self._fh.close()
        except OSError:
            pass


class SafetensorsReader:
    """All tensors of a model folder: the shards that a ``*.safetensors.index.json`` names if
    the folder has one (any prefix, ``model.`` being the usual one), else ``model.safetensors``,
    else the folder's only ``*.safetensors`` file (safetensors.rs:62-153 looks in that order)."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        self._files: List[SafetensorsFile] = []
        self._where: Dict[str, SafetensorsFile] = {}
        try:
            found = sorted(os.listdir(model_dir))
        except OSError as e:
            raise WeightError(f"{model_dir}: {e.strerror or e}") from None
        indexes = [n for n in found if n.endswith(".safetensors.index.json")]
        singles = [n for n in found if n.endswith(".safetensors")]
        if indexes:
            if len(indexes) > 1 and "model.safetensors.index.json" not in indexes:
                raise WeightError(f"{model_dir}: several shard indexes ({', '.join(indexes)})")
            index = os.path.join(model_dir, "model.safetensors.index.json"
                                 if "model.safetensors.index.json" in indexes else indexes[0])
            try:
                with open(index, "r", encoding="utf-8") as f:
                    wm = json.load(f)["weight_map"]
                shards = sorted(set(wm.values()))
            except (OSError, KeyError, AttributeError, TypeError, json.JSONDecodeError) as e:
                raise WeightError(f"{index}: unreadable shard index: {e}") from None
            gone = [p for p in shards if not os.path.isfile(os.path.join(model_dir, p))]
            if gone:
                raise WeightError(f"{index} names shards that are not in the folder: {', '.join(gone)}")
            paths = [os.path.join(model_dir, p) for p in shards]
        elif "model.safetensors" in singles:
            paths = [os.path.join(model_dir, "model.safetensors")]
        elif len(singles) == 1:
            paths = [os.path.join(model_dir, singles[0])]
        elif singles:
            raise WeightError(f"{model_dir}: several .safetensors files ({', '.join(singles)}) and no "
                              f"*.safetensors.index.json that says which tensors each holds")
        else:
            raise WeightError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json found")
        for p in paths:
            f = SafetensorsFile(p)
            self._files.append(f)
            for n in f.names():
                if n in self._where:
                    raise WeightError(f"tensor '{n}' appears in both {self._where[n].path} and {p}")
                self._where[n] = f

    def names(self) -> List[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def info(self, name: str):
        return self._where[name].info(name)

    def tensor(self, name: str) -> torch.Tensor:
        if name not in self._where:
            raise WeightError(f"{self.model_dir}: tensor '{name}' not found")
        return self._where[name].tensor(name)


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] = None) -> None:
    """Write CPU tensors in the given order; data is aligned so offsets start at a multiple of 8."""
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise WeightError(f"tensor '{name}': dtype {t.dtype} cannot be stored")
        t = t.detach().cpu().contiguous()
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        blobs.append(t)
    hjson = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hjson += b" " * ((8 - len(hjson) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hjson)))
        f.write(hjson)
        for t in blobs:
            if t.numel():
                f.write(t.view(torch.uint8).reshape(-1).numpy().tobytes()
                        if t.numel() * t.element_size() < (1 << 28)
                        else memoryview(t.view(torch.uint8).reshape(-1).numpy()))
    os.replace(tmp, path)
