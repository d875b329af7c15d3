"""Reading and writing safetensors files.

Layout: 8-byte little-endian header length, a JSON header (tensor name -> dtype, shape,
data_offsets relative to the end of the header), then the data.  The reader rejects what the
reference's reader rejects (rust/checkpoint/src/safetensors.rs:46-154): a truncated or oversized
header, a header that is no object, bad shapes, `start > end`, a byte count that does not match
shape x dtype, data past the end of the file, overlapping tensors, gaps and trailing bytes.
Sharded checkpoints are resolved through `model.safetensors.index.json` (safetensors.rs:156-264).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


_DTYPES = {
    # name: (bytes per element, numpy dtype used to map the bytes, torch dtype of the view)
    "F64": (8, np.float64, torch.float64),
    "F32": (4, np.float32, torch.float32),
    "F16": (2, np.float16, torch.float16),
    "BF16": (2, np.uint16, torch.bfloat16),
    "I64": (8, np.int64, torch.int64),
    "I32": (4, np.int32, torch.int32),
    "I16": (2, np.int16, torch.int16),
    "I8": (1, np.int8, torch.int8),
    "U8": (1, np.uint8, torch.uint8),
    "BOOL": (1, np.uint8, torch.bool),
}
_TORCH_TO_NAME = {torch.float64: "F64", torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
                  torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8",
                  torch.uint8: "U8", torch.bool: "BOOL"}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    start: int       # byte offsets inside the file
    end: int


class SafetensorsFile:
    """One mapped file; `tensor(name)` gives a read-only CPU tensor that views the mapping."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: truncated header")
        with open(path, "rb") as fh:
            (header_len,) = struct.unpack("<Q", fh.read(8))
            if header_len > size - 8:
                raise SafetensorsError(f"{path}: header runs past the end of the file")
            try:
                header = json.loads(fh.read(header_len).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as exc:
                raise SafetensorsError(f"{path}: header is not valid JSON: {exc}") from None
            self._map = mmap.mmap(fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not a JSON object")
        base = 8 + header_len
        data_len = size - base
        self.metadata = header.pop("__metadata__", None)
        entries: Dict[str, TensorEntry] = {}
        spans: List[Tuple[int, int, str]] = []
        for name, info in header.items():
            if not isinstance(info, dict):
                raise SafetensorsError(f"{path}: entry {name!r} is not an object")
            dtype = info.get("dtype")
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dtype!r}")
            shape = info.get("shape")
            if not isinstance(shape, list) or any(not isinstance(d, int) or isinstance(d, bool) or d < 0 for d in shape):
                raise SafetensorsError(f"{path}: tensor {name!r} has an invalid shape {shape!r}")
            offs = info.get("data_offsets")
            if (not isinstance(offs, list) or len(offs) != 2
                    or any(not isinstance(o, int) or isinstance(o, bool) or o < 0 for o in offs)):
                raise SafetensorsError(f"{path}: tensor {name!r} has invalid data_offsets {offs!r}")
            start, end = offs
            if start > end:
                raise SafetensorsError(f"{path}: tensor {name!r} has start > end")
            count = 1
            for d in shape:
                count *= d
            if end - start != count * _DTYPES[dtype][0]:
                raise SafetensorsError(f"{path}: tensor {name!r} holds {end - start} bytes, "
                                       f"shape {shape} of {dtype} needs {count * _DTYPES[dtype][0]}")
            if end > data_len:
                raise SafetensorsError(f"{path}: tensor {name!r} runs past the end of the file")
            entries[name] = TensorEntry(name, dtype, tuple(shape), base + start, base + end)
            spans.append((start, end, name))
        spans.sort()
        cursor = 0
        for start, end, name in spans:
            if start < cursor:
                raise SafetensorsError(f"{path}: tensor {name!r} overlaps another tensor")
            if start > cursor:
                raise SafetensorsError(f"{path}: gap of {start - cursor} bytes before tensor {name!r}")
            cursor = end
        if cursor != data_len:
            raise SafetensorsError(f"{path}: {data_len - cursor} trailing bytes after the last tensor")
        self.entries = entries

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def tensor(self, name: str) -> torch.Tensor:
        e = self.entries[name]
        _, np_dtype, torch_dtype = _DTYPES[e.dtype]
        count = 1
        for d in e.shape:
            count *= d
        if count == 0:
            return torch.empty(e.shape, dtype=torch_dtype)
        arr = np.frombuffer(self._map, dtype=np_dtype, count=count, offset=e.start)
        t = _readonly_view(arr) if arr.flags.aligned else torch.from_numpy(arr.copy())
        if torch_dtype != t.dtype:
            t = t.view(torch_dtype)
        return t.reshape(e.shape)


def _readonly_view(arr: np.ndarray) -> torch.Tensor:
    # torch warns about non-writable arrays; the mapping is never written through this view
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        return torch.from_numpy(arr)


def _plain_file_name(name: str) -> bool:
    return bool(name) and name not in (".", "..") and "/" not in name and "\\" not in name and "\0" not in name


def open_checkpoint(model_dir: str) -> Dict[str, Tuple[SafetensorsFile, str]]:
    """All tensors of a checkpoint folder: name -> (file, name).  Uses the shard index when there
    is one, else `model.safetensors`, else every `*.safetensors` in sorted order; a tensor held
    by two files is an error."""
    index_path = os.path.join(model_dir, "model.safetensors.index.json")
    found: Dict[str, Tuple[SafetensorsFile, str]] = {}
    if os.path.isfile(index_path):
        with open(index_path, "r", encoding="utf-8") as fh:
            index = json.load(fh)
        weight_map = index.get("weight_map") if isinstance(index, dict) else None
        if not isinstance(weight_map, dict) or not weight_map:
            raise SafetensorsError(f"{index_path}: weight_map is missing or empty")
        by_shard: Dict[str, List[str]] = {}
        for tensor_name, shard in weight_map.items():
            if not isinstance(shard, str) or not _plain_file_name(shard):
                raise SafetensorsError(f"{index_path}: shard name {shard!r} is not a plain file name")
            by_shard.setdefault(shard, []).append(tensor_name)
        for shard in sorted(by_shard):
            path = os.path.join(model_dir, shard)
            if not os.path.isfile(path) or os.path.islink(path) and not os.path.realpath(path).startswith(
                    os.path.realpath(model_dir) + os.sep):
                raise SafetensorsError(f"{index_path}: shard {shard!r} is not a regular file inside the folder")
            f = SafetensorsFile(path)
            if set(f.names()) != set(by_shard[shard]):
                raise SafetensorsError(f"{path}: tensors differ from those the index lists for this shard")
            for n in f.names():
                found[n] = (f, n)
        return found
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        files = [single]
    else:
        files = sorted(os.path.join(model_dir, n) for n in os.listdir(model_dir) if n.endswith(".safetensors"))
        if not files:
            raise SafetensorsError(f"{model_dir}: no safetensors file found")
    for path in files:
        f = SafetensorsFile(path)
        for n in f.names():
            if n in found:
                raise SafetensorsError(f"tensor {n!r} is held by both {found[n][0].path} and {path}")
            found[n] = (f, n)
    return found


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor]) -> None:
    """Writes CPU tensors in the given order, contiguous, no gaps."""
    header: Dict[str, dict] = {}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _TORCH_TO_NAME:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TORCH_TO_NAME[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        blobs.append(t)
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(raw)))
        fh.write(raw)
        for t in blobs:
            if t.numel():
                fh.write(t.view(torch.uint8).reshape(-1).numpy().tobytes() if t.dtype != torch.bool
                         else t.to(torch.uint8).numpy().tobytes())
