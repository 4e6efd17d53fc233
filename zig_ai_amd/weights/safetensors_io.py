"""Reading and writing safetensors files without loading them whole.

Layout of a file: an unsigned 64-bit little-endian header length ``n``, ``n``
bytes of JSON mapping each tensor name to ``{"dtype", "shape", "data_offsets"}``,
then the data section; offsets count from the start of the data section, that
is from byte ``8 + n`` (the reference's own reader leaves the header length
out of that sum: /root/reference/src/loader/safetensors.zig:225-230).
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Mapping, Tuple

import torch


class SafetensorsError(ValueError):
    pass


_DTYPES = {
    "BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One memory-mapped file; tensors are views into the mapping."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: shorter than its 8-byte length prefix")
        self._file = open(path, "rb")
        # A private copy-on-write mapping: writable for torch, never written back.
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_COPY)
        (header_len,) = struct.unpack("<Q", self._map[:8])
        if 8 + header_len > size:
            raise SafetensorsError(
                f"{path}: header claims {header_len} bytes but the file has {size}")
        try:
            header = json.loads(self._map[8:8 + header_len].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from e
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not a JSON object")
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + header_len
        data_size = size - self._data_start
        self.entries: Dict[str, dict] = {}
        for name, info in header.items():
            try:
                dtype, shape = info["dtype"], [int(s) for s in info["shape"]]
                begin, end = (int(v) for v in info["data_offsets"])
            except (KeyError, TypeError, ValueError) as e:
                raise SafetensorsError(f"{path}: malformed entry for {name!r}") from e
            if not 0 <= begin <= end <= data_size:
                raise SafetensorsError(
                    f"{path}: tensor {name!r} spans bytes {begin}..{end} of a {data_size}-byte "
                    "data section (file truncated?)")
            self.entries[name] = {"dtype": dtype, "shape": tuple(shape), "begin": begin, "end": end}

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name]["shape"]

    def dtype_name(self, name: str) -> str:
        return self.entries[name]["dtype"]

    def tensor(self, name: str) -> torch.Tensor:
        e = self.entries[name]
        if e["dtype"] not in _DTYPES:
            raise SafetensorsError(f"{self.path}: tensor {name!r} has unsupported dtype {e['dtype']}")
        dtype = _DTYPES[e["dtype"]]
        count = 1
        for s in e["shape"]:
            count *= s
        itemsize = torch.empty((), dtype=dtype).element_size()
        if count * itemsize != e["end"] - e["begin"]:
            raise SafetensorsError(
                f"{self.path}: tensor {name!r} of shape {e['shape']} and dtype {e['dtype']} "
                f"needs {count * itemsize} bytes but spans {e['end'] - e['begin']}")
        if count == 0:
            return torch.empty(e["shape"], dtype=dtype)
        flat = torch.frombuffer(self._map, dtype=dtype, count=count,
                                offset=self._data_start + e["begin"])
        return flat.view(e["shape"])

    def close(self) -> None:
        # Views handed out keep the mapping alive; closing the descriptor is safe.
        self._file.close()


class Checkpoint:
    """All tensors of a model folder: ``model.safetensors``, or the shards that
    ``model.safetensors.index.json`` lists."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.isfile(single):
            f = SafetensorsFile(single)
            self._files[single] = f
            for n in f.names():
                self._where[n] = single
        elif os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as fh:
                weight_map = json.load(fh).get("weight_map", {})
            for n, shard in weight_map.items():
                path = os.path.join(model_dir, shard)
                if path not in self._files:
                    if not os.path.isfile(path):
                        raise SafetensorsError(f"{index} names {shard}, which does not exist")
                    self._files[path] = SafetensorsFile(path)
                if n not in self._files[path].entries:
                    raise SafetensorsError(f"{index} places {n!r} in {shard}, which lacks it")
                self._where[n] = path
        else:
            raise SafetensorsError(
                f"{model_dir} holds neither model.safetensors nor model.safetensors.index.json")

    def names(self) -> Iterable[str]:
        return self._where.keys()

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._files[self._where[name]].shape(name)

    def dtype_name(self, name: str) -> str:
        return self._files[self._where[name]].dtype_name(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._files[self._where[name]].tensor(name)


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor],
                      metadata: Mapping[str, str] | None = None) -> None:
    """Write ``tensors`` (CPU, any supported dtype) in the order given."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot write {name!r} of dtype {t.dtype}")
        t = t.detach().cpu().contiguous()
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        blobs.append(t)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * ((8 - len(text) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for t in blobs:
            if t.numel():
                f.write(memoryview(t.reshape(-1).view(torch.uint8).numpy()))
