"""Reads and writes the safetensors container: 8 bytes little-endian header
length, a JSON header {name: {dtype, shape, data_offsets}}, then raw
little-endian tensor data.  Files are memory-mapped and tensors are taken out
one by one, so a large checkpoint never sits in host memory twice.

The reference reads GGUF the same way (mmap, tensor infos, data slices:
internal/gguf/reader.go:16-227) and reports truncated data
(internal/engine/engine.go:771-773); this is the same role for the file format
of config.json + model.safetensors folders.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Mapping, Tuple

import torch


class WeightFileError(ValueError):
    pass


_DTYPES = {
    "F32": torch.float32,
    "BF16": torch.bfloat16,
    "F16": torch.float16,
    "F64": torch.float64,
    "I32": torch.int32,
    "I64": torch.int64,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One .safetensors file, mapped read-only."""

    def __init__(self, path: str) -> None:
        self.path = path
        self._map = None
        size = os.path.getsize(path)
        if size < 8:
            raise WeightFileError(f"{path}: too short to be a safetensors file ({size} bytes)")
        self._f = open(path, "rb")
        try:
            self._read_header(size)
            self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        except BaseException:
            self._f.close()  # a rejected file leaves no handle behind
            raise

    def _read_header(self, size: int) -> None:
        path = self.path
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise WeightFileError(f"{path}: header length {hlen} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: header is not valid JSON ({e})") from e
        if not isinstance(header, dict):
            raise WeightFileError(f"{path}: header is not a JSON object")
        self.metadata = header.pop("__metadata__", {})
        self.data_start = 8 + hlen
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            try:
                dt = info.get("dtype")
                if dt not in _DTYPES:
                    raise WeightFileError(f"{path}: tensor {name!r} has unsupported dtype {dt!r}")
                shape = tuple(int(s) for s in info["shape"])
                begin, end = (int(o) for o in info["data_offsets"])
            except (KeyError, TypeError, ValueError, AttributeError) as e:
                raise WeightFileError(f"{path}: tensor {name!r} has a malformed header entry ({e!r})") from e
            n = 1
            for s in shape:
                n *= s
            want = n * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if end - begin != want:
                raise WeightFileError(
                    f"{path}: tensor {name!r} of shape {list(shape)} {dt} needs {want} bytes, header gives {end - begin}")
            if begin < 0 or self.data_start + end > size:
                raise WeightFileError(f"{path}: tensor {name!r} data truncated (ends at {self.data_start + end}, file has {size})")
            self.entries[name] = (_DTYPES[dt], shape, begin, end)

    def names(self) -> List[str]:
        return list(self.entries)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        dt, shape, _, _ = self.entries[name]
        return dt, shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that owns its memory (copied out of the map)."""
        dt, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=dt)
        raw = bytearray(self._map[self.data_start + begin : self.data_start + end])
        return torch.frombuffer(raw, dtype=dt).reshape(shape)

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._map = None
        self._f.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] = None) -> None:
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order: List[str] = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise WeightFileError(f"cannot write tensor {name!r} of dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)


def open_model_files(folder: str) -> List[SafetensorsFile]:
    """model.safetensors, or the shards that model.safetensors.index.json lists."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    if os.path.isfile(index):
        try:
            with open(index, "r", encoding="utf-8") as f:
                shards = sorted(set(json.load(f)["weight_map"].values()))
        except (KeyError, TypeError, AttributeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{index}: not an index with a weight_map ({e!r})") from e
        opened: List[SafetensorsFile] = []
        try:
            for s in shards:
                opened.append(SafetensorsFile(os.path.join(folder, s)))
        except BaseException:
            for f in opened:  # a later shard was refused: the earlier ones are closed again
                f.close()
            raise
        return opened
    raise WeightFileError(f"no model.safetensors (or model.safetensors.index.json) in {folder!r}")
