"""Reading and writing safetensors files by tensor name.

Format (as the reference parses it, model/src/qwen3_checkpoint.cpp:114-149): an
8-byte little-endian header length, a JSON header mapping each tensor name to
``dtype``, ``shape`` and ``data_offsets [begin, end)`` relative to the end of
the header, an optional ``__metadata__`` entry, then the raw little-endian
data.  A folder holds either one ``model.safetensors`` or several shards named
by the ``weight_map`` of ``model.safetensors.index.json``
(model/src/qwen3_checkpoint.cpp:61-91).  Files are memory-mapped; a tensor's
bytes are touched only when it is asked for.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch


class WeightFileError(ValueError):
    """A safetensors file or its index is malformed."""


_DTYPES = {
    "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2), "F32": (torch.float32, 4),
    "F64": (torch.float64, 8), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except OSError as exc:
            raise WeightFileError(f"cannot open weight file {path}: {exc.strerror}") from None
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise WeightFileError(f"{path}: too short for a safetensors header")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen > size - 8:
            raise WeightFileError(f"{path}: header length {hlen} exceeds file size {size}")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as exc:
            raise WeightFileError(f"{path}: header is not valid JSON ({exc})") from None
        self._data_start = 8 + hlen
        self._data_len = size - self._data_start
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                dtype, shape = info["dtype"], tuple(int(s) for s in info["shape"])
                begin, end = (int(x) for x in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightFileError(f"{path}: malformed header entry for '{name}'") from None
            if dtype not in _DTYPES:
                raise WeightFileError(f"{path}: tensor '{name}' has unsupported dtype {dtype}")
            count = 1
            for s in shape:
                count *= s
            if begin < 0 or end < begin or end > self._data_len:
                raise WeightFileError(f"{path}: tensor '{name}' has data offsets [{begin}, {end}) "
                                      f"outside the file's {self._data_len} data bytes")
            if end - begin != count * _DTYPES[dtype][1]:
                raise WeightFileError(f"{path}: tensor '{name}' of shape {list(shape)} and dtype "
                                      f"{dtype} does not fill its {end - begin} bytes")
            self.entries[name] = (dtype, shape, begin, end)

    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name][0]][0]

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (read-only memory: copy or
        convert it before writing)."""
        dtype, shape, begin, end = self.entries[name]
        tdtype = _DTYPES[dtype][0]
        if end == begin:
            return torch.empty(shape, dtype=tdtype)
        buf = memoryview(self._map)[self._data_start + begin:self._data_start + end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # non-writable buffer
            flat = torch.frombuffer(buf, dtype=tdtype)
        return flat.reshape(shape)

    def close(self) -> None:
        # tensors returned by read() keep the mapping alive through their buffer
        self._fh.close()


class Checkpoint:
    """All tensors of a model folder, by name, over one or several files."""

    def __init__(self, model_path: str):
        folder = model_path if os.path.isdir(model_path) else os.path.dirname(model_path)
        self.folder = folder
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        index = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        if not os.path.isdir(model_path):
            self._add_file(model_path)
        elif os.path.exists(index):
            try:
                with open(index, "r", encoding="utf-8") as fh:
                    weight_map = json.load(fh)["weight_map"]
                assert isinstance(weight_map, dict)
            except (json.JSONDecodeError, KeyError, AssertionError):
                raise WeightFileError(f"{index}: no valid 'weight_map'") from None
            for shard in sorted(set(weight_map.values())):
                self._add_file(os.path.join(folder, shard))
            for name, shard in weight_map.items():
                f = self._files[os.path.join(folder, shard)]
                if name not in f.entries:
                    raise WeightFileError(f"{index}: tensor '{name}' is not in shard {shard}")
        elif os.path.exists(single):
            self._add_file(single)
        else:
            raise WeightFileError(f"{folder} holds neither model.safetensors nor "
                                  f"model.safetensors.index.json")

    def _add_file(self, path: str) -> None:
        f = SafetensorsFile(path)
        self._files[path] = f
        for name in f.names():
            self._where.setdefault(name, path)

    def names(self) -> List[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._files[self._where[name]].shape(name)

    def dtype(self, name: str) -> torch.dtype:
        return self._files[self._where[name]].dtype(name)

    def read(self, name: str) -> torch.Tensor:
        return self._files[self._where[name]].read(name)

    def close(self) -> None:
        for f in self._files.values():
            f.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]]) -> None:
    """Write (name, tensor) pairs to one safetensors file.  The iterable is
    walked twice if it is a list/dict items; a generator is materialised one
    tensor at a time into a temporary data file so that large models need
    little memory."""
    header: Dict[str, dict] = {}
    offset = 0
    tmp = path + ".data.tmp"
    with open(tmp, "wb") as data:
        for name, t in tensors:
            if t.dtype not in _NAMES:
                raise WeightFileError(f"cannot store dtype {t.dtype} of '{name}'")
            t = t.detach().cpu().contiguous()
            nbytes = t.numel() * t.element_size()
            if nbytes:
                data.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                           t.reshape(1).view(torch.uint8).numpy().tobytes())
            header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                            "data_offsets": [offset, offset + nbytes]}
            offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as out, open(tmp, "rb") as data:
        out.write(struct.pack("<Q", len(blob)))
        out.write(blob)
        while True:
            chunk = data.read(1 << 24)
            if not chunk:
                break
            out.write(chunk)
    os.remove(tmp)
