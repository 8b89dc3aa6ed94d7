"""Reading and writing safetensors files without loading them whole.

File layout: 8 bytes little-endian header length N, N bytes of JSON
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`, then the
raw little-endian tensor data.  The reader maps the file and hands out tensors that view the
mapping, so a checkpoint of many GB costs no host memory until a tensor is copied to the GPU.
(The reference reads the same files with `safetensors.torch.load_file`,
serve/hf_utils/convert_hf_checkpoint.py:9,123.)
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One mapped `.safetensors` file."""

    def __init__(self, path: str):
        self.path = path
        self._file = open(path, "rb")
        head = self._file.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", head)
        size = os.fstat(self._file.fileno()).st_size
        if n <= 0 or 8 + n > size:
            raise ValueError(f"{path}: header length {n} does not fit the file size {size}")
        header = json.loads(self._file.read(n).decode("utf-8"))
        header.pop("__metadata__", None)
        self._base = 8 + n
        self._entries: Dict[str, dict] = header
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        for name, e in header.items():
            if e["dtype"] not in _DTYPES:
                raise ValueError(f"{path}: tensor {name!r} has the unsupported dtype {e['dtype']}")
            b, end = e["data_offsets"]
            if not (0 <= b <= end and self._base + end <= size):
                raise ValueError(f"{path}: tensor {name!r} lies outside the file")

    def names(self) -> List[str]:
        return list(self._entries)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        e = self._entries[name]
        return _DTYPES[e["dtype"]], tuple(e["shape"])

    def read(self, name: str) -> torch.Tensor:
        e = self._entries[name]
        dtype, shape = _DTYPES[e["dtype"]], tuple(e["shape"])
        b, end = e["data_offsets"]
        count = 1
        for s in shape:
            count *= s
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        if (end - b) != count * torch.empty((), dtype=dtype).element_size():
            raise ValueError(f"{self.path}: tensor {name!r}: {end - b} bytes do not match shape {shape}")
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")      # the mapping is read-only; the tensor is only read
            t = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._base + b)
        return t.view(shape)


class CheckpointReader:
    """All tensors of a model folder: `model.safetensors`, or the shards that
    `model.safetensors.index.json` lists (serve/hf_utils/convert_hf_checkpoint.py:70-96)."""

    def __init__(self, folder: str):
        self.folder = folder
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        if os.path.isfile(single):
            files = [single]
        elif os.path.isfile(index):
            with open(index) as f:
                shard_names = sorted(set(json.load(f)["weight_map"].values()))
            files = [os.path.join(folder, s) for s in shard_names]
        else:
            raise FileNotFoundError(f"{folder}: neither model.safetensors nor model.safetensors.index.json found")
        self._files = [SafetensorsFile(p) for p in files]
        self._where: Dict[str, SafetensorsFile] = {}
        for sf in self._files:
            for name in sf.names():
                self._where[name] = sf

    def names(self) -> List[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def info(self, name: str):
        return self._where[name].info(name)

    def read(self, name: str) -> torch.Tensor:
        return self._where[name].read(name)


class DictReader:
    """The same interface over tensors held in memory."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self._t = tensors

    def names(self) -> List[str]:
        return list(self._t)

    def __contains__(self, name: str) -> bool:
        return name in self._t

    def info(self, name: str):
        t = self._t[name]
        return t.dtype, tuple(t.shape)

    def read(self, name: str) -> torch.Tensor:
        return self._t[name]


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write tensors in the order given.  They are streamed: one tensor in memory at a time
    when `tensors` is a generator."""
    items = []
    header: Dict[str, dict] = {}
    offset = 0
    tmp = path + ".tmp"
    with open(tmp, "wb") as data:
        for name, t in tensors:
            if t.dtype not in _NAMES:
                raise ValueError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
            t = t.detach().cpu().contiguous()
            raw = t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
            header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                            "data_offsets": [offset, offset + len(raw)]}
            data.write(raw)
            offset += len(raw)
            items.append(name)
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
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
