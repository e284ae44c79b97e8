"""Reading and writing safetensors files by tensor name.

The format: an 8-byte little-endian header length, a JSON header
{name: {dtype, shape, data_offsets}}, then the raw little-endian data.  The reader
maps the file and hands out zero-copy CPU tensors, the way the reference maps its
model file and binds tensors in place (/root/reference/internal/gguf/gguf.go:39-51,
/root/reference/internal/llm/model.go:162-201); its bounds check on each tensor's
data (/root/reference/internal/gguf/gguf.go:101-113) is kept.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass

import torch

_DTYPES = {
    "F32": (torch.float32, 4), "F16": (torch.float16, 2), "BF16": (torch.bfloat16, 2),
    "F64": (torch.float64, 8), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: tuple
    begin: int      # absolute file offsets
    end: int
    file: str


class SafetensorsFile:
    """One mapped .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: not a safetensors file (shorter than its header length field)")
        self._fh = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen > size - 8 or hlen > (100 << 20):
            raise SafetensorsError(f"{path}: header length {hlen} is out of range (truncated file?)")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: malformed header ({e})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: malformed header (not an object)")
        self.metadata = header.pop("__metadata__", None) or {}
        base = 8 + hlen
        self.entries: dict[str, TensorEntry] = {}
        for name, info in header.items():
            try:
                dtype, shape = info["dtype"], tuple(int(s) for s in info["shape"])
                b, e = (int(o) for o in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: tensor {name}: malformed header entry") from None
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name}: unsupported type {dtype}")
            count = 1
            for s in shape:
                count *= s
            if b < 0 or e < b or base + e > size:
                raise SafetensorsError(f"{path}: tensor {name}: data out of range (truncated file?)")
            if e - b != count * _DTYPES[dtype][1]:
                raise SafetensorsError(f"{path}: tensor {name}: {e - b} bytes do not hold shape "
                                       f"{list(shape)} of {dtype}")
            self.entries[name] = TensorEntry(name, dtype, shape, base + b, base + e, path)
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self):
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor over the mapped bytes (read-only: copy before writing)."""
        e = self.entries[name]
        dtype, width = _DTYPES[e.dtype]
        count = (e.end - e.begin) // width
        if count == 0:
            return torch.empty(e.shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")   # the buffer is not writable; it is never written
            flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=e.begin)
        return flat.reshape(e.shape)

    def close(self):
        # tensors handed out keep the map alive through the buffer protocol
        self._fh.close()


class Checkpoint:
    """All tensors of a model folder: model.safetensors, or the shards that
    model.safetensors.index.json lists."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        self.files: dict[str, SafetensorsFile] = {}
        self.where: dict[str, str] = {}
        if os.path.isfile(single):
            f = SafetensorsFile(single)
            self.files[single] = f
            for n in f.names():
                self.where[n] = single
        elif os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as fh:
                try:
                    weight_map = json.load(fh)["weight_map"]
                except (json.JSONDecodeError, KeyError, TypeError):
                    raise SafetensorsError(f"{index}: malformed index (no weight_map)") from None
            for name, shard in weight_map.items():
                path = os.path.join(model_dir, shard)
                if path not in self.files:
                    if not os.path.isfile(path):
                        raise SafetensorsError(f"{index}: shard {shard} is listed but absent")
                    self.files[path] = SafetensorsFile(path)
                if name not in self.files[path].entries:
                    raise SafetensorsError(f"{index}: tensor {name} is not in shard {shard}")
                self.where[name] = path
        else:
            raise SafetensorsError(f"{model_dir}: no model.safetensors (or model.safetensors.index.json) "
                                   "in the model folder")

    def names(self):
        return list(self.where)

    def entry(self, name: str) -> TensorEntry:
        return self.files[self.where[name]].entries[name]

    def tensor(self, name: str) -> torch.Tensor:
        return self.files[self.where[name]].tensor(name)


def write_safetensors(path: str, tensors: dict, metadata: dict | None = None) -> None:
    """Write CPU tensors to one file, in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name}: unsupported type {t.dtype}")
        raw = t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    hjson = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hjson += b" " * ((8 - len(hjson) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hjson)))
        f.write(hjson)
        for raw in blobs:
            f.write(raw)
    os.replace(tmp, path)
