"""Reading and writing safetensors files.

The container is an 8-byte little-endian header length, a JSON header
``{name: {dtype, shape, data_offsets}}`` and the raw little-endian data, with offsets
counted from the end of the header (src/safetensors.rs:56-79).  Files are mapped,
not read: a tensor is a view of the mapping until it is copied to the device.  A
folder holds either ``model.safetensors`` or shards named by
``model.safetensors.index.json`` (src/safetensors.rs:157-174).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from dataclasses import dataclass

import torch

from ..errors import UnsupportedError, WeightsError

# safetensors dtype names (src/dtype.rs:32-44) that this library stores; sizes in bytes
_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


@dataclass(frozen=True)
class TensorInfo:
    dtype: torch.dtype | None   # None: stored in a format this library does not read (see stored_as)
    shape: tuple
    start: int      # byte offsets into the file
    end: int
    stored_as: str = ""         # the file's own name of the dtype


class SafeTensorFile:
    """One mapped safetensors file."""

    def __init__(self, path: str):
        self.path = path
        try:
            with open(path, "rb") as f:
                size = os.fstat(f.fileno()).st_size
                if size < 8:
                    raise WeightsError(f"{path} is too small to be a safetensors file")
                self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        except OSError as e:
            raise WeightsError(f"cannot open {path}: {e.strerror or e}") from None
        (hlen,) = struct.unpack("<Q", self._map[:8])
        if 8 + hlen > size:
            raise WeightsError(f"{path}: header runs past the end of the file")
        try:
            header = json.loads(self._map[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightsError(f"{path}: header is not valid JSON: {e}") from None
        base = 8 + hlen
        self.tensors: dict[str, TensorInfo] = {}
        for name, raw in header.items():
            if name == "__metadata__":
                continue
            # a tensor in a format this library does not read (F16, U8, BOOL, ...) is refused when it is
            # asked for, not when the file is opened: a folder may hold such tensors beside the model's
            dtype, esize = _DTYPES.get(raw["dtype"], (None, None))
            shape = tuple(int(s) for s in raw["shape"])
            start, end = base + int(raw["data_offsets"][0]), base + int(raw["data_offsets"][1])
            numel = 1
            for s in shape:
                numel *= s
            if end > size or start < base or end < start or (esize is not None and end - start != numel * esize):
                raise WeightsError(f"{path}: bad data offsets for {name}")
            self.tensors[name] = TensorInfo(dtype, shape, start, end, str(raw["dtype"]))

    def names(self):
        return self.tensors.keys()

    def load(self, name: str) -> torch.Tensor:
        """A read-only view of the mapped bytes as a tensor (copy it before writing)."""
        info = self.tensors[name]
        if info.dtype is None:
            raise UnsupportedError(f"{self.path}: tensor {name} has dtype {info.stored_as}, supported: {', '.join(_DTYPES)}")
        if info.end == info.start:
            return torch.empty(info.shape, dtype=info.dtype)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)      # the mapping is read-only on purpose
            flat = torch.frombuffer(memoryview(self._map)[info.start:info.end], dtype=info.dtype)
        return flat.reshape(info.shape)


class ModelFolder:
    """All tensors of a model folder by name, whichever shard holds them."""

    INDEX = "model.safetensors.index.json"
    SINGLE = "model.safetensors"

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        self._files: dict[str, SafeTensorFile] = {}
        self._where: dict[str, str] = {}
        index = os.path.join(model_dir, self.INDEX)
        if os.path.exists(index):
            try:
                with open(index, "r", encoding="utf-8") as f:
                    weight_map = json.load(f)["weight_map"]
            except (OSError, json.JSONDecodeError, KeyError) as e:
                raise WeightsError(f"cannot read {index}: {e}") from None
            self._where = {name: shard for name, shard in weight_map.items()}
        else:
            single = os.path.join(model_dir, self.SINGLE)
            if not os.path.exists(single):
                raise WeightsError(f"{model_dir} has neither {self.SINGLE} nor {self.INDEX}")
            f = self._open(self.SINGLE)
            self._where = {name: self.SINGLE for name in f.names()}

    def _open(self, shard: str) -> SafeTensorFile:
        if shard not in self._files:
            self._files[shard] = SafeTensorFile(os.path.join(self.model_dir, shard))
        return self._files[shard]

    def names(self) -> list[str]:
        return sorted(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def info(self, name: str) -> TensorInfo:
        f = self._open(self._where[name])
        if name not in f.tensors:
            raise WeightsError(f"{name} is listed for {f.path} but is not in it")
        return f.tensors[name]

    def load(self, name: str) -> torch.Tensor:
        if name not in self._where:
            raise WeightsError(f"tensor {name} is not in {self.model_dir}")
        self.info(name)
        return self._open(self._where[name]).load(name)


def save_file(tensors: dict, path: str, metadata: dict | None = None) -> None:
    """Write tensors in name order, header first, data 8-byte aligned
    (src/safetensors.rs:251-254, :294-306)."""
    header, offset, order = {}, 0, sorted(tensors)
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise UnsupportedError(f"cannot store {name} of dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - (8 + len(blob)) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())
