"""Reading and writing safetensors files.

Layout of a file: an 8-byte little-endian header length ``n``, ``n`` bytes of
JSON ``{name: {"dtype", "shape", "data_offsets": [begin, end]}, ...}`` (plus an
optional ``"__metadata__"`` entry), then the tensors' little-endian bytes;
offsets are relative to the first byte after the header.  (The reference keeps
its weights in a private container, engine/src/loader.cpp:55-135, read the
same way: a directory of names, then a data section.)

Tensors are memory-mapped, so a large file is never read whole.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

from ..errors import WeightError

# safetensors dtype -> (numpy dtype used to view the bytes, bytes per element)
_NP_VIEW = {
    "F64": (np.dtype("<f8"), 8), "F32": (np.dtype("<f4"), 4), "F16": (np.dtype("<f2"), 2),
    "BF16": (np.dtype("<u2"), 2), "I64": (np.dtype("<i8"), 8), "I32": (np.dtype("<i4"), 4),
    "I16": (np.dtype("<i2"), 2), "I8": (np.dtype("i1"), 1), "U8": (np.dtype("u1"), 1),
    "BOOL": (np.dtype("u1"), 1),
}
_TORCH_TO_ST = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16",
                torch.int32: "I32", torch.int64: "I64", torch.float64: "F64"}


class SafetensorsFile:
    """One .safetensors file, opened read-only and memory-mapped."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except OSError as e:
            raise WeightError(f"cannot open {path}: {e.strerror}") from None
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise WeightError(f"{path}: truncated (no header length)")
        (n,) = struct.unpack("<Q", self._fh.read(8))
        if n > size - 8:
            raise WeightError(f"{path}: truncated (header says {n} bytes, file has {size - 8} after the length)")
        try:
            header = json.loads(self._fh.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightError(f"{path}: header is not valid JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + n
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        self.entries: Dict[str, dict] = {}
        if not isinstance(header, dict):
            raise WeightError(f"{path}: header is not a JSON object")
        for name, e in header.items():
            if not isinstance(e, dict):
                raise WeightError(f"{path}: header entry of tensor '{name}' is not an object")
            dt, shape, offsets = e.get("dtype"), e.get("shape"), e.get("data_offsets")
            if dt not in _NP_VIEW:
                raise WeightError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
            if not isinstance(shape, list) or any(not isinstance(d, int) or isinstance(d, bool) or d < 0 for d in shape):
                raise WeightError(f"{path}: tensor '{name}' has a bad shape {shape!r} (a list of non-negative integers is needed)")
            if (not isinstance(offsets, list) or len(offsets) != 2
                    or any(not isinstance(o, int) or isinstance(o, bool) for o in offsets) or not 0 <= offsets[0] <= offsets[1]):
                raise WeightError(f"{path}: tensor '{name}' has bad data_offsets {offsets!r} (a pair 0 <= begin <= end is needed)")
            b, end = offsets
            count = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
            if end - b != count * _NP_VIEW[dt][1]:
                raise WeightError(f"{path}: tensor '{name}' of shape {shape} and dtype {dt} "
                                  f"claims {end - b} bytes")
            if b < 0 or self._data_start + end > size:
                raise WeightError(f"{path}: data of tensor '{name}' lies outside the file")
            self.entries[name] = {"dtype": dt, "shape": tuple(int(s) for s in shape), "begin": b, "end": end}

    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name]["shape"]

    def stored_dtype(self, name: str) -> str:
        return self.entries[name]["dtype"]

    def tensor(self, name: str) -> torch.Tensor:
        """The tensor as the host hands it on: BF16 stays bfloat16, F32 stays float32, F16 stays
        float16 (the device then keeps it in bfloat16, or widens it for the 32-bit path), F64 becomes
        float32; integers become int32."""
        e = self.entries[name]
        npdt, _ = _NP_VIEW[e["dtype"]]
        arr = np.frombuffer(self._mm, dtype=npdt, count=int(np.prod(e["shape"], dtype=np.int64)) if e["shape"] else 1,
                            offset=self._data_start + e["begin"]).reshape(e["shape"])
        dt = e["dtype"]
        if dt == "BF16":
            return torch.from_numpy(arr.copy()).view(torch.bfloat16)
        if dt in ("F32",):
            return torch.from_numpy(arr.copy())
        if dt == "F16":
            return torch.from_numpy(arr.copy())
        if dt == "F64":
            return torch.from_numpy(arr.astype(np.float32))
        if dt == "BOOL":
            return torch.from_numpy(arr.astype(np.int32))
        big = arr.astype(np.int64)
        if big.size and (big.max() > np.iinfo(np.int32).max or big.min() < np.iinfo(np.int32).min):
            raise WeightError(f"{self.path}: integer tensor '{name}' does not fit int32")
        return torch.from_numpy(big.astype(np.int32))

    def close(self) -> None:
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._fh.close()


class SafetensorsWriter:
    """Writes one file tensor by tensor; shapes and dtypes are declared first so
    the header can be written before any data (a large model is never held
    whole in memory)."""

    def __init__(self, path: str, layout: Iterable[Tuple[str, Tuple[int, ...], torch.dtype]],
                 metadata: Dict[str, str] = None):
        self.path = path
        header, offset, self._order = {}, 0, []
        for name, shape, dtype in layout:
            st = _TORCH_TO_ST[dtype]
            nbytes = int(np.prod(shape, dtype=np.int64)) * _NP_VIEW[st][1] if len(shape) else _NP_VIEW[st][1]
            header[name] = {"dtype": st, "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
            self._order.append((name, tuple(shape), dtype, nbytes))
            offset += nbytes
        if metadata:
            header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
        blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
        blob += b" " * ((8 - len(blob) % 8) % 8)
        self._fh = open(path, "wb")
        self._fh.write(struct.pack("<Q", len(blob)))
        self._fh.write(blob)
        self._next = 0

    def write(self, name: str, tensor: torch.Tensor) -> None:
        want_name, shape, dtype, nbytes = self._order[self._next]
        if name != want_name or tuple(tensor.shape) != shape or tensor.dtype != dtype:
            raise WeightError(f"writer expected '{want_name}' {shape} {dtype}, got '{name}' "
                              f"{tuple(tensor.shape)} {tensor.dtype}")
        t = tensor.detach().contiguous().cpu()
        if dtype == torch.bfloat16:
            data = t.view(torch.int16).numpy().tobytes()
        else:
            data = t.numpy().tobytes()
        assert len(data) == nbytes
        self._fh.write(data)
        self._next += 1

    def close(self) -> None:
        if self._next != len(self._order):
            raise WeightError(f"{self.path}: {len(self._order) - self._next} declared tensors were not written")
        self._fh.close()


def open_model_tensors(model_dir: str) -> Dict[str, Tuple[SafetensorsFile, str]]:
    """name -> (file, name) over a model folder: ``model.safetensors``, or the
    shards listed in ``model.safetensors.index.json``."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    files: List[SafetensorsFile] = []
    if os.path.exists(single):
        files.append(SafetensorsFile(single))
    elif os.path.exists(index):
        with open(index, "r", encoding="utf-8") as fh:
            shard_names = sorted(set(json.load(fh).get("weight_map", {}).values()))
        files.extend(SafetensorsFile(os.path.join(model_dir, s)) for s in shard_names)
    else:
        raise WeightError(f"no model.safetensors (or model.safetensors.index.json) in {model_dir}")
    out: Dict[str, Tuple[SafetensorsFile, str]] = {}
    for f in files:
        for n in f.names():
            if n in out:
                raise WeightError(f"tensor '{n}' appears in both {out[n][0].path} and {f.path}")
            out[n] = (f, n)
    return out
