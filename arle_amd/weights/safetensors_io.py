"""Reading and writing of safetensors files without any library.

Format: 8 bytes little-endian header length, a JSON header
{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}},
then the raw tensor bytes.  Files are memory-mapped; a tensor is copied out only
when it is asked for.  The reference maps shards the same way
(infer/src/weight_loader.rs:27-84) but ignores the dtype field
(crates/cuda-kernels/src/tensor.rs:1140-1178); this reader honours it.
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import numpy as np
import torch

# safetensors dtype -> (numpy carrier type, torch type)
_DTYPES = {
    "F64": (np.float64, torch.float64),
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.uint16, torch.bfloat16),
    "I64": (np.int64, torch.int64),
    "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16),
    "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8),
    "BOOL": (np.bool_, torch.bool),
}
_NAMES = {tt: name for name, (_, tt) in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped .safetensors file: names, shapes, dtypes and lazy tensor reads."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except OSError as exc:
            raise SafetensorsError(f"cannot open {path}: {exc}") from exc
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds the file size")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as exc:
            raise SafetensorsError(f"{path}: header is not valid JSON: {exc}") from exc
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: the header is not a JSON object")
        metadata = header.pop("__metadata__", None)
        self.metadata = metadata if isinstance(metadata, dict) else {}
        self._data_start = 8 + hlen
        self._entries = {}
        whole = lambda v: isinstance(v, int) and not isinstance(v, bool) and v >= 0
        for name, info in header.items():
            # a damaged header is refused here, with the tensor's name, and not by whatever trips over it later
            if not (isinstance(info, dict) and isinstance(info.get("dtype"), str) and isinstance(info.get("shape"), list)
                    and all(whole(n) for n in info["shape"]) and isinstance(info.get("data_offsets"), list)
                    and len(info["data_offsets"]) == 2 and all(whole(n) for n in info["data_offsets"])):
                raise SafetensorsError(f"{path}: tensor '{name}': the header entry must hold a dtype, a shape of "
                                       f"non-negative integers and two non-negative data_offsets, got {info!r}")
            dtype, shape, (begin, end) = info["dtype"], tuple(info["shape"]), info["data_offsets"]
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dtype}")
            count = 1
            for n in shape:     # exact integers: a shape whose product does not fit 64 bits must not wrap round
                count *= n
            nbytes = count * np.dtype(_DTYPES[dtype][0]).itemsize
            if end - begin != nbytes or self._data_start + end > size:
                raise SafetensorsError(
                    f"{path}: tensor '{name}': data length mismatch: expected {nbytes} bytes for "
                    f"shape {list(shape)} {dtype}, got {end - begin}")
            self._entries[name] = (dtype, shape, begin, count)
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self):
        return list(self._entries)

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def info(self, name: str):
        """(torch dtype, shape) of a tensor."""
        dtype, shape, _, _ = self._entries[name]
        return _DTYPES[dtype][1], shape

    def read(self, name: str) -> torch.Tensor:
        """A fresh CPU tensor holding a copy of the stored values, in the stored dtype."""
        dtype, shape, begin, count = self._entries[name]
        np_type, torch_type = _DTYPES[dtype]
        arr = np.frombuffer(self._mm, dtype=np_type, count=count, offset=self._data_start + begin)
        t = torch.from_numpy(arr.copy())
        if dtype == "BF16":
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def close(self) -> None:
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._fh.close()


def write_safetensors(path: str, tensors: dict, metadata: dict | None = None) -> None:
    """Write CPU tensors to `path` (names sorted, data 8-byte aligned through header padding)."""
    header = {}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}' has dtype {t.dtype}, which safetensors cannot hold")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = f"{path}.tmp{os.getpid()}"
    with open(tmp, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)))
        fh.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            if t.dtype == torch.bfloat16:
                t = t.view(torch.int16)
            fh.write(t.numpy().tobytes())
    os.replace(tmp, path)
