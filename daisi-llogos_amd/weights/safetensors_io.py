"""Reading and writing safetensors files: 8 bytes little-endian header length, a JSON
header {name: {dtype, shape, data_offsets}}, then the tensors' bytes.  Files are memory
mapped, so a tensor's bytes are touched only when it is copied to the device."""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped file: `names`, `shape(name)`, `dtype(name)`, `tensor(name)`."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"cannot open {path}: {e}") from e
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors file")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} does not fit the file")
        try:
            header = json.loads(self._fh.read(hlen))
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from e
        self._base = 8 + hlen
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries: Dict[str, dict] = {}
        for name, ent in header.items():
            if name == "__metadata__":
                continue
            if ent.get("dtype") not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {ent.get('dtype')}")
            b, e = ent["data_offsets"]
            if not (0 <= b <= e and self._base + e <= size):
                raise SafetensorsError(f"{path}: tensor '{name}' lies outside the file")
            self.entries[name] = ent

    @property
    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.entries[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name]["dtype"]]

    def tensor(self, name: str) -> torch.Tensor:
        """A read-only host view of the tensor's bytes in the file's own element type."""
        ent = self.entries[name]
        b, e = ent["data_offsets"]
        dtype = _DTYPES[ent["dtype"]]
        shape = tuple(ent["shape"])
        n = 1
        for s in shape:
            n *= s
        if n * torch.empty((), dtype=dtype).element_size() != e - b:
            raise SafetensorsError(f"{self.path}: tensor '{name}' has {e - b} bytes, its shape needs "
                                   f"{n * torch.empty((), dtype=dtype).element_size()}")
        if n == 0:
            return torch.empty(shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")          # the mapping is read-only and never written through
            t = torch.frombuffer(self._mm, dtype=dtype, count=n, offset=self._base + b)
        return t.reshape(shape)

    def close(self) -> None:
        try:
            self._mm.close()
        except (BufferError, ValueError):
            pass                                     # views are still alive; the mapping goes with them
        self._fh.close()


def open_model_files(folder: str) -> List[SafetensorsFile]:
    """model.safetensors, or the shards that model.safetensors.index.json lists."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    if os.path.isfile(index):
        with open(index) as fh:
            weight_map = json.load(fh).get("weight_map", {})
        return [SafetensorsFile(os.path.join(folder, f)) for f in sorted(set(weight_map.values()))]
    raise SafetensorsError(f"no model.safetensors (or model.safetensors.index.json) in '{folder}'")


def write_safetensors(path: str, tensors, layout=None) -> None:
    """Write named host tensors.  `tensors` is a dict or an iterable of (name, tensor).
    With `layout`, a list of (name, shape, dtype) in the same order, the header is written
    from the layout and the tensors are streamed one at a time, never all in memory."""
    if isinstance(tensors, dict):
        tensors = list(tensors.items())
    if layout is None:
        tensors = list(tensors)
        layout = [(n, tuple(t.shape), t.dtype) for n, t in tensors]
    header, offset = {}, 0
    for name, shape, dtype in layout:
        if dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}': dtype {dtype} cannot be stored")
        n = 1
        for d in shape:
            n *= d
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)))
        fh.write(blob)
        for (name, shape, dtype), (tname, t) in zip(layout, tensors):
            if tname != name or tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise SafetensorsError(f"tensor '{tname}' does not match the layout entry '{name}'")
            t = t.detach().cpu().contiguous()
            if t.numel():
                fh.write(t.view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
