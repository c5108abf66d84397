"""A small reader and writer of the safetensors format.

The format is an 8-byte little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets"}}`` and the raw little-endian data.  The
reference reads such files tensor by tensor with ``safe_open(...).get_tensor``
(scripts/tools/convert_checkpoint.py:43-55); this reader maps the file and hands out
views, so a tensor is copied once, straight to the device.
"""

from __future__ import annotations

import json
import mmap
import os
import struct

import torch

_DTYPES = {
    "F32": torch.float32,
    "BF16": torch.bfloat16,
    "F16": torch.float16,
    "F64": torch.float64,
    "I64": torch.int64,
    "I32": torch.int32,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped file; ``entries[name] = (dtype name, shape, begin, end)``."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._f.read(n))
        except json.JSONDecodeError as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from e
        self.metadata = header.pop("__metadata__", {})
        self._base = 8 + n
        self.entries = {}
        for name, info in header.items():
            begin, end = info["data_offsets"]
            if self._base + end > size or begin > end:
                raise SafetensorsError(f"{path}: tensor {name!r} lies outside the file")
            self.entries[name] = (info["dtype"], tuple(info["shape"]), begin, end)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self):
        return list(self.entries)

    def dtype_of(self, name: str) -> str:
        return self.entries[name][0]

    def shape_of(self, name: str) -> tuple[int, ...]:
        return self.entries[name][1]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (do not write to it)."""
        dt, shape, begin, end = self.entries[name]
        if dt not in _DTYPES:
            raise SafetensorsError(f"{self.path}: tensor {name!r} has unsupported dtype {dt}")
        dtype = _DTYPES[dt]
        count = 1
        for s in shape:
            count *= s
        if count * dtype.itemsize != end - begin:
            raise SafetensorsError(f"{self.path}: tensor {name!r}: {end - begin} bytes for shape {shape} of {dt}")
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the buffer is read-only; nothing writes to it
            flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._base + begin)
        return flat.view(shape)

    def close(self):
        if self._map is not None:
            self._map.close()
            self._map = None
        self._f.close()


class ModelFiles:
    """The tensors of a model folder: ``model.safetensors``, or the shards that
    ``model.safetensors.index.json`` lists."""

    def __init__(self, folder: str):
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        self.files: list[SafetensorsFile] = []
        self.where: dict[str, SafetensorsFile] = {}
        self.notes: list[str] = []  # where the index and the shards disagree
        problems = []
        shard_of = {}
        if os.path.isfile(single):
            paths = [single]
        elif os.path.isfile(index):
            with open(index) as f:
                shard_of = json.load(f)["weight_map"]
            paths = []
            for shard in sorted(set(shard_of.values())):
                p = os.path.join(folder, shard)
                if os.path.isfile(p):
                    paths.append(p)
                else:
                    problems.append(f"missing shard file {shard}")
        else:
            raise SafetensorsError(f"{folder}: no model.safetensors and no model.safetensors.index.json")
        if problems:
            raise SafetensorsError(f"{folder}: " + "; ".join(problems))
        names_in = {}  # path of a file -> the names of its tensors
        for p in paths:
            sf = SafetensorsFile(p)
            self.files.append(sf)
            names_in[p] = set(sf.names())
            for name in names_in[p]:
                self.where[name] = sf
        for name, shard in shard_of.items():  # (a shard may be named with a subfolder)
            if name not in names_in[os.path.join(folder, shard)]:
                self.notes.append(f"the index lists {name} in {shard}, which does not hold it")

    def names(self):
        return list(self.where)

    def dtype_of(self, name):
        return self.where[name].dtype_of(name)

    def shape_of(self, name):
        return self.where[name].shape_of(name)

    def tensor(self, name):
        return self.where[name].tensor(name)

    def close(self):
        for f in self.files:
            f.close()


class SafetensorsWriter:
    """Writes a file whose tensors are produced one at a time: the header is fixed
    from names, dtypes and shapes first, then the data follows in that order."""

    def __init__(self, path: str, layout: list[tuple[str, torch.dtype, tuple[int, ...]]], metadata=None):
        header = {}
        if metadata:
            header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
        offset = 0
        self._expect = []
        for name, dtype, shape in layout:
            count = 1
            for s in shape:
                count *= s
            nbytes = count * dtype.itemsize
            header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
            self._expect.append((name, dtype, tuple(shape), nbytes))
            offset += nbytes
        raw = json.dumps(header, separators=(",", ":")).encode()
        raw += b" " * ((8 - len(raw) % 8) % 8)
        self._f = open(path, "wb")
        self._f.write(struct.pack("<Q", len(raw)))
        self._f.write(raw)
        self._next = 0

    def write(self, name: str, tensor: torch.Tensor):
        want_name, dtype, shape, nbytes = self._expect[self._next]
        if name != want_name or tensor.dtype != dtype or tuple(tensor.shape) != shape:
            raise SafetensorsError(
                f"writer expected {want_name} {dtype} {shape}, got {name} {tensor.dtype} {tuple(tensor.shape)}"
            )
        t = tensor.detach().cpu().contiguous()
        self._f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
        self._next += 1

    def close(self):
        if self._next != len(self._expect):
            raise SafetensorsError(f"writer closed after {self._next} of {len(self._expect)} tensors")
        self._f.close()


def save_file(tensors: dict[str, torch.Tensor], path: str, metadata=None):
    layout = [(k, v.dtype, tuple(v.shape)) for k, v in tensors.items()]
    w = SafetensorsWriter(path, layout, metadata)
    for k, v in tensors.items():
        w.write(k, v)
    w.close()
