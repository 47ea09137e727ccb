"""Checkpoint files -> name -> tensor, with no code executed from the file.

A .safetensors file is: 8 bytes little-endian header length, that many bytes of JSON {name: {"dtype", "shape", "data_offsets"}}, then the
raw little-endian data.  The file is memory-mapped and each tensor is a view of the map, so a large checkpoint is never read whole; the
model's loader moves one tensor at a time to the device.
"""
import json
import mmap
import os
import struct
import warnings

import torch

_DTYPES = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64, "I32": torch.int32, "I64": torch.int64,
           "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8, "BOOL": torch.bool}


class SafetensorsFile:
    def __init__(self, path):
        self.path = path
        self._fh = open(path, "rb")
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise ValueError(f"{path}: not a safetensors file")
        (n,) = struct.unpack("<Q", self._fh.read(8))
        if n > size - 8:
            raise ValueError(f"{path}: header length past the end of the file")
        self.header = json.loads(self._fh.read(n).decode("utf-8"))
        self.header.pop("__metadata__", None)
        self._base = 8 + n
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        self._size = size

    def keys(self):
        return list(self.header)

    def shape(self, name):
        return tuple(self.header[name]["shape"])

    def get(self, name):
        """a CPU tensor that views the mapped file (read-only memory: copy or move it before writing)"""
        e = self.header[name]
        dt = _DTYPES.get(e["dtype"])
        if dt is None:
            raise ValueError(f"{self.path}: tensor {name}: dtype {e['dtype']} is not supported")
        lo, hi = e["data_offsets"]
        shape = tuple(e["shape"])
        count = 1
        for s in shape:
            count *= s
        if hi - lo != count * torch.empty((), dtype=dt).element_size() or self._base + hi > self._size:
            raise ValueError(f"{self.path}: tensor {name}: data range does not fit its shape")
        if count == 0:
            return torch.empty(shape, dtype=dt)
        with warnings.catch_warnings():                 # (the map is read-only; nothing here writes through the view)
            warnings.simplefilter("ignore", UserWarning)
            flat = torch.frombuffer(self._map, dtype=dt, count=count, offset=self._base + lo)
        return flat.reshape(shape)

    def __contains__(self, name):
        return name in self.header


def load_dir(path):
    """every *.safetensors file of a model folder as one lazily read mapping"""
    files = [SafetensorsFile(os.path.join(path, f)) for f in sorted(os.listdir(path)) if f.endswith(".safetensors")]
    if not files:
        raise FileNotFoundError(f"{path}: no .safetensors file")
    return Checkpoint(files)


class Checkpoint:
    def __init__(self, files):
        self.files = files
        self.where = {}
        for f in files:
            for k in f.keys():
                self.where[k] = f

    def keys(self):
        return list(self.where)

    def __contains__(self, name):
        return name in self.where

    def __getitem__(self, name):
        if name not in self.where:
            raise KeyError(f"tensor {name} is not in the checkpoint")
        return self.where[name].get(name)

    def shape(self, name):
        return self.where[name].shape(name)
