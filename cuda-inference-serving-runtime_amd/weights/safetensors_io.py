"""Reading and writing safetensors files without any third-party reader.

Format (as the reference parses it, runtime/checkpoint.py:23-33): 8 bytes of
little-endian header length, a JSON header mapping tensor name to ``dtype``,
``shape`` and ``data_offsets`` relative to the end of the header, then the raw
little-endian data.  Tensors are memory-mapped, never read whole.
"""
import json
import mmap
import struct
from pathlib import Path

import numpy as np
import torch

# safetensors dtype -> (numpy dtype of the raw bytes, torch dtype of the tensor)
_DTYPES = {
    "F32": ("<f4", torch.float32), "F16": ("<f2", torch.float16), "BF16": ("<u2", torch.bfloat16),
    "F64": ("<f8", torch.float64), "I64": ("<i8", torch.int64), "I32": ("<i4", torch.int32),
    "I16": ("<i2", torch.int16), "I8": ("i1", torch.int8), "U8": ("u1", torch.uint8), "BOOL": ("u1", torch.bool),
}
_NAMES = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16", torch.float64: "F64",
          torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8"}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """Header of one file plus lazily mapped tensors."""

    def __init__(self, path):
        self.path = Path(path)
        with self.path.open("rb") as f:
            head = f.read(8)
            if len(head) != 8:
                raise SafetensorsError(f"{self.path}: too short for a safetensors header")
            (size,) = struct.unpack("<Q", head)
            total = self.path.stat().st_size
            if size > total - 8:
                raise SafetensorsError(f"{self.path}: header length {size} exceeds the file")
            header = json.loads(f.read(size))
        self.data_start = 8 + size
        self.entries = {}
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            if meta["dtype"] not in _DTYPES:
                raise SafetensorsError(f"{self.path}: tensor {name} has unsupported dtype {meta['dtype']}")
            begin, end = meta["data_offsets"]
            itemsize = np.dtype(_DTYPES[meta["dtype"]][0]).itemsize
            if end - begin != int(np.prod(meta["shape"], dtype=np.int64)) * itemsize or self.data_start + end > total:
                raise SafetensorsError(f"{self.path}: tensor {name} has an invalid size")
            self.entries[name] = (meta["dtype"], tuple(meta["shape"]), begin, end)
        self._map = None

    def names(self):
        return list(self.entries)

    def info(self, name):
        dtype, shape, _, _ = self.entries[name]
        return _DTYPES[dtype][1], shape

    def tensor(self, name):
        """A CPU tensor that views the mapped file (copy before the file goes away)."""
        dtype, shape, begin, end = self.entries[name]
        if self._map is None:
            with self.path.open("rb") as f:
                self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        np_dtype, torch_dtype = _DTYPES[dtype]
        count = int(np.prod(shape, dtype=np.int64))
        raw = np.frombuffer(self._map, dtype=np_dtype, count=count, offset=self.data_start + begin)
        if dtype == "BF16":
            t = torch.from_numpy(raw.view(np.int16).copy()).view(torch.bfloat16)
        elif dtype == "BOOL":
            t = torch.from_numpy(raw.copy()).to(torch.bool)
        else:
            t = torch.from_numpy(raw.copy())
        return t.reshape(shape)


def write_safetensors(path, tensors, metadata=None):
    """Write CPU tensors {name: tensor} in name order."""
    header, blobs, offset = {}, [], 0
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    for name in sorted(tensors):
        t = tensors[name].detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {t.dtype}")
        data = (t.view(torch.int16) if t.dtype == torch.bfloat16 else t).numpy().tobytes()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(data)]}
        blobs.append(data)
        offset += len(data)
    raw = json.dumps(header, separators=(",", ":")).encode()
    raw += b" " * (-len(raw) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for blob in blobs:
            f.write(blob)
