"""The safetensors container, read and written directly: an 8-byte little-endian header length,
a JSON header {name: {dtype, shape, data_offsets}}, then raw little-endian data.  Tensors are
memory-mapped and handed out one at a time, so a large file is never held whole in host memory.
"""
import json
import mmap
import os
import struct

import numpy as np
import torch

_NP = {"F64": np.float64, "F32": np.float32, "F16": np.float16, "BF16": np.uint16, "I64": np.int64,
       "I32": np.int32, "I16": np.int16, "I8": np.int8, "U8": np.uint8, "BOOL": np.bool_}
_TORCH = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
          "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
          "BOOL": torch.bool}
_FROM_TORCH = {v: k for k, v in _TORCH.items()}


class SafetensorsFile:
    def __init__(self, path):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise ValueError(f"{path}: too short to be a safetensors file")
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n <= 0 or 8 + n > size:
            raise ValueError(f"{path}: header length {n} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(n))
        except ValueError as e:
            raise ValueError(f"{path}: the header is not JSON ({e})") from None
        self.metadata = header.pop("__metadata__", {})
        self.entries = header
        self._base = 8 + n
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        for name, info in header.items():
            lo, hi = info["data_offsets"]
            if info["dtype"] not in _NP:
                raise ValueError(f"{path}: tensor {name} has unsupported dtype {info['dtype']}")
            want = int(np.prod(info["shape"], dtype=np.int64)) * np.dtype(_NP[info["dtype"]]).itemsize
            if hi - lo != want or self._base + hi > size:
                raise ValueError(f"{path}: tensor {name} is truncated or its offsets are wrong")

    def names(self):
        return list(self.entries)

    def shape(self, name):
        return tuple(self.entries[name]["shape"])

    def dtype(self, name) -> torch.dtype:
        return _TORCH[self.entries[name]["dtype"]]

    def tensor(self, name) -> torch.Tensor:
        """A CPU tensor that views the mapped file (copy before the file is closed)."""
        info = self.entries[name]
        lo, hi = info["data_offsets"]
        arr = np.frombuffer(self._mm, dtype=_NP[info["dtype"]], count=(hi - lo) // np.dtype(_NP[info["dtype"]]).itemsize,
                            offset=self._base + lo).reshape(info["shape"])
        t = torch.from_numpy(arr) if arr.flags.writeable else torch.from_numpy(arr.copy())
        return t.view(torch.bfloat16) if info["dtype"] == "BF16" else t

    def close(self):
        self._mm.close()
        self._f.close()


def write_safetensors(path, tensors, metadata=None):
    """tensors: ordered {name: CPU torch tensor}."""
    header, offset = {}, 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        raw = (t.view(torch.int16) if t.dtype == torch.bfloat16 else t).numpy().tobytes()
        header[name] = {"dtype": _FROM_TORCH[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    head = json.dumps(header, separators=(",", ":")).encode()
    head += b" " * ((8 - len(head) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(head)))
        f.write(head)
        for raw in blobs:
            f.write(raw)
