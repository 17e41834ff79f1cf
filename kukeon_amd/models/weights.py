"""Checkpoint reading: a safetensors file is an 8-byte little-endian header
length, that many bytes of JSON (name -> dtype, shape, data_offsets) and the
raw tensor data. The file is memory-mapped and each tensor is copied out on
request, so nothing is executed from the file and a large checkpoint is
never held twice in host memory."""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterator, Tuple

import torch

_DTYPES = {
    "BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32,
    "F64": torch.float64, "I32": torch.int32, "I64": torch.int64,
    "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n > (1 << 30):
            raise ValueError("safetensors header is implausibly large")
        self.meta = json.loads(self._f.read(n).decode("utf-8"))
        self.meta.pop("__metadata__", None)
        self._base = 8 + n
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)

    def keys(self):
        return self.meta.keys()

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.meta[name]["shape"])

    def get(self, name: str) -> torch.Tensor:
        m = self.meta[name]
        dt = _DTYPES.get(m["dtype"])
        if dt is None:
            raise ValueError(f"{name}: unsupported dtype {m['dtype']}")
        a, b = m["data_offsets"]
        numel = 1
        for d in m["shape"]:
            numel *= d
        if numel == 0:
            return torch.empty(m["shape"], dtype=dt)
        # one copy out of the mapping; the tensor owns its bytes
        buf = bytearray(self._mm[self._base + a: self._base + b])
        return torch.frombuffer(buf, dtype=dt, count=numel).reshape(
            m["shape"])

    def items(self) -> Iterator[Tuple[str, torch.Tensor]]:
        for k in self.meta:
            yield k, self.get(k)

    def close(self) -> None:
        try:
            self._mm.close()
        except BufferError:
            pass
        self._f.close()


def read_checkpoint(model_dir: str) -> Tuple[dict, Dict[str, torch.Tensor]]:
    """-> (config.json as a dict, {tensor name: CPU tensor})."""
    with open(os.path.join(model_dir, "config.json")) as f:
        config = json.load(f)
    st = SafetensorsFile(os.path.join(model_dir, "model.safetensors"))
    try:
        tensors = dict(st.items())
    finally:
        st.close()
    return config, tensors
