"""Reader and writer of the safetensors container: an 8-byte little-endian header length, a JSON
header {name: {dtype, shape, data_offsets}}, then the raw little-endian data.

The reference memory-maps the files through candle's VarBuilder
(core/src/model_executor/models/model_factory.rs:133-139) and lists them from
model.safetensors.index.json (:64-77). Here the file is memory-mapped and a tensor's bytes are
touched only when that tensor is fetched, so a checkpoint larger than host memory can be loaded
tensor by tensor.
"""
import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import torch


class SafetensorsError(ValueError):
    pass


# safetensors dtype string -> (torch dtype of the raw view, bytes per element)
_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_DTYPE_NAMES = {v[0]: k for k, v in _DTYPES.items()}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    file: str
    dtype: str            # safetensors dtype string
    shape: Tuple[int, ...]
    begin: int            # byte offsets inside the data section
    end: int


class SafetensorsFile:
    """One memory-mapped .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError("%s: too short to be a safetensors file (%d bytes)" % (path, size))
        self._f = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError("%s: header length %d does not fit the file of %d bytes" % (path, hlen, size))
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError("%s: header is not valid JSON: %s" % (path, e))
        if not isinstance(header, dict):
            raise SafetensorsError("%s: header is not a JSON object" % path)
        self.data_start = 8 + hlen
        self.data_size = size - self.data_start
        self.entries: Dict[str, TensorEntry] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                dtype = info["dtype"]
                shape = tuple(int(s) for s in info["shape"])
                begin, end = (int(x) for x in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError("%s: malformed header entry for %r" % (path, name))
            if dtype not in _DTYPES:
                raise SafetensorsError("%s: tensor %r has unsupported dtype %s" % (path, name, dtype))
            n = 1
            for s in shape:
                n *= s
            if end - begin != n * _DTYPES[dtype][1]:
                raise SafetensorsError("%s: tensor %r: %d bytes for shape %s of %s" % (path, name, end - begin,
                                                                                      list(shape), dtype))
            if begin < 0 or end > self.data_size:
                raise SafetensorsError("%s: tensor %r lies outside the file (truncated?)" % (path, name))
            self.entries[name] = TensorEntry(name, path, dtype, shape, begin, end)
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def read(self, name: str) -> torch.Tensor:
        """The tensor as a CPU tensor that owns its memory."""
        e = self.entries[name]
        tdtype, _ = _DTYPES[e.dtype]
        nbytes = e.end - e.begin
        if nbytes == 0:
            return torch.empty(e.shape, dtype=tdtype)
        buf = bytearray(self._mm[self.data_start + e.begin:self.data_start + e.end])
        return torch.frombuffer(buf, dtype=tdtype).reshape(e.shape)

    def close(self):
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._f.close()


def list_weight_files(folder: str) -> List[str]:
    """model.safetensors.index.json's files if present, else model.safetensors, else *.safetensors."""
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            try:
                wm = json.load(f)["weight_map"]
            except (json.JSONDecodeError, KeyError, TypeError) as e:
                raise SafetensorsError("%s is not a weight index: %s" % (index, e))
        files = sorted(set(wm.values()))
        missing = [x for x in files if not os.path.isfile(os.path.join(folder, x))]
        if missing:
            raise SafetensorsError("%s names files that are not there: %s" % (index, ", ".join(missing)))
        return [os.path.join(folder, x) for x in files]
    single = os.path.join(folder, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    files = sorted(x for x in os.listdir(folder) if x.endswith(".safetensors")) if os.path.isdir(folder) else []
    if not files:
        raise SafetensorsError("no safetensors file in model folder %r" % folder)
    return [os.path.join(folder, x) for x in files]


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata: Dict[str, str] = None) -> None:
    """Write CPU tensors in the order given."""
    items = [(n, t.detach().contiguous().cpu()) for n, t in tensors]
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    for name, t in items:
        if t.dtype not in _DTYPE_NAMES:
            raise SafetensorsError("cannot store dtype %s of tensor %r" % (t.dtype, name))
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _DTYPE_NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
    hbytes = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hbytes += b" " * ((8 - len(hbytes) % 8) % 8)
    tmp = path + ".tmp%d" % os.getpid()
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hbytes)))
        f.write(hbytes)
        for _, t in items:
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
