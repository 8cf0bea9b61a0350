"""Reader and writer of the safetensors container: an 8-byte little-endian header length, a JSON
header {name: {dtype, shape, data_offsets}}, then the raw little-endian data.

The reference memory-maps the files through candle's VarBuilder
(core/src/model_executor/models/model_factory.rs:133-139) and lists them from
model.safetensors.index.json (:64-77). Here the file is memory-mapped (in C++, csrc/host/safetensors.cc)
and a tensor's bytes are touched only when that tensor is fetched, so a checkpoint larger than host
memory can be loaded tensor by tensor.
"""
import ctypes
import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import torch

from ..host.library import last_error, load_host_library


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


class _NativeRecord(ctypes.Structure):
    # LmsfTensorRecord of csrc/host/api.cc
    _fields_ = [("name", ctypes.c_char_p), ("dtype", ctypes.c_char * 8), ("ndim", ctypes.c_int),
                ("shape", ctypes.c_int64 * 8), ("begin", ctypes.c_int64), ("end", ctypes.c_int64)]


class SafetensorsFile:
    """One memory-mapped .safetensors file. The file is opened, mapped and its header read and checked in C++
    (``csrc/host/safetensors.cc``: every tensor's dtype, byte count against its shape, place inside the file, no
    two overlapping or of one name); this class is the face of that object and turns a tensor's bytes into a
    torch tensor."""

    def __init__(self, path: str):
        self.path = path
        self._lib = lib = load_host_library()
        handle = ctypes.c_void_p()
        if lib.lmsf_safetensors_open(os.fsencode(path), ctypes.byref(handle)) != 0:
            raise SafetensorsError(last_error(lib))
        self._handle = handle
        size = ctypes.c_int64()
        self._data = lib.lmsf_safetensors_data(handle, ctypes.byref(size))
        self.data_size = size.value
        self.entries: Dict[str, TensorEntry] = {}
        rec = _NativeRecord()
        for i in range(lib.lmsf_safetensors_count(handle)):
            if lib.lmsf_safetensors_record(handle, i, ctypes.byref(rec)) != 0:
                msg = last_error(lib)
                self.close()
                raise SafetensorsError("%s: %s" % (path, msg))
            name = rec.name.decode("utf-8")
            self.entries[name] = TensorEntry(name, path, rec.dtype.decode("ascii"),
                                             tuple(int(rec.shape[k]) for k in range(rec.ndim)), rec.begin, rec.end)

    def read(self, name: str, copy: bool = True) -> torch.Tensor:
        """The tensor as a CPU tensor that owns its memory. ``copy=False``: a tensor over the mapped file itself,
        which must be gone before the file is closed (the loader copies it to the device at once and drops it: one
        pass over the bytes fewer)."""
        e = self.entries[name]
        tdtype, _ = _DTYPES[e.dtype]
        nbytes = e.end - e.begin
        if nbytes == 0:
            return torch.empty(e.shape, dtype=tdtype)
        if self._handle is None:
            raise SafetensorsError("%s is closed" % self.path)
        mapped = (ctypes.c_ubyte * nbytes).from_address(self._data + e.begin)
        # (bytes -> a tensor over the mapping -> a copy that outlives it)
        view = torch.frombuffer(mapped, dtype=tdtype).reshape(e.shape)
        return view.clone() if copy else view

    def close(self):
        if self._handle is not None:
            self._lib.lmsf_safetensors_close(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001 - nothing to do about it at this point
            pass


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
