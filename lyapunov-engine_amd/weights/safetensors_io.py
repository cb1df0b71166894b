"""Reader and writer of the safetensors file format.

Layout of a file: eight bytes, little endian, giving the length N of the header;
N bytes of JSON ``{name: {"dtype", "shape", "data_offsets": [begin, end]}}``
(plus an optional ``__metadata__`` entry); then the tensors' bytes, offsets
counted from the end of the header.

The reference reads these files through the safetensors package
(python/lyapunov_engine/models/weight_loader.py:41-71: every ``*.safetensors``
of a folder, sorted, later files overwriting earlier ones).  This module maps
the file and hands out tensors that view the mapping, so nothing is copied until
a tensor goes to the device.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass

import numpy as np
import torch

# dtype code -> (torch dtype, bytes per element, numpy dtype to view the bytes as)
_DTYPES = {
    "F32": (torch.float32, 4, np.float32),
    "F16": (torch.float16, 2, np.float16),
    "BF16": (torch.bfloat16, 2, np.uint16),
    "F64": (torch.float64, 8, np.float64),
    "I64": (torch.int64, 8, np.int64),
    "I32": (torch.int32, 4, np.int32),
    "I16": (torch.int16, 2, np.int16),
    "I8": (torch.int8, 1, np.int8),
    "U8": (torch.uint8, 1, np.uint8),
    "BOOL": (torch.bool, 1, np.bool_),
}
_CODES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str          # the file's code, e.g. "BF16"
    shape: tuple
    begin: int          # byte offsets into the data section
    end: int
    file: str


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} does not fit a file of {size} bytes")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + hlen
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None
        self.entries: dict[str, TensorEntry] = {}
        for name, info in header.items():
            code = info.get("dtype")
            if code not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unknown dtype {code!r}")
            shape = tuple(int(s) for s in info["shape"])
            begin, end = (int(x) for x in info["data_offsets"])
            want = int(np.prod(shape, dtype=np.int64)) * _DTYPES[code][1]
            if end - begin != want or begin < 0 or self._data_start + end > size:
                raise SafetensorsError(f"{path}: tensor {name!r} has {end - begin} bytes at [{begin}, {end}) "
                                       f"but shape {shape} of {code} needs {want}")
            self.entries[name] = TensorEntry(name, code, shape, begin, end, path)

    def names(self) -> list[str]:
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (read-only memory: convert or
        copy before writing to it)."""
        e = self.entries[name]
        tdtype, esz, ndtype = _DTYPES[e.dtype]
        count = (e.end - e.begin) // esz
        if count == 0:
            return torch.empty(e.shape, dtype=tdtype)
        arr = np.frombuffer(self._map, dtype=ndtype, count=count, offset=self._data_start + e.begin)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the mapping is read-only; the tensor is only read
            t = torch.from_numpy(arr)
        if e.dtype == "BF16":
            t = t.view(torch.bfloat16)
        return t.view(e.shape)

    def close(self) -> None:
        # Tensors handed out keep the mapping alive through their buffer; the
        # mapping is closed when the last of them goes.
        try:
            self._f.close()
        except Exception:
            pass


def open_model_files(model_dir: str) -> list[SafetensorsFile]:
    """Every ``*.safetensors`` of the folder, in sorted order."""
    if not os.path.isdir(model_dir):
        raise FileNotFoundError(f"{model_dir} is not a folder")
    files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors files found in {model_dir}")
    return [SafetensorsFile(os.path.join(model_dir, f)) for f in files]


def write_safetensors(path: str, tensors: dict[str, torch.Tensor], metadata: dict | None = None) -> None:
    """Write the tensors (CPU, any of the dtypes above) in the order given."""
    header: dict = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        if t.dtype not in _CODES:
            raise SafetensorsError(f"tensor {name!r} has dtype {t.dtype}, which the format does not hold")
        t = t.detach().cpu().contiguous()
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _CODES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        blobs.append(t)
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)  # keep the data section 8-byte aligned
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for t in blobs:
            if t.numel() == 0:
                continue
            flat = t.reshape(-1)
            if t.dtype == torch.bfloat16:
                flat = flat.view(torch.int16)
            f.write(flat.numpy().tobytes())
    os.replace(tmp, path)
