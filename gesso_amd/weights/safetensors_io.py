"""Reading and writing safetensors files, with the format's integrity rules enforced.

A file is an 8-byte little-endian header length, a JSON header ``name -> {dtype, shape,
data_offsets}``, then the tensors' bytes.  The reader checks what the reference's reader
checks (``src/Inference/llama_import.jl:288-345``): the header length lies inside the file,
no key occurs twice, every span equals shape x item size, spans neither overlap nor leave
gaps nor stop short of the file's end.  Tensors are handed out as torch tensors over a
private memory map, so a large file is never read whole.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, List, Tuple

import torch

from ..config.jsonio import loads_strict
from ..errors import WeightError

_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2), "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8), "I32": (torch.int32, 4), "I16": (torch.int16, 2), "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024


class SafetensorsFile:
    """One open file: ``names()``, ``shape(name)``, ``dtype(name)``, ``tensor(name)``."""

    def __init__(self, path: str):
        self.path = path
        try:
            size = os.path.getsize(path)
            self._f = open(path, "rb")
        except OSError as err:
            raise WeightError(f"cannot open {path}: {err}", path=path) from err
        if size < 8:
            raise WeightError(f"{path}: too short for a safetensors header", size=size)
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen > _MAX_HEADER or 8 + hlen > size:
            raise WeightError(f"{path}: header length {hlen} outside the file", size=size)
        try:
            header = loads_strict(self._f.read(hlen).decode("utf-8"), what=f"{path} header")
        except Exception as err:
            raise WeightError(f"{path}: bad header: {err}") from err
        self.metadata = header.pop("__metadata__", {})
        self._data0 = 8 + hlen
        data_len = size - self._data0
        self._info: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        spans: List[Tuple[int, int, str]] = []
        for name, info in header.items():
            try:
                dt, item = _DTYPES[info["dtype"]]
            except (KeyError, TypeError):
                raise WeightError(f"{path}: tensor {name!r} has unsupported dtype {info.get('dtype') if isinstance(info, dict) else info!r}") from None
            shape = tuple(int(s) for s in info["shape"])
            b, e = (int(v) for v in info["data_offsets"])
            n = 1
            for s in shape:
                if s < 0:
                    raise WeightError(f"{path}: tensor {name!r} has a negative extent", shape=shape)
                n *= s
            if not (0 <= b <= e <= data_len) or e - b != n * item:
                raise WeightError(f"{path}: tensor {name!r} spans {e - b} bytes at [{b}, {e}), "
                                  f"its shape {shape} needs {n * item} inside {data_len}")
            self._info[name] = (dt, shape, b, e)
            spans.append((b, e, name))
        spans.sort()
        at = 0
        for b, e, name in spans:
            if b != at:
                raise WeightError(f"{path}: bytes [{at}, {b}) before tensor {name!r} "
                                  + ("overlap another tensor" if b < at else "belong to no tensor"))
            at = e
        if at != data_len:
            raise WeightError(f"{path}: {data_len - at} trailing bytes belong to no tensor")
        self._map = None

    def names(self):
        return list(self._info)

    def shape(self, name: str):
        return self._info[name][1]

    def dtype(self, name: str):
        return self._info[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        dt, shape, b, e = self._info[name]
        if e == b:
            return torch.empty(shape, dtype=dt)
        if self._map is None:
            # a private (copy-on-write) map: torch wants a writable buffer and nobody writes it
            self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_COPY)
        n = 1
        for s in shape:
            n *= s
        return torch.frombuffer(self._map, dtype=dt, count=n, offset=self._data0 + b).reshape(shape)

    def close(self):
        self._map = None
        self._f.close()


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] = None) -> None:
    """Write ``tensors`` (CPU, any supported dtype) in the given order."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    at = 0
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise WeightError(f"cannot store tensor {name!r} of type {t.dtype}")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [at, at + n]}
        at += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)
    tmp = path + f".tmp{os.getpid()}"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t in tensors.items():
            c = t.detach().cpu().contiguous()
            if c.numel():
                f.write(c.view(torch.uint8).numpy().tobytes() if c.dtype != torch.bool
                        else c.to(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)


def open_model_files(model_dir: str) -> List[SafetensorsFile]:
    """The safetensors files of a folder: one ``model.safetensors`` or the shards of an index."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(single):
        return [SafetensorsFile(single)]
    if os.path.exists(index):
        with open(index, "r", encoding="utf-8") as f:
            idx = loads_strict(f.read(), what=index)
        wm = idx.get("weight_map")
        if not isinstance(wm, dict) or not wm:
            raise WeightError(f"{index}: no weight_map")
        files = {}
        for name, fn in wm.items():
            files.setdefault(fn, []).append(name)
        out = []
        for fn in sorted(files):
            sf = SafetensorsFile(os.path.join(model_dir, fn))
            lacking = [n for n in files[fn] if n not in sf._info]
            if lacking:
                raise WeightError(f"{fn} lacks tensors the index places there", missing=lacking[:8])
            out.append(sf)
        return out
    raise WeightError(f"{model_dir} holds neither model.safetensors nor model.safetensors.index.json")
