"""Reader and writer of the safetensors container.

Container: 8-byte little-endian header length, a JSON object (``__metadata__`` plus one
entry ``{dtype, shape, data_offsets}`` per tensor), then the data section
(`src/format/safetensors.zig:188-234,250-283`).  The reader maps the file and checks the
layout as the reference does (`:285-327`): every tensor inside the data section, byte size
equal to shape x dtype size, no overlap, no holes, the section fully covered.  Error names are
the reference's (`:38,139-156,193-204,241-245,255-275,302-336`).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

from ..errors import FormatError

# dtype name -> bytes per element (`src/format/safetensors.zig:3-70`)
DTYPE_SIZES = {"BOOL": 1, "U8": 1, "I8": 1, "F8_E5M2": 1, "F8_E4M3": 1, "I16": 2, "U16": 2,
               "F16": 2, "BF16": 2, "I32": 4, "U32": 4, "F32": 4, "F64": 8, "I64": 8, "U64": 8}
_NUMPY = {"F32": np.float32, "BF16": np.uint16, "F16": np.float16, "I32": np.int32,
          "I64": np.int64, "U8": np.uint8, "I8": np.int8, "F64": np.float64, "I16": np.int16,
          "U16": np.uint16, "U32": np.uint32, "U64": np.uint64, "BOOL": np.bool_}
MAX_HEADER_BYTES = 100 * 1024 * 1024


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int
    end: int

    @property
    def numel(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n


def _as_index(v, what: str) -> int:
    if isinstance(v, bool) or not isinstance(v, int):
        if isinstance(v, float):
            raise FormatError("InvalidIntegerValue", f"{what}: {v!r}")
        raise FormatError("InvalidTensorField", f"{what}: {v!r}")
    if v < 0:
        raise FormatError("InvalidIntegerValue", f"{what}: {v}")
    return v


def parse_header(header: bytes, data_len: int) -> Tuple[Dict[str, TensorInfo], Dict[str, str]]:
    try:
        root = json.loads(header.decode("utf-8").rstrip(" "))
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise FormatError("InvalidHeaderJson", str(e)) from None
    if not isinstance(root, dict):
        raise FormatError("InvalidHeaderJson", "the header's root is not an object")
    metadata: Dict[str, str] = {}
    infos: Dict[str, TensorInfo] = {}
    for name, entry in root.items():
        if name == "__metadata__":
            if not isinstance(entry, dict) or any(not isinstance(v, str) for v in entry.values()):
                raise FormatError("InvalidMetadataEntry", repr(entry)[:80])
            metadata = dict(entry)
            continue
        if not isinstance(entry, dict):
            raise FormatError("InvalidTensorEntry", name)
        for key in ("dtype", "shape", "data_offsets"):
            if key not in entry:
                raise FormatError("MissingTensorField", f"{name}: {key}")
        if not isinstance(entry["dtype"], str):
            raise FormatError("InvalidTensorField", f"{name}: dtype")
        if entry["dtype"] not in DTYPE_SIZES:
            raise FormatError("UnsupportedDType", f"{name}: {entry['dtype']}")
        if not isinstance(entry["shape"], list):
            raise FormatError("InvalidTensorField", f"{name}: shape")
        shape = tuple(_as_index(d, f"{name}: shape") for d in entry["shape"])
        offs = entry["data_offsets"]
        if not isinstance(offs, list) or len(offs) != 2:
            raise FormatError("InvalidTensorField", f"{name}: data_offsets")
        begin = _as_index(offs[0], f"{name}: data_offsets")
        end = _as_index(offs[1], f"{name}: data_offsets")
        if end < begin:
            raise FormatError("InvalidDataOffsets", f"{name}: {begin}..{end}")
        infos[name] = TensorInfo(name, entry["dtype"], shape, begin, end)
    # layout validation
    for info in infos.values():
        if info.end > data_len:
            raise FormatError("TensorOutOfBounds", f"{info.name}: ends at {info.end}, the data "
                              f"section has {data_len} bytes")
        if info.numel * DTYPE_SIZES[info.dtype] != info.end - info.begin:
            raise FormatError("TensorByteSizeMismatch",
                              f"{info.name}: shape {list(info.shape)} of {info.dtype} needs "
                              f"{info.numel * DTYPE_SIZES[info.dtype]} bytes, has "
                              f"{info.end - info.begin}")
    cursor = 0
    for info in sorted(infos.values(), key=lambda i: (i.begin, i.end)):
        if info.begin < cursor:
            raise FormatError("OverlappingTensorData", info.name)
        if info.begin > cursor:
            raise FormatError("NonContiguousTensorData", f"hole before {info.name}")
        cursor = info.end
    if cursor != data_len:
        raise FormatError("NonContiguousTensorData",
                          f"{data_len - cursor} bytes at the end belong to no tensor")
    return infos, metadata


class SafetensorsFile:
    """A mapped safetensors file; ``tensor(name)`` copies one tensor out as a torch tensor."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            self._f.close()
            raise FormatError("InvalidSafetensorsFile", f"{path}: {size} bytes")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._mm[:8])
        if hlen > MAX_HEADER_BYTES:
            self.close()
            raise FormatError("HeaderTooLarge", f"{path}: {hlen}")
        if 8 + hlen > size:
            self.close()
            raise FormatError("InvalidHeaderLength", f"{path}: header of {hlen} bytes in a file "
                              f"of {size}")
        self._data_start = 8 + hlen
        try:
            self.infos, self.metadata = parse_header(bytes(self._mm[8:8 + hlen]),
                                                     size - self._data_start)
        except FormatError:
            self.close()
            raise

    def close(self) -> None:
        try:
            self._mm.close()
        except Exception:
            pass
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def names(self) -> List[str]:
        return list(self.infos)

    def tensor(self, name: str) -> torch.Tensor:
        info = self.infos[name]
        if info.dtype not in _NUMPY:
            raise FormatError("UnsupportedDType", f"{name}: {info.dtype} cannot be read")
        arr = np.frombuffer(self._mm, dtype=_NUMPY[info.dtype], count=info.numel,
                            offset=self._data_start + info.begin).reshape(info.shape).copy()
        t = torch.from_numpy(arr)
        if info.dtype == "BF16":
            t = t.view(torch.bfloat16)
        return t


_TORCH_TO_NAME = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16",
                  torch.int32: "I32", torch.int64: "I64", torch.uint8: "U8", torch.int8: "I8",
                  torch.float64: "F64", torch.int16: "I16", torch.bool: "BOOL"}


def _raw_bytes(t: torch.Tensor) -> bytes:
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().tobytes()
    return t.numpy().tobytes()


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor],
                      metadata: Dict[str, str] = None) -> None:
    """Writes ``tensors`` in the order given, tightly packed, header padded with spaces to a
    multiple of 8 bytes."""
    header = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    for name, t in tensors.items():
        if t.dtype not in _TORCH_TO_NAME:
            raise FormatError("UnsupportedDType", f"{name}: {t.dtype}")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _TORCH_TO_NAME[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + n]}
        offset += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for t in tensors.values():
            f.write(_raw_bytes(t))
    os.replace(tmp, path)
