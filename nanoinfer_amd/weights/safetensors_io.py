"""Reading and writing the safetensors container without a third-party reader.

Layout (as drawn in the reference's design note, docs/optimization_roadmap.md:522-536): eight
bytes of little-endian header length, that many bytes of JSON mapping each tensor name to
``{"dtype", "shape", "data_offsets": [begin, end]}`` with offsets counted from the first byte
after the header, then the data.  The file is memory-mapped; a tensor is a view of the map until
it is copied to the GPU.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterator, List, Tuple

import numpy as np
import torch


class WeightFileError(ValueError):
    pass


# tag -> (torch dtype, bytes per element, numpy dtype used to view the bytes)
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
_TAG_OF = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """An open, memory-mapped safetensors file: names, shapes, types, and tensors by name."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise WeightFileError(f"no weight file at {path!r}")
        size = os.path.getsize(path)
        if size < 8:
            raise WeightFileError(f"{path}: {size} bytes is too short for a safetensors header")
        self._fh = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise WeightFileError(f"{path}: header length {hlen} does not fit a file of {size} bytes")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: the header is not JSON: {e}") from e
        self.metadata = header.pop("__metadata__", None)
        self._data_start = 8 + hlen
        self._entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        data_len = size - self._data_start
        for name, info in header.items():
            try:
                tag, shape, (b, e) = info["dtype"], tuple(int(s) for s in info["shape"]), info["data_offsets"]
            except (KeyError, TypeError, ValueError) as ex:
                raise WeightFileError(f"{path}: malformed entry for {name!r}: {info}") from ex
            if tag not in _DTYPES:
                raise WeightFileError(f"{path}: tensor {name!r} has the unsupported type {tag!r}")
            n = 1
            for s in shape:
                n *= s
            if e - b != n * _DTYPES[tag][1]:
                raise WeightFileError(f"{path}: tensor {name!r} of shape {shape} and type {tag} should take "
                                      f"{n * _DTYPES[tag][1]} bytes, its offsets give {e - b}")
            if b < 0 or e > data_len:
                raise WeightFileError(f"{path}: tensor {name!r} ends at byte {e} of a data region of {data_len} "
                                      "bytes (truncated file?)")
            self._entries[name] = (tag, shape, b, e)
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> List[str]:
        return list(self._entries)

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._entries[name][0]][0]

    def tensor(self, name: str) -> torch.Tensor:
        """The tensor as stored (a CPU tensor over the mapped bytes; do not write to it)."""
        tag, shape, b, e = self._entries[name]
        tdtype, _, ndtype = _DTYPES[tag]
        n = 1
        for s in shape:
            n *= s
        arr = np.frombuffer(self._map, dtype=ndtype, count=n, offset=self._data_start + b)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the mapped array is read-only
            t = torch.from_numpy(arr)
        if tag == "BF16":
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def items(self) -> Iterator[Tuple[str, torch.Tensor]]:
        for name in self._entries:
            yield name, self.tensor(name)

    def close(self) -> None:
        # views handed out keep the map alive; dropping our references is all that is needed
        self._map = None
        self._fh.close()


def _raw(t: torch.Tensor) -> memoryview:
    """The bytes of a contiguous CPU tensor, without a copy."""
    t = t.detach().contiguous()
    arr = t.view(torch.uint16).numpy() if t.dtype == torch.bfloat16 else t.numpy()
    return memoryview(arr.reshape(-1)).cast("B")


def write_safetensors_streamed(path: str, entries, metadata: Dict[str, str] = None) -> None:
    """Write tensors that are produced piece by piece.  ``entries`` is a list of ``(name, dtype,
    shape, pieces)``; ``pieces()`` returns an iterator of flat CPU tensors of that type which
    together hold the tensor's elements in order.  The header is written first, from the shapes
    alone, and every piece goes to the file as it comes: no tensor is ever held whole, so a model
    larger than the host's memory can be written (the reference's loader, for contrast, maps views
    of a file that an exporter held whole: src/model/llama.cpp:568-706)."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    sizes = []
    for name, dtype, shape, _ in entries:
        if dtype not in _TAG_OF:
            raise WeightFileError(f"tensor {name!r}: type {dtype} cannot be stored")
        n = 1
        for d in shape:
            n *= int(d)
        nbytes = n * _DTYPES[_TAG_OF[dtype]][1]
        if name in header:
            raise WeightFileError(f"tensor {name!r} is listed twice")
        header[name] = {"dtype": _TAG_OF[dtype], "shape": [int(d) for d in shape], "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        sizes.append(nbytes)
    hjson = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hjson += b" " * ((8 - len(hjson) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as fh:
        fh.write(struct.pack("<Q", len(hjson)))
        fh.write(hjson)
        for (name, dtype, shape, pieces), nbytes in zip(entries, sizes):
            written = 0
            for piece in pieces():
                if piece.dtype != dtype:
                    raise WeightFileError(f"tensor {name!r}: a piece of type {piece.dtype} for a tensor of type {dtype}")
                raw = _raw(piece)
                fh.write(raw)
                written += len(raw)
            if written != nbytes:
                raise WeightFileError(f"tensor {name!r} of shape {tuple(shape)} takes {nbytes} bytes, its pieces gave {written}")
    os.replace(tmp, path)


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] = None) -> None:
    """Write CPU tensors under their names, in the given order, 8-byte aligned header."""
    entries = []
    for name, t in tensors.items():
        t = t.detach().cpu()
        entries.append((name, t.dtype, tuple(t.shape), lambda t=t: iter([t.reshape(-1)])))
    write_safetensors_streamed(path, entries, metadata)
