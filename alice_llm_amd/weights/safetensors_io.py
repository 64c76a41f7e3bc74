"""Reading and writing safetensors files by tensor name.

Format: an 8-byte little-endian header length, a JSON header mapping each name
to {dtype, shape, data_offsets}, then the raw little-endian data.  The file is
memory-mapped; a tensor is a view into the map until it is copied to the device.
The reference's container is GGUF (gguf.rs:439-503, lookups 557-618); the same
three services are kept: a table of names, a bounds-checked view of a tensor's
bytes, and errors that name what is wrong.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Callable, Dict, Iterable, List, Sequence, Tuple

import torch


class WeightFileError(ValueError):
    """The file is not a readable safetensors file."""


_DTYPES = {
    "F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2),
    "F64": (torch.float64, 8), "I32": (torch.int32, 4), "I64": (torch.int64, 8),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise WeightFileError(f"{path}: truncated, {size} bytes is shorter than the header length field")
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if 8 + n > size:
            raise WeightFileError(f"{path}: truncated, header of {n} bytes does not fit in a file of {size} bytes")
        raw = self._f.read(n)
        try:
            header = json.loads(raw.decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: header is not JSON ({e})") from None
        if not isinstance(header, dict):
            raise WeightFileError(f"{path}: header is not a JSON object")
        self.metadata = header.pop("__metadata__", {})
        self._data_start = 8 + n
        data_size = size - self._data_start
        self._entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, e in header.items():
            try:
                dt, shape, (b, end) = e["dtype"], tuple(int(s) for s in e["shape"]), e["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise WeightFileError(f"{path}: malformed header entry for '{name}'") from None
            if dt not in _DTYPES:
                raise WeightFileError(f"{path}: tensor '{name}' has unknown dtype '{dt}'")
            tdt, width = _DTYPES[dt]
            count = 1
            for s in shape:
                count *= s
            if end - b != count * width:
                raise WeightFileError(f"{path}: tensor '{name}' of shape {list(shape)} and dtype {dt} "
                                      f"needs {count * width} bytes, its offsets span {end - b}")
            if b < 0 or end > data_size:
                raise WeightFileError(f"{path}: truncated, tensor '{name}' ends at byte {end} of a data "
                                      f"section of {data_size} bytes")
            self._entries[name] = (tdt, shape, b, end)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def keys(self) -> List[str]:
        return list(self._entries)

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        dt, shape, _, _ = self._entries[name]
        return dt, shape

    def tensor(self, name: str) -> torch.Tensor:
        """A read-only CPU view of the tensor's bytes in the map (copy before the file is closed)."""
        dt, shape, b, end = self._entries[name]
        if end == b:
            return torch.empty(shape, dtype=dt)
        buf = memoryview(self._map)[self._data_start + b:self._data_start + end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")            # the buffer is read-only; it is never written
            return torch.frombuffer(buf, dtype=dt).view(shape)

    def close(self) -> None:
        # Views handed out keep the map alive; closing is best effort.
        try:
            if self._map is not None:
                self._map.close()
        except BufferError:
            pass
        self._f.close()


class TensorSource:
    """The tensors of a model folder: one file, or shards named by model.safetensors.index.json."""

    def __init__(self, folder: str):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.exists(index):
            try:
                with open(index) as f:
                    weight_map = json.load(f)["weight_map"]
            except (json.JSONDecodeError, KeyError, TypeError) as e:
                raise WeightFileError(f"{index}: not a shard index ({e})") from None
            for fname in sorted(set(weight_map.values())):
                path = os.path.join(folder, fname)
                if not os.path.exists(path):
                    raise WeightFileError(f"{index}: names shard '{fname}', which is not in the folder")
                self._files[fname] = SafetensorsFile(path)
                for k in self._files[fname].keys():
                    self._where[k] = fname
        elif os.path.exists(single):
            self._files["model.safetensors"] = SafetensorsFile(single)
            for k in self._files["model.safetensors"].keys():
                self._where[k] = "model.safetensors"
        else:
            raise WeightFileError(f"{folder}: holds neither model.safetensors nor model.safetensors.index.json")

    def keys(self) -> List[str]:
        return list(self._where)

    def info(self, name: str):
        return self._files[self._where[name]].info(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._files[self._where[name]].tensor(name)

    def close(self) -> None:
        for f in self._files.values():
            f.close()


def write_safetensors(path: str, specs: Sequence[Tuple[str, torch.dtype, Sequence[int]]],
                      produce: Callable[[str], torch.Tensor], metadata: Dict[str, str] = None) -> None:
    """Write tensors in the order of `specs`, asking `produce(name)` for one at a time,
    so that a model larger than host memory can be written."""
    header = {}
    off = 0
    for name, dt, shape in specs:
        if dt not in _NAMES:
            raise WeightFileError(f"cannot store dtype {dt} of tensor '{name}'")
        count = 1
        for s in shape:
            count *= int(s)
        nbytes = count * _DTYPES[_NAMES[dt]][1]
        header[name] = {"dtype": _NAMES[dt], "shape": [int(s) for s in shape], "data_offsets": [off, off + nbytes]}
        off += nbytes
    if metadata:
        header["__metadata__"] = metadata
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for name, dt, shape in specs:
            t = produce(name)
            if tuple(t.shape) != tuple(shape) or t.dtype != dt:
                raise WeightFileError(f"producer gave {tuple(t.shape)} {t.dtype} for '{name}', "
                                      f"declared {tuple(shape)} {dt}")
            t = t.detach().contiguous().cpu()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
