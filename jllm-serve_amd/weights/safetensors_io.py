"""Memory-mapped safetensors reader and a writer.

Format (safetensors/SafeTensors.java:23-29): u64 little-endian header length N, N bytes of JSON
``{name: {dtype, shape, data_offsets: [begin, end]}, "__metadata__": {...}}``, then the raw data; offsets
are relative to the first byte after the header. The whole file is mapped and tensors are views into the
map (:228-258, :341-348). Header validation follows :269-362; a folder is read through
``model.safetensors.index.json``'s ``weight_map`` when present, else every ``*.safetensors`` file in
sorted order (:198-225).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Mapping, Tuple

import torch

MAX_HEADER_BYTES = 100 * 1024 * 1024

_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2), "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8), "I32": (torch.int32, 4), "I16": (torch.int16, 2), "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(IOError):
    pass


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    begin: int  # absolute byte offset in the file
    nbytes: int
    file: str


class SafetensorsFile:
    """One mapped file. ``tensor(name)`` returns a CPU tensor that views the map (zero copy)."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too small to be a safetensors file ({size} bytes)")
        self._fh = open(path, "rb")
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        (n,) = struct.unpack("<Q", self._map[:8])
        if n <= 0 or n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} is not inside the file ({size} bytes)")
        if n > MAX_HEADER_BYTES:
            raise SafetensorsError(f"{path}: header of {n} bytes exceeds the limit of {MAX_HEADER_BYTES}")
        try:
            header = json.loads(self._map[8:8 + n].decode("utf-8"), object_pairs_hook=_no_duplicates)
        except SafetensorsError as e:
            raise SafetensorsError(f"{path}: {e}") from None
        except (ValueError, UnicodeDecodeError) as e:
            raise SafetensorsError(f"{path}: invalid header JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: the header is not a JSON object")
        data_start = 8 + n
        data_size = size - data_start
        self.metadata = header.get("__metadata__") or {}
        self.tensors: Dict[str, TensorInfo] = {}
        ranges: List[Tuple[int, int, str]] = []
        for name, e in header.items():
            if name == "__metadata__":
                continue
            if not isinstance(e, dict) or "shape" not in e or "data_offsets" not in e:
                raise SafetensorsError(f"{path}: malformed entry for tensor '{name}'")
            dt = e.get("dtype")
            if not isinstance(dt, str):
                raise SafetensorsError(f"{path}: tensor '{name}' has no dtype")
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
            shape = e["shape"]
            offs = e["data_offsets"]
            if not isinstance(shape, list) or not all(isinstance(d, int) and not isinstance(d, bool) for d in shape):
                raise SafetensorsError(f"{path}: malformed shape for tensor '{name}'")
            if any(d < 0 for d in shape):
                raise SafetensorsError(f"{path}: tensor '{name}' has a negative dimension {shape}")
            numel = 1
            for d in shape:
                numel *= d
                if numel > 2**62:
                    raise SafetensorsError(f"{path}: shape of tensor '{name}' overflows {shape}")
            if (not isinstance(offs, list) or len(offs) != 2
                    or not all(isinstance(o, int) and not isinstance(o, bool) for o in offs)):
                raise SafetensorsError(f"{path}: malformed data_offsets for tensor '{name}'")
            b, en = offs
            tdtype, width = _DTYPES[dt]
            if b < 0 or en < b or en > data_size or en - b != numel * width:
                raise SafetensorsError(
                    f"{path}: data_offsets {offs} of tensor '{name}' do not fit shape {shape} of {dt} "
                    f"({numel * width} bytes) inside {data_size} data bytes")
            self.tensors[name] = TensorInfo(name, tdtype, tuple(shape), data_start + b, en - b, path)
            if en > b:
                ranges.append((b, en, name))
        ranges.sort()
        for (b0, e0, n0), (b1, e1, n1) in zip(ranges, ranges[1:]):
            if b1 < e0:
                raise SafetensorsError(f"{path}: tensors '{n0}' and '{n1}' overlap")

    def names(self) -> List[str]:
        return list(self.tensors)

    def tensor(self, name: str) -> torch.Tensor:
        if name not in self.tensors:
            raise SafetensorsError(f"tensor not found: {name}")
        t = self.tensors[name]
        numel = 1
        for d in t.shape:
            numel *= d
        if numel == 0:
            return torch.empty(t.shape, dtype=t.dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the map is read-only; the tensor is only ever read
            flat = torch.frombuffer(self._map, dtype=t.dtype, count=numel, offset=t.begin)
        return flat.view(t.shape)

    def close(self) -> None:
        try:
            self._map.close()
        except (BufferError, ValueError):
            pass  # tensors still view the map; it is released with them
        self._fh.close()


def _no_duplicates(pairs):
    out = {}
    for k, v in pairs:
        if k in out:
            raise SafetensorsError(f"duplicate tensor '{k}'")
        out[k] = v
    return out


class SafetensorsSource:
    """All tensors of a model folder (or one file), by name (safetensors/SafeTensors.java:198-258)."""

    def __init__(self, path: str):
        self.path = path
        self.files: List[SafetensorsFile] = []
        self._where: Dict[str, SafetensorsFile] = {}
        if os.path.isdir(path):
            index = os.path.join(path, "model.safetensors.index.json")
            if os.path.exists(index):
                try:
                    with open(index, "r", encoding="utf-8") as f:
                        idx = json.load(f)
                except ValueError as e:
                    raise SafetensorsError(f"{index}: {e}") from None
                wm = idx.get("weight_map") if isinstance(idx, dict) else None
                if not isinstance(wm, dict):
                    raise SafetensorsError(f"{index}: no weight_map")
                shard_names = sorted(set(wm.values()))
                for s in shard_names:
                    _check_shard_name(index, s)
            else:
                shard_names = sorted(f for f in os.listdir(path) if f.endswith(".safetensors"))
                if not shard_names:
                    raise SafetensorsError(f"no .safetensors files in {path}")
            paths = [os.path.join(path, s) for s in shard_names]
        else:
            paths = [path]
        for p in paths:
            if not os.path.exists(p):
                raise SafetensorsError(f"{p}: no such file")
            f = SafetensorsFile(p)
            self.files.append(f)
            for n in f.names():
                if n in self._where:
                    raise SafetensorsError(f"duplicate tensor '{n}' in {p} and {self._where[n].path}")
                self._where[n] = f

    def names(self) -> List[str]:
        return list(self._where)

    def info(self, name: str) -> TensorInfo:
        return self._where[name].tensors[name]

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.info(name).shape

    def dtype(self, name: str) -> torch.dtype:
        return self.info(name).dtype

    def get(self, name: str) -> torch.Tensor:
        if name not in self._where:
            raise SafetensorsError(f"tensor not found: {name}")
        return self._where[name].tensor(name)

    def close(self) -> None:
        for f in self.files:
            f.close()


def _check_shard_name(index: str, s) -> None:
    """model/ShardProvider.java:35-51: a plain file name ending in .safetensors."""
    if (not isinstance(s, str) or not s.endswith(".safetensors") or "/" in s or "\\" in s or ".." in s or "\0" in s
            or not s):
        raise SafetensorsError(f"{index}: bad shard name {s!r}")


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] = None) -> None:
    """Writes ``tensors`` in the given order; the header is padded with spaces to a multiple of 8 bytes
    (as scripts/make-tiny-model.py:805-822 does)."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    order: List[Tuple[str, torch.Tensor]] = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot write tensor '{name}' of dtype {t.dtype}")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
        order.append((name, t))
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for _, t in order:
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
