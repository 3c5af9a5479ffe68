"""Reading and writing safetensors files: an 8-byte little-endian header length, a JSON header
``{name: {dtype, shape, data_offsets}, "__metadata__": {...}}`` and the raw little-endian
tensor bytes.  Files are memory-mapped and tensors are views into the map, so a large
checkpoint is never read whole.  (The reference maps every ``*.safetensors`` of a model
folder as one namespace: crates/model/src/llama.rs:125-138.)"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, List, Optional, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped file; ``entries`` maps tensor name to (dtype name, shape, begin, end)."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"{path}: {e.strerror}") from None
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen > size - 8:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds the file size {size}")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
        self.metadata = header.pop("__metadata__", None) or {}
        self._base = 8 + hlen
        data_len = size - self._base
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            try:
                dt, shape = info["dtype"], tuple(int(s) for s in info["shape"])
                begin, end = (int(o) for o in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed header entry for '{name}'") from None
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unknown dtype '{dt}'")
            n = 1
            for s in shape:
                n *= s
            want = n * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if not (0 <= begin <= end <= data_len) or end - begin != want:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' ({dt} {list(shape)}) has data offsets "
                    f"[{begin}, {end}) that do not fit its size {want} or the file ({data_len} "
                    "bytes of data): the file is truncated or corrupt")
            self.entries[name] = (dt, shape, begin, end)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self) -> List[str]:
        return list(self.entries)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        dt, shape, _, _ = self.entries[name]
        return _DTYPES[dt], shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped bytes (read-only: clone before writing)."""
        dt, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=_DTYPES[dt])
        buf = memoryview(self._map)[self._base + begin:self._base + end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")   # the map is read-only; callers copy
            t = torch.frombuffer(buf, dtype=_DTYPES[dt])
        return t.reshape(shape)


def open_folder(folder: str) -> List[SafetensorsFile]:
    """Every ``*.safetensors`` of a folder, sorted by name (llama.rs:126-135)."""
    try:
        files = sorted(f for f in os.listdir(folder) if f.endswith(".safetensors"))
    except OSError as e:
        raise SafetensorsError(f"{folder}: {e.strerror}") from None
    if not files:
        raise SafetensorsError(f"no .safetensors files in {folder}")
    return [SafetensorsFile(os.path.join(folder, f)) for f in files]


def save_file(tensors: Dict[str, torch.Tensor], path: str,
              metadata: Optional[Dict[str, str]] = None) -> None:
    """Write ``tensors`` (CPU or GPU, any of the known dtypes) to ``path``."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}' has dtype {t.dtype}, which safetensors lacks")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + n]}
        offset += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)
    tmp = path + f".tmp{os.getpid()}"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                        t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
