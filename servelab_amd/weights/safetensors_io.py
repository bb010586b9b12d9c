"""Reader and writer for the safetensors container.

Layout: 8 bytes little-endian header length N, N bytes of JSON mapping each
tensor name to {"dtype", "shape", "data_offsets": [begin, end]} (offsets
relative to the end of the header), then the raw little-endian data.  The file
is memory-mapped; a tensor is a view until it is converted or copied to the
device.

The reference documents "safetensors single file / sharded"
(docs/architecture.md:70) but its loader is not in its tree; this is written
from the format alone.
"""
import json
import mmap
import os
import struct
from typing import Dict, Iterable, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16,
    "BF16": torch.bfloat16, "I64": torch.int64, "I32": torch.int32,
    "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        self._fh = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds file size {size}")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})")
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + hlen
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            try:
                dtype = _DTYPES[info["dtype"]]
            except KeyError:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' has unsupported dtype {info.get('dtype')!r}")
            shape = tuple(int(s) for s in info["shape"])
            begin, end = (int(x) for x in info["data_offsets"])
            numel = 1
            for s in shape:
                numel *= s
            itemsize = torch.empty((), dtype=dtype).element_size()
            if end - begin != numel * itemsize or self._data_start + end > size or begin < 0:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' shape {list(shape)} does not match its "
                    f"byte range [{begin}, {end})")
            self.entries[name] = (dtype, shape, begin, end)

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return self.entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A read-only view into the mapped file (copy before writing to it)."""
        dtype, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        numel = 1
        for s in shape:
            numel *= s
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")      # non-writable buffer notice
            flat = torch.frombuffer(self._map, dtype=dtype, count=numel,
                                    offset=self._data_start + begin)
        return flat.view(shape)


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata=None) -> None:
    """Write tensors in the order given (contiguous, CPU)."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    items = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}': dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        items.append(t)
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for t in items:
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                        t.reshape(1).view(torch.uint8).numpy().tobytes())
