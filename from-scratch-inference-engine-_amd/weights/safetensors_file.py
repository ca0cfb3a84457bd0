"""Reader and writer of the safetensors container, with the format checks of the reference.

Layout: 8 bytes little-endian header length, a JSON header {name: {dtype, shape, data_offsets}},
then the raw little-endian tensor data.  The reader maps the file and hands out tensors that
alias the mapping (no copy until the caller converts or moves them).
"""

from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path
from typing import Dict, Mapping, Tuple

import torch


class SafetensorsError(RuntimeError):
    pass


_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


def _itemsize(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class SafetensorsFile:
    """One mapped .safetensors file.

    The checks are those of the reference's parser (src/model/safetensors.cpp:23-111): header
    length within the file, valid JSON, known dtype, offsets inside the data region and in
    order, non-negative dimensions, byte count equal to the shape's (checked by division),
    no overlapping regions.  Unlike the reference, tensors are not converted to float32 here.
    """

    def __init__(self, path):
        self.path = Path(path)
        if not self.path.is_file():
            raise SafetensorsError(f"safetensors: no such file {self.path}")
        self._file = open(self.path, "rb")
        size = self.path.stat().st_size
        if size < 8:
            raise SafetensorsError("safetensors: file smaller than the 8-byte header length")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        (header_len,) = struct.unpack("<Q", self._map[:8])
        if header_len > size - 8:
            raise SafetensorsError("safetensors: header length exceeds the file")
        try:
            pairs = json.loads(self._map[8:8 + header_len].decode("utf-8"),
                               object_pairs_hook=lambda p: p)
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise SafetensorsError(f"safetensors: invalid header JSON: {e}") from e
        if not isinstance(pairs, list):
            raise SafetensorsError("safetensors: header must be a JSON object")
        self._base = 8 + header_len
        region = size - self._base
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        spans = []
        for name, meta in pairs:
            if name == "__metadata__":
                continue
            if name in self.entries:
                raise SafetensorsError(f"safetensors: duplicate tensor name '{name}'")
            try:
                meta = dict(meta)
                dtype_name, shape, offsets = meta["dtype"], meta["shape"], meta["data_offsets"]
                begin, end = int(offsets[0]), int(offsets[1])
                shape = tuple(int(d) for d in shape)
            except (KeyError, TypeError, ValueError, IndexError) as e:
                raise SafetensorsError(f"safetensors: malformed header entry '{name}': {e}") from e
            if dtype_name not in _DTYPES:
                raise SafetensorsError(f"safetensors: unsupported dtype '{dtype_name}' for {name}")
            dtype = _DTYPES[dtype_name]
            if begin < 0 or end < begin or end > region:
                raise SafetensorsError(f"safetensors: data_offsets out of range for {name}")
            if any(d < 0 for d in shape):
                raise SafetensorsError(f"safetensors: negative dimension for {name}")
            numel = 1
            for d in shape:
                numel *= d
            item = _itemsize(dtype)
            nbytes = end - begin
            if nbytes % item or nbytes // item != numel:
                raise SafetensorsError(f"safetensors: byte count does not match shape for {name}")
            self.entries[name] = (dtype, shape, begin, end)
            spans.append((begin, end))
        spans.sort()
        for (b0, e0), (b1, _) in zip(spans, spans[1:]):
            if b1 < e0:
                raise SafetensorsError("safetensors: overlapping tensor data regions")

    def names(self):
        return list(self.entries.keys())

    def __contains__(self, name: str) -> bool:
        return name in self.entries

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return self.entries[name][0]

    def get(self, name: str) -> torch.Tensor:
        """The stored tensor, in its stored dtype, aliasing the mapped file (read-only)."""
        if name not in self.entries:
            raise SafetensorsError(f"safetensors: missing tensor '{name}'")
        dtype, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        view = memoryview(self._map)[self._base + begin:self._base + end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the buffer is not writable
            flat = torch.frombuffer(view, dtype=dtype)
        return flat.reshape(shape)

    def close(self):
        # tensors handed out may still alias the mapping; closing is left to the collector
        pass


def write_safetensors(path, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] | None = None):
    """Write ``tensors`` (CPU, any supported dtype) in name order."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors.keys())
    blobs = []
    for name in order:
        t = tensors[name].detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"safetensors: cannot store dtype {t.dtype} ({name})")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        blobs.append(t)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * ((8 - len(text) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for t in blobs:
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())
