"""Reader and writer of the safetensors container.

The file is an 8-byte little-endian header length, a JSON header that maps each
tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets
relative to the end of the header), and the raw little-endian tensor bytes.
The reader maps the file and hands out tensors that view the mapping, so a
large checkpoint is never held twice in host memory.

The reference reads the same container through the ``safetensors`` crate and
checks names, shapes and dtypes itself
(/root/reference/crates/nnis-model/src/safetensors_loader.rs:689-753).
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

from ..errors import WeightError

_DTYPE_OF = {
    "F32": torch.float32,
    "BF16": torch.bfloat16,
    "F16": torch.float16,
    "F64": torch.float64,
    "I64": torch.int64,
    "I32": torch.int32,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAME_OF = {v: k for k, v in _DTYPE_OF.items()}
_MAX_HEADER = 100 * 1024 * 1024


class SafetensorsFile:
    """One mapped safetensors file.  ``entries`` maps a tensor name to
    ``(dtype_name, shape)``; ``tensor(name)`` returns a CPU tensor that views
    the mapping (read-only by contract: do not write through it)."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._file = open(path, "rb")
        except OSError as error:
            raise WeightError(f"cannot open {path}: {error}") from None
        size = os.fstat(self._file.fileno()).st_size
        if size < 8:
            raise WeightError(f"{path}: too short to be a safetensors file ({size} bytes)")
        (header_len,) = struct.unpack("<Q", self._file.read(8))
        if header_len > _MAX_HEADER or 8 + header_len > size:
            raise WeightError(f"{path}: malformed safetensors header length {header_len}")
        try:
            header = json.loads(self._file.read(header_len).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as error:
            raise WeightError(f"{path}: malformed safetensors header: {error}") from None
        if not isinstance(header, dict):
            raise WeightError(f"{path}: safetensors header is not a JSON object")
        self._data_start = 8 + header_len
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_COPY)
        self.metadata = header.pop("__metadata__", {})
        self._entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        data_size = size - self._data_start
        for name, info in header.items():
            try:
                dtype = info["dtype"]
                shape = tuple(int(d) for d in info["shape"])
                begin, end = (int(o) for o in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightError(f"{path}: malformed header entry for tensor {name}") from None
            if dtype not in _DTYPE_OF:
                raise WeightError(f"{path}: tensor {name} has unsupported dtype {dtype}")
            count = 1
            for d in shape:
                count *= d
            expect = count * torch.empty((), dtype=_DTYPE_OF[dtype]).element_size()
            if begin < 0 or end < begin or end > data_size or end - begin != expect:
                raise WeightError(
                    f"{path}: tensor {name} byte range [{begin}, {end}) does not fit "
                    f"dtype {dtype} shape {list(shape)} ({expect} bytes) in {data_size} data bytes"
                )
            self._entries[name] = (dtype, shape, begin, end)

    @property
    def entries(self) -> Dict[str, Tuple[str, Tuple[int, ...]]]:
        return {name: (e[0], e[1]) for name, e in self._entries.items()}

    def names(self) -> List[str]:
        return list(self._entries)

    def tensor(self, name: str) -> torch.Tensor:
        dtype, shape, begin, end = self._entries[name]
        count = 1
        for d in shape:
            count *= d
        if count == 0:
            return torch.empty(shape, dtype=_DTYPE_OF[dtype])
        flat = torch.frombuffer(self._map, dtype=_DTYPE_OF[dtype], count=count, offset=self._data_start + begin)
        return flat.view(shape)

    def close(self) -> None:
        """Closes the file.  The mapping stays valid for as long as a tensor
        handed out views it, and is released with the last of them."""
        self._file.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata: Dict[str, str] = None) -> None:
    """Writes ``(name, tensor)`` pairs in the order given."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    blobs: List[bytes] = []
    offset = 0
    for name, tensor in tensors:
        if name in header:
            raise WeightError(f"duplicate tensor name {name}")
        if tensor.dtype not in _NAME_OF:
            raise WeightError(f"tensor {name}: dtype {tensor.dtype} cannot be stored")
        t = tensor.detach().cpu().contiguous()
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {
            "dtype": _NAME_OF[tensor.dtype],
            "shape": list(t.shape),
            "data_offsets": [offset, offset + len(raw)],
        }
        offset += len(raw)
        blobs.append(raw)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * ((8 - len(text) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as handle:
        handle.write(struct.pack("<Q", len(text)))
        handle.write(text)
        for raw in blobs:
            handle.write(raw)
    os.replace(tmp, path)
