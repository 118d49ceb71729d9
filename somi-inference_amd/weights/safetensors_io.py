"""Reading and writing of ``.safetensors`` files by tensor name.

The format is: eight bytes (little-endian u64) with the length of a JSON
header, the header (``name -> {dtype, shape, data_offsets}``), then the raw
little-endian tensor bytes.  The reference never touches the file format; it
goes through a library model object's ``state_dict()``
(somi_inference/models/qwen2_adapter.py:228-229).  Reading the file directly
lets the loader stream one tensor at a time to the GPU and report every
missing or misshapen tensor before anything is copied.
"""

from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass

import numpy as np
import torch

_TORCH_OF = {
    "BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_CODE_OF = {v: k for k, v in _TORCH_OF.items()}
_ITEMSIZE = {"BF16": 2, "F16": 2, "F32": 4, "F64": 8, "I64": 8, "I32": 4, "I16": 2, "I8": 1,
             "U8": 1, "BOOL": 1}


class SafetensorsError(ValueError):
    """The file is not a well-formed safetensors file."""


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: tuple[int, ...]
    begin: int          # absolute byte offsets in the file
    end: int
    path: str


def read_header(path: str) -> dict[str, TensorEntry]:
    size = os.path.getsize(path)
    with open(path, "rb") as handle:
        head = handle.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header")
        (length,) = struct.unpack("<Q", head)
        if length <= 0 or 8 + length > size:
            raise SafetensorsError(f"{path}: header length {length} does not fit the file ({size} bytes)")
        try:
            header = json.loads(handle.read(length).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as err:
            raise SafetensorsError(f"{path}: header is not valid JSON ({err})") from err
    base = 8 + length
    entries: dict[str, TensorEntry] = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        code = meta.get("dtype")
        if code not in _TORCH_OF:
            raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {code!r}")
        shape = tuple(int(s) for s in meta["shape"])
        begin, end = (int(x) for x in meta["data_offsets"])
        count = 1
        for s in shape:
            count *= s
        if end - begin != count * _ITEMSIZE[code] or base + end > size or begin < 0:
            raise SafetensorsError(
                f"{path}: tensor {name!r} of shape {shape} and dtype {code} does not match its "
                f"byte range [{begin}, {end})")
        entries[name] = TensorEntry(name, _TORCH_OF[code], shape, base + begin, base + end, path)
    return entries


def read_tensor(entry: TensorEntry) -> torch.Tensor:
    """One tensor as a host tensor of its stored dtype (a private copy of the bytes)."""
    nbytes = entry.end - entry.begin
    if nbytes == 0:
        return torch.empty(entry.shape, dtype=entry.dtype)
    raw = np.fromfile(entry.path, dtype=np.uint8, count=nbytes, offset=entry.begin)
    return torch.from_numpy(raw).view(entry.dtype).reshape(entry.shape)


def write_file(path: str, tensors: dict[str, torch.Tensor], metadata: dict[str, str] | None = None) -> None:
    """Write tensors (any device) under their names, in the given order."""
    header: dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, tensor in tensors.items():
        if tensor.dtype not in _CODE_OF:
            raise SafetensorsError(f"tensor {name!r}: dtype {tensor.dtype} cannot be stored")
        nbytes = tensor.numel() * tensor.element_size()
        header[name] = {"dtype": _CODE_OF[tensor.dtype], "shape": list(tensor.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)))
        handle.write(blob)
        for tensor in tensors.values():
            host = tensor.detach().contiguous().cpu()
            handle.write(host.view(torch.uint8).numpy().tobytes() if host.numel() else b"")
    os.replace(tmp, path)
