"""Reading and writing safetensors files without any library beside numpy and torch.

Format (as read by the reference's converter, tools/convert.py:41-50): an 8-byte
little-endian header length n, n bytes of JSON ``{name: {"dtype", "shape",
"data_offsets": [start, end]}}`` (the ``__metadata__`` entry is dropped), then the data
region, to which the offsets are relative.  Files are memory-mapped; tensors are views.
"""

from __future__ import annotations

import json
import struct
from pathlib import Path
from typing import Dict, Iterable, Tuple

import numpy as np
import torch

_NP_OF = {"F32": np.float32, "F16": np.float16, "BF16": np.uint16, "I32": np.int32, "I64": np.int64}
_TORCH_TAG = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
              torch.int32: "I32", torch.int64: "I64"}


class SafetensorsError(ValueError):
    pass


def read_header(path: Path) -> Tuple[Dict[str, dict], int]:
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", head)
        size = path.stat().st_size
        if n <= 0 or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} does not fit the file ({size} bytes)")
        try:
            header = json.loads(f.read(n))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
    header.pop("__metadata__", None)
    return header, 8 + n


def read_file(path: str | Path) -> Dict[str, torch.Tensor]:
    """All tensors of one file as CPU tensors viewing the memory map (BF16 as bfloat16)."""
    path = Path(path)
    header, base = read_header(path)
    data = np.memmap(path, dtype=np.uint8, mode="r")
    out: Dict[str, torch.Tensor] = {}
    spans = []
    for name, info in header.items():
        tag = info["dtype"]
        if tag not in _NP_OF:
            raise SafetensorsError(f"{path}: unsupported dtype {tag} for {name}")
        start, end = (int(v) for v in info["data_offsets"])
        shape = tuple(int(s) for s in info["shape"])
        if any(s < 0 for s in shape) or not 0 <= start <= end:
            raise SafetensorsError(f"{path}: tensor {name} has a negative size or offsets that run backwards")
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        item = np.dtype(_NP_OF[tag]).itemsize
        if end - start != count * item or base + end > data.size:
            raise SafetensorsError(f"{path}: truncated tensor {name}")
        if end > start:
            spans.append((start, end, name))
        arr = np.frombuffer(data, dtype=_NP_OF[tag], count=count, offset=base + start).reshape(shape)
        t = torch.from_numpy(arr)
        if tag == "BF16":
            t = t.view(torch.int16).view(torch.bfloat16)
        out[name] = t
    spans.sort()
    for (_, e0, n0), (s1, _, n1) in zip(spans, spans[1:]):
        if s1 < e0:
            raise SafetensorsError(f"{path}: tensors {n0} and {n1} overlap")
    return out


def read_folder(folder: str | Path) -> Dict[str, torch.Tensor]:
    """Tensors of every ``*.safetensors`` shard of a model folder, shards in sorted order."""
    folder = Path(folder)
    shards = sorted(folder.glob("*.safetensors"))
    if not shards:
        raise SafetensorsError(f"cannot open {folder}: no *.safetensors file in it")
    out: Dict[str, torch.Tensor] = {}
    for shard in shards:
        out.update(read_file(shard))
    return out


def write_file(path: str | Path, tensors: Iterable[Tuple[str, torch.Tensor]]) -> None:
    """Write (name, tensor) pairs in the given order, back to back (the format allows no gaps)."""
    path = Path(path)
    header: Dict[str, dict] = {}
    blobs = []
    offset = 0
    for name, t in tensors:
        if t.dtype not in _TORCH_TAG:
            raise SafetensorsError(f"cannot store dtype {t.dtype} of {name}")
        t = t.detach().contiguous().cpu()
        raw = t.view(torch.int16).numpy().tobytes() if t.dtype == torch.bfloat16 else t.numpy().tobytes()
        header[name] = {"dtype": _TORCH_TAG[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        blobs.append(raw)
        offset += len(raw)
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * ((-(8 + len(text))) % 64)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for b in blobs:
            f.write(b)
