"""Reading and writing safetensors files by tensor name.

The format: 8 bytes little-endian header length, a JSON header mapping each
tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets
relative to the end of the header), then the raw little-endian data.  A folder
holds either one ``model.safetensors`` or shards named by
``model.safetensors.index.json`` (``weight_map``: name -> shard file), as the
reference's lazy reader expects too (yalis/model_loading.py:41-88).
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, Iterator, List, Tuple

import numpy as np
import torch

_DTYPES = {
    "F64": (torch.float64, 8),
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(RuntimeError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str  # safetensors dtype tag
    shape: Tuple[int, ...]
    file: str
    begin: int  # absolute byte offsets in the file
    end: int

    @property
    def torch_dtype(self) -> torch.dtype:
        return _DTYPES[self.dtype][0]


def _read_header(path: str) -> Tuple[Dict[str, dict], int]:
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: truncated file (no header length)")
        (n,) = struct.unpack("<Q", head)
        if n <= 0 or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} does not fit the file size {size}")
        try:
            header = json.loads(f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
    return header, 8 + n


def index_file(path: str) -> Dict[str, TensorEntry]:
    header, base = _read_header(path)
    size = os.path.getsize(path)
    out: Dict[str, TensorEntry] = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        dtype = meta.get("dtype")
        if dtype not in _DTYPES:
            raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dtype!r}")
        shape = tuple(int(s) for s in meta["shape"])
        begin, end = (int(x) for x in meta["data_offsets"])
        want = int(np.prod(shape, dtype=np.int64)) * _DTYPES[dtype][1] if shape else _DTYPES[dtype][1]
        if end - begin != want:
            raise SafetensorsError(
                f"{path}: tensor {name!r} of shape {shape} and dtype {dtype} spans {end - begin} bytes, expected {want}"
            )
        if base + end > size:
            raise SafetensorsError(f"{path}: tensor {name!r} reaches beyond the end of the file (truncated?)")
        out[name] = TensorEntry(name, dtype, shape, path, base + begin, base + end)
    return out


def index_folder(model_dir: str) -> Dict[str, TensorEntry]:
    """Name -> entry for every tensor of the folder's checkpoint."""
    idx = os.path.join(model_dir, "model.safetensors.index.json")
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(idx):
        with open(idx, "r", encoding="utf-8") as f:
            weight_map = json.load(f).get("weight_map", {})
        if not weight_map:
            raise SafetensorsError(f"{idx}: empty weight_map")
        out: Dict[str, TensorEntry] = {}
        per_file: Dict[str, Dict[str, TensorEntry]] = {}
        for name, shard in weight_map.items():
            if shard not in per_file:
                spath = os.path.join(model_dir, shard)
                if not os.path.isfile(spath):
                    raise FileNotFoundError(f"{idx} names shard {shard!r}, which is missing")
                per_file[shard] = index_file(spath)
            if name not in per_file[shard]:
                raise SafetensorsError(f"{idx}: tensor {name!r} is not in shard {shard!r}")
            out[name] = per_file[shard][name]
        return out
    if os.path.isfile(single):
        return index_file(single)
    raise FileNotFoundError(f"no model.safetensors (or model.safetensors.index.json) in {model_dir!r}")


def read_tensor(entry: TensorEntry) -> torch.Tensor:
    """The tensor as stored (CPU, storage dtype)."""
    nbytes = entry.end - entry.begin
    buf = np.fromfile(entry.file, dtype=np.uint8, count=nbytes, offset=entry.begin)
    if buf.size != nbytes:
        raise SafetensorsError(f"{entry.file}: short read for tensor {entry.name!r}")
    t = torch.from_numpy(buf).view(entry.torch_dtype)
    return t.reshape(entry.shape)


def write_file(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], shapes: Dict[str, Tuple[torch.dtype, Tuple[int, ...]]]) -> None:
    """Stream tensors into one safetensors file.  ``shapes`` gives every tensor's
    dtype and shape up front (the header precedes the data); ``tensors`` yields
    them in the same order, one at a time, so that a large model never sits in
    memory whole."""
    header: Dict[str, dict] = {}
    off = 0
    order: List[str] = []
    for name, (dtype, shape) in shapes.items():
        if dtype not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {dtype} (tensor {name!r})")
        n = int(np.prod(shape, dtype=np.int64)) * _DTYPES[_NAMES[dtype]][1]
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [off, off + n]}
        off += n
        order.append(name)
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        it: Iterator[Tuple[str, torch.Tensor]] = iter(tensors)
        for want in order:
            name, t = next(it)
            if name != want:
                raise SafetensorsError(f"tensor order mismatch: expected {want!r}, got {name!r}")
            dtype, shape = shapes[name]
            if t.dtype != dtype or tuple(t.shape) != tuple(shape):
                raise SafetensorsError(
                    f"tensor {name!r}: declared {dtype} {tuple(shape)}, got {t.dtype} {tuple(t.shape)}"
                )
            t = t.detach().contiguous().cpu()
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)


def write_dict(path: str, tensors: Dict[str, torch.Tensor]) -> None:
    shapes = {k: (v.dtype, tuple(v.shape)) for k, v in tensors.items()}
    write_file(path, tensors.items(), shapes)
