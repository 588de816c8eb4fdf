"""Reading and writing safetensors files without loading them whole.

Format as the reference parses it (reference: src/SharpInference.Core/SafetensorsLoader.cs:190-231):
an unsigned 64-bit little-endian header length, a JSON header mapping each tensor name to
``dtype``, ``shape`` and ``data_offsets`` (relative to the end of the header), with an optional
``__metadata__`` entry, then the raw little-endian data.  Sharded folders carry
``model.safetensors.index.json`` with a ``weight_map`` (SafetensorsLoader.cs:49-101).
"""
from __future__ import annotations

import glob
import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "F64": (torch.float64, 8),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    file: str
    begin: int   # absolute byte offset in the file
    nbytes: int


def read_header(path: str) -> Dict[str, TensorEntry]:
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header")
        (n,) = struct.unpack("<Q", head)
        if n <= 0 or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file ({size} bytes)")
        try:
            meta = json.loads(f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
    out: Dict[str, TensorEntry] = {}
    base = 8 + n
    for name, info in meta.items():
        if name == "__metadata__":
            continue
        try:
            dtype, width = _DTYPES[info["dtype"]]
        except KeyError:
            raise SafetensorsError(f"{path}: tensor {name} has unsupported dtype {info.get('dtype')!r}") from None
        shape = tuple(int(s) for s in info["shape"])
        b, e = (int(x) for x in info["data_offsets"])
        count = 1
        for s in shape:
            count *= s
        if e - b != count * width:
            raise SafetensorsError(f"{path}: tensor {name}: {e - b} bytes for shape {shape} of {info['dtype']}")
        if base + e > size:
            raise SafetensorsError(f"{path}: tensor {name} reaches beyond the end of the file")
        out[name] = TensorEntry(name, dtype, shape, path, base + b, e - b)
    return out


def index_folder(model_dir: str) -> Dict[str, TensorEntry]:
    """Every tensor of a model folder: through the shard index if there is one, else
    ``model.safetensors``, else every ``model*.safetensors``."""
    idx = os.path.join(model_dir, "model.safetensors.index.json")
    files: List[str]
    if os.path.isfile(idx):
        with open(idx) as f:
            wm = json.load(f).get("weight_map", {})
        files = sorted({os.path.join(model_dir, v) for v in wm.values()})
        missing = [p for p in files if not os.path.isfile(p)]
        if missing:
            raise SafetensorsError("shard file(s) named by the index are missing: " + ", ".join(missing))
    else:
        one = os.path.join(model_dir, "model.safetensors")
        files = [one] if os.path.isfile(one) else sorted(glob.glob(os.path.join(model_dir, "model*.safetensors")))
    if not files:
        raise SafetensorsError(f"no model.safetensors in {model_dir}")
    out: Dict[str, TensorEntry] = {}
    for p in files:
        out.update(read_header(p))
    return out


def read_tensor(entry: TensorEntry) -> torch.Tensor:
    """One tensor, read from its file into host memory in its stored dtype."""
    raw = torch.empty(entry.nbytes, dtype=torch.uint8)
    if entry.nbytes:
        with open(entry.file, "rb") as f:
            f.seek(entry.begin)
            got = f.readinto(memoryview(raw.numpy()))
        if got != entry.nbytes:
            raise SafetensorsError(f"{entry.file}: short read of {entry.name}")
    return raw.view(entry.dtype).reshape(entry.shape)


def write_file(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata: Dict[str, str] = None) -> None:
    """Write tensors (host, contiguous) in the order given."""
    items = [(n, t.detach().cpu().contiguous()) for n, t in tensors]
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    for name, t in items:
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for _, t in items:
            if t.numel():
                f.write(memoryview(t.reshape(-1).view(torch.uint8).numpy()))
    os.replace(tmp, path)
