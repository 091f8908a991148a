"""Reading and writing safetensors files by tensor name.

File layout: 8 bytes little-endian header length n, n bytes of JSON
``{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}``,
then the raw little-endian tensor data.  The file is memory-mapped and tensors
are views into the map until they are converted or copied.

The reference reads GGUF in the same spirit: a table of tensor infos with
name, shape, type and offset (src/core/model/gguf/GGUFLoader.cpp:142-220),
checks of the header (:78-93) and of offsets against the running size
(:189-203).  Its container and its Q8_0 types are not used here.
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import torch


class WeightFileError(ValueError):
    """A weight file that cannot be parsed."""


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


def read_header(path: str) -> tuple[dict, int]:
    size = os.path.getsize(path)
    if size < 8:
        raise WeightFileError(f"{path}: file of {size} bytes is too short for a safetensors header")
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        if n <= 0 or 8 + n > size:
            raise WeightFileError(f"{path}: header length {n} does not fit the file of {size} bytes")
        raw = f.read(n)
    twice = []

    def pairs(items):
        # a name that stands twice in an object: json.loads would keep the last without a word
        seen = {}
        for k, v in items:
            if k in seen:
                twice.append(k)
            seen[k] = v
        return seen

    try:
        header = json.loads(raw.decode("utf-8"), object_pairs_hook=pairs)
    except (UnicodeDecodeError, ValueError) as e:
        raise WeightFileError(f"{path}: header is not JSON: {e}") from None
    if twice:
        raise WeightFileError(f"{path}: the header names {sorted(set(twice))} more than once")
    if not isinstance(header, dict):
        raise WeightFileError(f"{path}: header is not a JSON object")
    return header, 8 + n


def load_file(path: str) -> dict[str, torch.Tensor]:
    """All tensors of one file by name, in the type the file stores."""
    header, base = read_header(path)
    size = os.path.getsize(path)
    data_len = size - base
    with open(path, "rb") as f:
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)  # private pages: torch wants a writable buffer
    out = {}
    spans = []
    for name, info in header.items():
        if name == "__metadata__":
            continue
        try:
            dt, shape, (b, e) = info["dtype"], info["shape"], info["data_offsets"]
        except (KeyError, TypeError, ValueError):
            raise WeightFileError(f"{path}: entry '{name}' lacks dtype, shape or data_offsets") from None
        if dt not in _DTYPES:
            raise WeightFileError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
        tdt, isz = _DTYPES[dt]
        numel = 1
        for s in shape:
            if not isinstance(s, int) or s < 0:
                raise WeightFileError(f"{path}: tensor '{name}' has a bad shape {shape}")
            numel *= s
        if not (0 <= b <= e <= data_len) or e - b != numel * isz:
            raise WeightFileError(
                f"{path}: tensor '{name}' of shape {shape} and dtype {dt} needs {numel * isz} bytes, "
                f"its offsets [{b}, {e}) give {e - b} of the {data_len} data bytes (truncated file?)")
        spans.append((b, e, name))
        if numel == 0:
            out[name] = torch.empty(shape, dtype=tdt)
        else:
            out[name] = torch.frombuffer(mm, dtype=tdt, count=numel, offset=base + b).reshape(shape)
    spans.sort()
    for (b0, e0, n0), (b1, e1, n1) in zip(spans, spans[1:]):
        if b1 < e0:
            raise WeightFileError(f"{path}: tensors '{n0}' and '{n1}' overlap in the file")
    return out


def load_model_dir(model_dir: str) -> dict[str, torch.Tensor]:
    """Tensors of ``model.safetensors``, or of the shards that
    ``model.safetensors.index.json`` lists."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(single):
        return load_file(single)
    if os.path.exists(index):
        with open(index) as f:
            wm = json.load(f).get("weight_map", {})
        out = {}
        for shard in sorted(set(wm.values())):
            part = load_file(os.path.join(model_dir, shard))
            for k, v in part.items():
                if k in out:
                    raise WeightFileError(f"{model_dir}: tensor '{k}' appears in more than one shard")
                out[k] = v
        return out
    raise WeightFileError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json found")


def save_file(tensors: dict[str, torch.Tensor], path: str, metadata: dict | None = None) -> None:
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise WeightFileError(f"cannot store tensor '{name}' of dtype {t.dtype}")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    tmp = path + f".tmp{os.getpid()}"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
