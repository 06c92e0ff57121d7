"""Reads a model folder's safetensors files by tensor name and checks them against what the
model's parts declare.

The reference reads ``model.safetensors`` by exact tensor name too (``base/src/model.cu:15-84``)
but checks neither shape nor dtype and aborts on a missing name.  Here every problem found -
missing tensors, unexpected tensors, wrong shapes, unusable dtypes - is collected into ONE
:class:`WeightError`.

Dtypes.  A tensor stored in bfloat16 stays bfloat16 on a bfloat16 engine and is widened
(exactly) on a float32 engine.  A tensor stored in 32-bit float stays 32-bit on either engine.
A tensor stored in float16 is widened to 32-bit (exactly: bfloat16 would drop three of its
mantissa bits) and from then on is a tensor in 32-bit.  Integer tables become int32.
"""
from __future__ import annotations

import fnmatch
import json
import os
from typing import Dict, Iterable, List, Mapping, Tuple

import torch

from ..models.spec import TensorSpec

_FLOAT_TAGS = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16}
_INT_TAGS = {"I64", "I32", "I16", "I8", "U8"}


class WeightError(ValueError):
    """The checkpoint does not fit the model (one message lists everything that is wrong)."""


def _weight_files(model_dir: str) -> List[str]:
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            files = sorted(set(json.load(f).get("weight_map", {}).values()))
        return [os.path.join(model_dir, n) for n in files]
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    found = sorted(n for n in os.listdir(model_dir) if n.endswith(".safetensors")) \
        if os.path.isdir(model_dir) else []
    if not found:
        raise WeightError(f"no model.safetensors in model folder {model_dir!r}")
    return [os.path.join(model_dir, n) for n in found]


def _read_header(path: str) -> Dict[str, dict]:
    """The JSON header of a safetensors file: 8-byte little-endian length, then JSON."""
    if not os.path.isfile(path):
        raise WeightError(f"{path}: named by model.safetensors.index.json but not in the model folder")
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        raw = f.read(8)
        if len(raw) < 8:
            raise WeightError(f"{path}: truncated (no header length)")
        n = int.from_bytes(raw, "little")
        if n <= 0 or 8 + n > size:
            raise WeightError(f"{path}: header length {n} exceeds the file size {size}")
        try:
            header = json.loads(f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightError(f"{path}: header is not valid JSON ({e})") from None
    header.pop("__metadata__", None)
    payload = size - 8 - n
    for name, info in header.items():
        lo, hi = info.get("data_offsets", (0, 0))
        if not (0 <= lo <= hi <= payload):
            raise WeightError(f"{path}: tensor {name!r} lies outside the file (offsets {lo}..{hi}, "
                              f"payload {payload} bytes)")
    return header


def checkpoint_index(model_dir: str) -> Dict[str, Tuple[str, dict]]:
    """tensor name -> (file, header entry) over all weight files of the folder."""
    out: Dict[str, Tuple[str, dict]] = {}
    for path in _weight_files(model_dir):
        for name, info in _read_header(path).items():
            out[name] = (path, info)
    return out


def validate(index: Mapping[str, Tuple[str, dict]], specs: Mapping[str, TensorSpec],
             ignorable: Iterable[str] = (), where: str = "checkpoint") -> None:
    """Raises one WeightError naming every missing, unexpected, misshapen or mistyped tensor."""
    ignorable = tuple(ignorable)
    missing = sorted(n for n in specs if n not in index)
    unexpected = sorted(n for n in index if n not in specs
                        and not any(fnmatch.fnmatchcase(n, pat) for pat in ignorable))
    wrong_shape, wrong_dtype = [], []
    for name, spec in specs.items():
        if name not in index:
            continue
        info = index[name][1]
        shape = tuple(info.get("shape", ()))
        if shape != tuple(spec.shape):
            wrong_shape.append(f"{name}: stored {list(shape)}, the model needs {list(spec.shape)}")
        tag = info.get("dtype")
        ok = (tag in _INT_TAGS) if spec.role == "table" else (tag in _FLOAT_TAGS)
        if not ok:
            wrong_dtype.append(f"{name}: stored as {tag}")
    if not (missing or unexpected or wrong_shape or wrong_dtype):
        return
    lines = [f"{where} does not fit the model:"]
    for title, items in (("missing tensors", missing), ("unexpected tensors", unexpected),
                         ("wrong shapes", wrong_shape), ("unsupported dtypes", wrong_dtype)):
        if items:
            lines.append(f"  {title} ({len(items)}):")
            lines.extend(f"    {it}" for it in items)
    raise WeightError("\n".join(lines))


def target_dtype(stored: torch.dtype, role: str, engine_dtype: torch.dtype) -> torch.dtype:
    if role == "table":
        return torch.int32
    if stored in (torch.float32, torch.float16):
        return torch.float32            # a tensor stored in 32-bit stays so; float16 only fits into 32-bit exactly
    return engine_dtype                 # bf16 storage: the engine's dtype (widening to 32-bit is exact)


def load_tensors(model_dir: str, specs: Mapping[str, TensorSpec], engine_dtype: torch.dtype,
                 device, ignorable: Iterable[str] = ()) -> Dict[str, torch.Tensor]:
    """Validates the checkpoint against ``specs`` and returns the tensors on ``device``."""
    from safetensors import safe_open

    index = checkpoint_index(model_dir)
    validate(index, specs, ignorable, where=f"model folder {model_dir!r}")
    by_file: Dict[str, List[str]] = {}
    for name in specs:
        by_file.setdefault(index[name][0], []).append(name)
    out: Dict[str, torch.Tensor] = {}
    for path, names in by_file.items():
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in names:
                t = f.get_tensor(name)
                dt = target_dtype(t.dtype, specs[name].role, engine_dtype)
                out[name] = t.to(device=device, dtype=dt).contiguous()
    return out
