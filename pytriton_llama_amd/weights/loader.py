"""Reading a model folder's safetensors by tensor name.

The reference converts an HF checkpoint to its own .pth first and loads that
with load_state_dict(strict=True) (lite_llama/executor/weight_convert.py:182-252,
lite_llama/executor/model_executor.py:92-127). Here the HF tensors are read
directly; what is wrong with a folder is reported in one error that lists every
missing tensor, every unexpected one and every wrong shape.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Tuple

import torch

INDEX_NAME = "model.safetensors.index.json"
SINGLE_NAME = "model.safetensors"

_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)
_INTS = (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8)


class WeightError(RuntimeError):
    """The tensors of a model folder do not fit the model."""

    def __init__(self, folder: str, missing=(), unexpected=(), wrong_shape=(), other=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.other = list(wrong_shape), list(other)
        lines = [f"weights in {folder!r} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the configuration wants {list(want)}")
        for msg in self.other:
            lines.append("  " + msg)
        super().__init__("\n".join(lines))


def _tensor_files(folder: str) -> Dict[str, str]:
    """tensor name -> file that holds it."""
    from safetensors import safe_open

    index = os.path.join(folder, INDEX_NAME)
    single = os.path.join(folder, SINGLE_NAME)
    out: Dict[str, str] = {}
    if os.path.isfile(index):
        with open(index) as f:
            weight_map = json.load(f)["weight_map"]
        missing_files = sorted({fn for fn in weight_map.values()
                                if not os.path.isfile(os.path.join(folder, fn))})
        if missing_files:
            raise WeightError(folder, other=[f"shard files named by the index are absent: {missing_files}"])
        for name, fn in weight_map.items():
            out[name] = os.path.join(folder, fn)
        return out
    if os.path.isfile(single):
        with safe_open(single, framework="pt") as f:
            for name in f.keys():
                out[name] = single
        return out
    raise WeightError(folder, other=[f"neither {SINGLE_NAME} nor {INDEX_NAME} is there"])


def load_weights(model, folder: str, dtype: torch.dtype, device) -> None:
    """Fill every part of ``model`` from the folder. Matrices are held in
    ``dtype``, vectors in float32, integer tables as int32."""
    from safetensors import safe_open

    files = _tensor_files(folder)
    if getattr(model, "before_load", None) is not None:
        model.before_load(set(files))
    expected = model.expected_tensors()
    missing = sorted(n for n in expected if n not in files)
    unexpected = sorted(n for n in files if n not in expected and not model.is_ignorable(n))
    handles = {}

    def handle(path):
        if path not in handles:
            handles[path] = safe_open(path, framework="pt")
        return handles[path]

    wrong: List[Tuple[str, tuple, tuple]] = []
    other: List[str] = []
    for name, (_, src) in expected.items():
        if name not in files:
            continue
        sl = handle(files[name]).get_slice(name)
        shape = tuple(sl.get_shape())
        if shape != tuple(src.shape):
            wrong.append((name, shape, tuple(src.shape)))
    if missing or unexpected or wrong or other:
        raise WeightError(folder, missing, unexpected, wrong, other)

    by_part: Dict[int, Tuple[object, Dict[str, torch.Tensor]]] = {}
    for name, (part, src) in expected.items():
        t = handle(files[name]).get_tensor(name)
        if src.kind == "table":
            if t.dtype not in _INTS:
                other.append(f"{name} should hold integers but is {t.dtype}")
        elif t.dtype not in _FLOATS:
            other.append(f"{name} should hold floats but is {t.dtype}")
        by_part.setdefault(id(part), (part, {}))[1][src.name] = t
    if other:
        raise WeightError(folder, other=other)
    fill(model, by_part, dtype, device)


def fill(model, by_part, dtype: torch.dtype, device) -> None:
    """Hand each part its tensors; parts without tensors still get load() so
    that they can put their constants on the device."""
    seen = set()
    for _, part in model.prefixes:
        if id(part) in seen:
            continue
        seen.add(id(part))
        tensors = by_part.get(id(part), (part, {}))[1]
        part.load(tensors, dtype, device)
    model.dtype, model.device = dtype, torch.device(device)
