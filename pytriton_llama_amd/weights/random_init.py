"""Random weights from a configuration and a seed.

The reference has no such mode (its only random tensor is a placeholder,
lite_llama/models/llama.py:23). Every tensor is drawn in float32 on the host
from a generator seeded by (seed, tensor name), so the values depend neither on
the order of creation nor on the device nor on the dtype they are stored in:
matrices ~ N(0, initializer_range), norm vectors 1 + N(0, norm_std), unless the part
that owns a tensor says otherwise (ParamSource.init).
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Any, Dict, Iterator, Tuple

import torch

from ..config.registry import architecture_of
from .loader import fill


def _generator(seed: int, name: str) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode())) % (2 ** 63 - 1))
    return g


def random_tensor(seed: int, name: str, shape, kind: str, std: float, norm_std: float,
                  vocab: int = 0, init=None) -> torch.Tensor:
    """``init``: the part's own wish for this tensor (ParamSource.init), which goes before the
    rule of its kind."""
    g = _generator(seed, name)
    if init is not None:
        how, *numbers = init
        if how == "normal" and len(numbers) == 2:
            t = numbers[0] + numbers[1] * torch.randn(shape, generator=g, dtype=torch.float32)
        elif how == "uniform" and len(numbers) == 2:
            t = numbers[0] + (numbers[1] - numbers[0]) * torch.rand(shape, generator=g, dtype=torch.float32)
        elif how == "constant" and len(numbers) == 1:
            t = torch.full(shape, float(numbers[0]), dtype=torch.float32)
        else:
            raise ValueError(f"tensor {name!r}: unknown init hint {init!r}; known: ('normal', mean, std), "
                             "('uniform', low, high), ('constant', value)")
        return t.round().to(torch.int32) if kind == "table" else t
    if kind == "vector":
        t = torch.ones(shape, dtype=torch.float32)
        if norm_std:
            t += norm_std * torch.randn(shape, generator=g, dtype=torch.float32)
        return t
    if kind == "table":
        return torch.randint(0, max(vocab, 1), shape, generator=g, dtype=torch.int32)
    return std * torch.randn(shape, generator=g, dtype=torch.float32)


def random_tensors(model, seed: int, norm_std: float = 0.0,
                   std: float = None) -> Iterator[Tuple[str, object, object, torch.Tensor]]:
    """(checkpoint name, part, source, float32 tensor) for every tensor of the model."""
    if std is None:
        std = float(getattr(model.config, "initializer_range", 0.02))
    for name, (part, src) in model.expected_tensors().items():
        yield name, part, src, random_tensor(seed, name, src.shape, src.kind, std, norm_std,
                                             init=getattr(src, "init", None))


def load_random_weights(model, seed: int, dtype: torch.dtype, device, norm_std: float = 0.0,
                        std: float = None) -> None:
    """Fill the model with the same values write_random_model would store,
    without a file. In bfloat16 they are the roundings of the float32 draws."""
    by_part: Dict[int, Tuple[object, Dict[str, torch.Tensor]]] = {}
    for name, part, src, t in random_tensors(model, seed, norm_std, std):
        by_part.setdefault(id(part), (part, {}))[1][src.name] = t
    fill(model, by_part, dtype, device)


def write_random_model(config: Dict[str, Any], folder: str, seed: int = 0,
                       dtype: torch.dtype = None, norm_std: float = 0.0,
                       std: float = None) -> str:
    """Write config.json and model.safetensors for ``config`` (a config.json
    dict) into ``folder``. ``dtype`` defaults to the config's torch_dtype."""
    from safetensors.torch import save_file

    arch = architecture_of(config)
    cfg = arch.config_class.from_dict(config)
    model = arch.build(cfg)
    if dtype is None:
        dtype = {"float32": torch.float32, "bfloat16": torch.bfloat16,
                 "float16": torch.float16}[str(config.get("torch_dtype", "bfloat16"))]
    os.makedirs(folder, exist_ok=True)
    tensors = {}
    for name, _, src, t in random_tensors(model, seed, norm_std, std):
        tensors[name] = t.to(torch.int32 if src.kind == "table" else dtype).contiguous()
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f, indent=1)
    return folder
