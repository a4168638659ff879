"""Random-weights mode: write a model folder from a configuration and a seed.

The reference has no such mode.  Linears and embeddings are drawn from N(0, 0.02); norm weights are 1, or
1 + N(0, norm_jitter).  Every tensor has a generator of its own, keyed by (seed, tensor name), so a tensor's
values do not depend on which other tensors the model has or on the order of writing.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Iterator, Tuple, Union

import torch

from ..config.base import ModelConfig
from ..config.registry import resolve_architecture
from ..parts.base import WeightSpec
from .loader import expected_tensors
from .safetensors_io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _generator(seed: int, name: str) -> torch.Generator:
    h = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def random_tensor(name: str, ws: WeightSpec, seed: int, dtype: torch.dtype, norm_jitter: float = 0.0,
                  ) -> torch.Tensor:
    g = _generator(seed, name)
    if ws.init in ("linear", "embedding"):
        t = torch.randn(ws.shape, generator=g, dtype=torch.float32) * 0.02
    elif ws.init == "norm":
        t = torch.ones(ws.shape, dtype=torch.float32)
        if norm_jitter:
            t += torch.randn(ws.shape, generator=g, dtype=torch.float32) * norm_jitter
    elif ws.init == "int_table":
        return torch.randint(0, max(ws.high, 1), ws.shape, generator=g, dtype=torch.int32)
    else:
        raise ValueError(f"tensor '{name}': unknown init '{ws.init}'")
    return t.to(dtype)


def random_tensors(spec, seed: int, dtype: torch.dtype, norm_jitter: float = 0.0,
                   ) -> Iterator[Tuple[str, torch.Tensor]]:
    for name, ws in expected_tensors(spec).items():
        yield name, random_tensor(name, ws, seed, dtype, norm_jitter)


def write_random_model(model_dir: str, config: Union[ModelConfig, Dict[str, Any]], seed: int = 0,
                       dtype: str = "bfloat16", norm_jitter: float = 0.0) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` into ``model_dir`` and return the folder.

    ``config`` is a typed configuration or the JSON object of a config.json (its ``architectures`` picks the
    model, as everywhere).  ``dtype`` is how the tensors are stored: "bfloat16" or "float32".
    """
    if dtype not in _STORE:
        raise ValueError(f"dtype must be one of {sorted(_STORE)}")
    if isinstance(config, ModelConfig):
        obj = config.to_dict()
    else:
        obj = dict(config)
    arch = resolve_architecture(obj)
    cfg = arch.config_cls.from_dict(obj)
    spec = arch.build(cfg)
    os.makedirs(model_dir, exist_ok=True)
    obj.setdefault("torch_dtype", dtype)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(obj, f, indent=2)
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      random_tensors(spec, seed, _STORE[dtype], norm_jitter),
                      metadata={"format": "pt", "seed": seed})
    return model_dir
