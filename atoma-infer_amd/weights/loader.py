"""Binding checkpoint tensors to a model's parts by name.

A checkpoint is ``model.safetensors`` or, for sharded ones, the files that
``model.safetensors.index.json`` lists under ``weight_map`` (the reference
merges shards by name the same way: backends/vllm/src/models/mod.rs:9-37).
Names are the checkpoint's own; nothing is renamed.  All faults of a
checkpoint against what the model expects are reported in one ``WeightsError``.
"""
from __future__ import annotations

import json
import os
import re
from typing import Dict, List, Tuple

import torch

from ..parts.base import WeightSpec
from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightsError(ValueError):
    """Lists tensors that are missing, unexpected, of a wrong shape or of a wrong kind."""

    def __init__(self, where: str, missing=(), unexpected=(), wrong_shape=(), wrong_kind=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_kind = list(wrong_kind)
        lines = [f"{where}: the checkpoint does not fit the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_kind:
            lines.append(f"  wrong kind ({len(self.wrong_kind)}): " + ", ".join(
                f"{n} is {got}, expected {want}" for n, got, want in self.wrong_kind))
        super().__init__("\n".join(lines))


class Checkpoint:
    """Tensor names of a model folder and lazy access to them."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        index = os.path.join(model_dir, "model.safetensors.index.json")
        single = os.path.join(model_dir, "model.safetensors")
        files: List[str] = []
        if os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as f:
                try:
                    wm = json.load(f)["weight_map"]
                except (json.JSONDecodeError, KeyError, TypeError) as e:
                    raise WeightsError(f"{index}: not a shard index ({e})") from None
            files = sorted({os.path.join(model_dir, v) for v in wm.values()})
        elif os.path.isfile(single):
            files = [single]
        else:
            raise WeightsError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json found")
        self._files: List[SafetensorsFile] = []
        self._where: Dict[str, SafetensorsFile] = {}
        for p in files:
            try:
                sf = SafetensorsFile(p)
            except SafetensorsError as e:
                raise WeightsError(str(e)) from None
            self._files.append(sf)
            for n in sf.names():
                self._where[n] = sf

    def names(self) -> List[str]:
        return list(self._where)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._where[name].shape(name)

    def dtype(self, name: str) -> torch.dtype:
        return self._where[name].dtype(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._where[name].tensor(name)

    def close(self):
        for f in self._files:
            f.close()


def expected_tensors(spec) -> Dict[str, WeightSpec]:
    """Full checkpoint name -> WeightSpec for every part of a ModelSpec."""
    out: Dict[str, WeightSpec] = {}
    for prefix, part in spec.parts():
        for rel, ws in part.weight_specs().items():
            name = f"{prefix}.{rel}" if prefix else rel
            if name in out:
                raise ValueError(f"two parts bind the tensor '{name}'")
            out[name] = ws
    return out


def check_checkpoint(spec, ckpt: Checkpoint) -> None:
    want = expected_tensors(spec)
    have = set(ckpt.names())
    ignorable = [re.compile(p) for p in spec.ignorable]
    missing = [n for n in want if n not in have]
    unexpected = sorted(n for n in have if n not in want and not any(r.fullmatch(n) for r in ignorable))
    wrong_shape, wrong_kind = [], []
    for n, ws in want.items():
        if n not in have:
            continue
        if tuple(ckpt.shape(n)) != tuple(ws.shape):
            wrong_shape.append((n, tuple(ckpt.shape(n)), tuple(ws.shape)))
        is_float = ckpt.dtype(n).is_floating_point
        if ws.is_int and is_float:
            wrong_kind.append((n, str(ckpt.dtype(n)), "an integer table"))
        elif not ws.is_int and not is_float:
            wrong_kind.append((n, str(ckpt.dtype(n)), "floating point"))
    if missing or unexpected or wrong_shape or wrong_kind:
        raise WeightsError(ckpt.model_dir, missing, unexpected, wrong_shape, wrong_kind)


def device_dtype_of(stored: torch.dtype) -> torch.dtype:
    """The dtype a stored tensor is kept in on the device.

    bfloat16 stays bfloat16, a tensor stored in 32 bits stays so; float16 and float64 are widened or narrowed to
    float32 (float16 -> float32 is exact); integer tables become int32.
    """
    if stored is torch.bfloat16:
        return torch.bfloat16
    if stored.is_floating_point:
        return torch.float32
    return torch.int32


def load_into(spec, model_dir: str, device: torch.device, act_dtype: torch.dtype) -> None:
    """Check the checkpoint of ``model_dir`` against ``spec`` and let every part take its tensors."""
    ckpt = Checkpoint(model_dir)
    try:
        check_checkpoint(spec, ckpt)
        for prefix, part in spec.parts():
            def get(rel: str, _p=prefix) -> torch.Tensor:
                name = f"{_p}.{rel}" if _p else rel
                t = ckpt.tensor(name)
                return t.to(device_dtype_of(t.dtype)) if t.dtype is not device_dtype_of(t.dtype) else t
            part.load(get, device, act_dtype)
    finally:
        ckpt.close()


def load_random_into(spec, seed: int, stored: torch.dtype, device: torch.device, act_dtype: torch.dtype,
                     norm_jitter: float = 0.0) -> None:
    """Give every part the tensors that ``write_random_model`` would have stored, without a file."""
    from .random_init import random_tensor
    want = expected_tensors(spec)
    for prefix, part in spec.parts():
        def get(rel: str, _p=prefix) -> torch.Tensor:
            name = f"{_p}.{rel}" if _p else rel
            return random_tensor(name, want[name], seed, stored, norm_jitter)
        part.load(get, device, act_dtype)
