"""A model at run time: the parts of a ModelSpec with their weights on the device, and its forward pass.

The forward pass runs only the tokens of one step, as one batch: embedding gather, the layer calls in run order
(each with its own view of the cache), the final norm on the rows whose logits are wanted, and the head
(models/src/llama.rs:456-478 of the reference, which norms every row and selects afterwards).
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from ..config.base import ModelConfig
from ..config.registry import Architecture, load_model_config
from ..parts.base import Begun
from ..parts.linear import Normed
from ..weights.loader import load_into, load_random_into
from .spec import ModelSpec

_ACT = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclasses.dataclass
class Model:
    arch: Architecture
    config: ModelConfig
    spec: ModelSpec
    device: torch.device
    act_dtype: torch.dtype

    @property
    def vocab_size(self) -> int:
        return self.spec.vocab_size

    def weight_bytes(self) -> int:
        """Bytes of weights that one step reads (each matrix once; the embedding table only through a tied head)."""
        return sum(part.device_bytes() for _, part in self.spec.parts())

    def forward(self, ctx) -> Optional[torch.Tensor]:
        """Logits [wanted rows, vocab] in float32, or None when the step wants none."""
        spec = self.spec
        blocks = [spec.layers[call.layer][1] for call in spec.run_order]
        # the norm that reads each block's output: a block that can lets its last product begin that norm
        readers = [b.entry_norm() for b in blocks[1:]]
        readers.append(spec.final_norm[1] if getattr(ctx, "wants_all_rows", False) else None)
        first = blocks[0].entry_norm() if blocks else None
        resid, pending = spec.embedding[1].forward(ctx.tokens, first) if first is not None else \
            (spec.embedding[1].forward(ctx.tokens), None)
        for pos, block in enumerate(blocks):
            if block.fuses_next_norm:
                pending = block.forward(resid, pending, ctx, ctx.layer_cache(pos), next_norm=readers[pos])
            else:
                pending = block.forward(resid, pending, ctx, ctx.layer_cache(pos))
        if ctx.n_want == 0:
            return None
        if isinstance(pending, Begun):      # the final norm, begun by the last product, on every row
            return spec.head[1].forward(pending)
        if isinstance(pending, Normed):     # ... or finished behind it
            return spec.head[1].forward(pending.data)
        x = spec.final_norm[1].add_norm(resid, pending, rows=ctx.want_rows)
        return spec.head[1].forward(x)


def load_model(model_dir: str, dtype: str = "bfloat16", device: str = "cuda:0",
               sliding_window: Optional[int] = None) -> Model:
    """Build the model that ``model_dir/config.json`` names and bind ``model_dir``'s weights to it.

    ``dtype`` is the activation and cache dtype: "bfloat16" runs the serving kernels, "float32" everything in
    true 32-bit arithmetic.  Weights stay as stored (bfloat16 or float32) in both.  ``sliding_window`` overrides
    what config.json says of it (the engine's ``[cache]`` option).
    """
    if dtype not in _ACT:
        raise ValueError(f"dtype must be bfloat16 or float32, got {dtype!r}")
    dev = torch.device(device)
    if dev.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("this engine runs on a GPU only (device 'cuda:N'); no GPU is visible")
    arch, cfg = load_model_config(model_dir)
    if sliding_window is not None:
        if not any(f.name == "sliding_window" for f in dataclasses.fields(cfg)):
            raise ValueError(f"the configuration of {arch.name} has no sliding_window to set")
        cfg = dataclasses.replace(cfg, sliding_window=int(sliding_window))
    spec = arch.build(cfg)
    load_into(spec, model_dir, dev, _ACT[dtype])
    return Model(arch, cfg, spec, dev, _ACT[dtype])


def random_model(config, seed: int = 0, dtype: str = "bfloat16", stored: str = "bfloat16", device: str = "cuda:0",
                 norm_jitter: float = 0.0) -> Model:
    """A model with the weights that the random-weights mode would write for (config, seed), built without files.

    ``config`` is a typed configuration or the JSON object of a config.json.
    """
    from ..config.registry import resolve_architecture
    obj = config.to_dict() if isinstance(config, ModelConfig) else dict(config)
    arch = resolve_architecture(obj)
    cfg = arch.config_cls.from_dict(obj)
    dev = torch.device(device)
    if dev.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("this engine runs on a GPU only (device 'cuda:N'); no GPU is visible")
    spec = arch.build(cfg)
    load_random_into(spec, seed, _ACT[stored], dev, _ACT[dtype], norm_jitter)
    return Model(arch, cfg, spec, dev, _ACT[dtype])
