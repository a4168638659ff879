"""Arrangements of parts around the residual stream.

``PreNormBlock``: ``h = x + mixer(norm1(x))``, ``y = h + ffn(norm2(h))`` (models/src/llama.rs:393-410).  The residual
stream is float32; each sum is fused with the norm that follows it, so a block receives the previous block's
output as a pending ``delta`` and returns its own.
"""
from __future__ import annotations

from typing import Dict

from .base import Begun, Block, FeedForward, Mixer, Norm, WeightSpec, register_block
from .linear import Normed, ResidualSink


class PreNormBlock(Block):
    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm, feed_forward: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward
        self.names = tuple(names)

    def _children(self):
        return zip(self.names, (self.norm1, self.mixer, self.norm2, self.feed_forward))

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {f"{n}.{k}": ws for n, part in self._children() for k, ws in part.weight_specs().items()}

    def load(self, get, device, act_dtype) -> None:
        for n, part in self._children():
            part.load(lambda rel, _n=n: get(f"{_n}.{rel}"), device, act_dtype)

    def graph_safe(self) -> bool:
        return all(part.graph_safe() for _, part in self._children())

    def device_bytes(self) -> int:
        return sum(part.device_bytes() for _, part in self._children())

    fuses_next_norm = True

    def entry_norm(self):
        return self.norm1

    @staticmethod
    def _normed(norm, resid, pending, reader):
        """The input of ``reader``: ``pending`` is either a delta still to be added and normed, or ``norm`` already
        begun or finished by the product that made it (which has also added it to ``resid``)."""
        if isinstance(pending, Normed):
            if pending.norm is not norm:
                raise RuntimeError("a finished norm reached another norm than the one it was made for")
            return pending.data
        if isinstance(pending, Begun):
            if pending.norm is not norm:
                raise RuntimeError("a begun norm reached another norm than the one it was begun for")
            return pending if reader.accepts_begun else pending.tensor()
        return norm.add_norm(resid, pending)

    def forward(self, resid, delta, ctx, cache, next_norm=None):
        x = self._normed(self.norm1, resid, delta, self.mixer)
        if self.mixer.takes_sink:
            a = self.mixer.forward(x, ctx, cache, sink=ResidualSink(resid, self.norm2))
        else:
            a = self.mixer.forward(x, ctx, cache)
        x = self._normed(self.norm2, resid, a, self.feed_forward)
        if self.feed_forward.takes_sink and next_norm is not None:
            return self.feed_forward.forward(x, ctx, sink=ResidualSink(resid, next_norm))
        return self.feed_forward.forward(x, ctx)


register_block("pre_norm", PreNormBlock)
