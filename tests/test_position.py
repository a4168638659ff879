"""The rotary frequencies of the product against the plain implementation's, on the CPU (the tables are built on the
host): the two tiny configurations, Llama 3.2's constants, and frequencies placed at the edges of the llama3 band."""
import math

import pytest
import torch

import plain_llama as P
from util import TINY_A, TINY_B, TINY_D

from atoma_infer_amd.parts.position import rotary_inv_freq


def _product(cfg):
    rs = cfg.get("rope_scaling")
    return rotary_inv_freq(P.head_size(cfg), cfg.get("rope_theta", 10000.0), rs)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_D])
def test_frequencies_equal_the_plain_ones(cfg):
    assert torch.equal(_product(cfg), P.rope_inv_freq(cfg))


def test_frequencies_at_the_edges_of_the_band():
    sc = dict(rope_type="llama3", original_max_position_embeddings=96, low_freq_factor=1.5, high_freq_factor=6.0,
              factor=5.0)
    for wl in (16 * (1 - 5e-4), 16 * (1 + 5e-4), 64 * (1 - 5e-4), 64 * (1 + 5e-4), 96 / 3.75, 96 / 2.625, 3.0, 900.0):
        cfg = {"hidden_size": 4, "num_attention_heads": 1, "rope_theta": (wl / (2 * math.pi)) ** 2, "rope_scaling": sc}
        got, want = _product(cfg), P.rope_inv_freq(cfg)
        assert torch.allclose(got, want, rtol=1e-6, atol=0), (wl, got, want)
