"""Shared pieces of the tests: the tiny configurations, model folders with random weights, comparisons."""
from __future__ import annotations

import json
import os
from typing import Dict, List

import torch

# Two tiny configurations that differ in every size and option: layers, width, heads, KV heads (one shared head
# against no grouping), head size, feed-forward width, vocabulary (none a power of two in B), eps, theta,
# scaling (none against llama3 with all three branches hit), tied against untied head.
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 64, "intermediate_size": 160, "vocab_size": 512, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 1, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
    "max_position_embeddings": 128, "tie_word_embeddings": True, "eos_token_id": 2,
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 96, "intermediate_size": 256, "vocab_size": 1000, "num_hidden_layers": 3,
    "num_attention_heads": 3, "num_key_value_heads": 3, "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
    "rope_scaling": {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64, "rope_type": "llama3"},
    "max_position_embeddings": 256, "tie_word_embeddings": False, "eos_token_id": [1, 7],
}
# a third shape: grouped heads (2 per KV head), head size 48 (a multiple of 16 that is no power of two)
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 192, "intermediate_size": 150, "vocab_size": 331, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
    "max_position_embeddings": 512, "tie_word_embeddings": True,
}
# the serving shape in small: heads of 64 in groups of four over two KV heads, sizes that take every fused bfloat16
# kernel (products with rotary and SiLU epilogues, K-split planes), llama3 scaling as Llama 3.2 has it, and room
# for contexts long enough that a decoded token's keys are split into chunks and merged
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 512, "intermediate_size": 1024, "vocab_size": 2003, "num_hidden_layers": 2,
    "num_attention_heads": 8, "num_key_value_heads": 2, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192, "rope_type": "llama3"},
    "max_position_embeddings": 2048, "tie_word_embeddings": True,
}
# heads of 128 in groups of three over one KV head (the larger Llamas' head size, where the bfloat16 attention has
# one wave per task only), an untied head, another eps and theta
TINY_E = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 384, "intermediate_size": 528, "vocab_size": 777, "num_hidden_layers": 2,
    "num_attention_heads": 3, "num_key_value_heads": 1, "rms_norm_eps": 3e-6, "rope_theta": 250000.0,
    "max_position_embeddings": 1024, "tie_word_embeddings": False,
}
# heads of 40 columns: a multiple of 8 that is no multiple of 16, which the reference's attention kernels take too
# (csrc/src/lib.rs:136-143, 790); here the general attention kernel runs them in both dtypes, while the bfloat16
# products with their rotary and SiLU epilogues still apply (widths that are multiples of 32)
TINY_F = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 160, "intermediate_size": 224, "vocab_size": 613, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "rms_norm_eps": 2e-5, "rope_theta": 10000.0,
    "rope_scaling": {"factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 128, "rope_type": "llama3"},
    "max_position_embeddings": 512, "tie_word_embeddings": True,
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F}
NORM_JITTER = {"A": 0.0, "B": 0.1, "C": 0.1, "D": 0.1, "E": 0.1, "F": 0.1}


def make_model_dir(path: str, cfg: dict, seed: int, dtype: str, norm_jitter: float = 0.0) -> str:
    from atoma_infer_amd.weights import write_random_model
    return write_random_model(path, cfg, seed=seed, dtype=dtype, norm_jitter=norm_jitter)


def plain_weights(model_dir: str) -> Dict[str, torch.Tensor]:
    """The checkpoint as float32 CPU tensors, read with the safetensors package (not with the framework's reader)."""
    from safetensors.torch import load_file
    return {k: v.to(torch.float32) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}


def plain_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest absolute difference relative to the largest wanted magnitude."""
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def frob_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).norm() / want.norm().clamp_min(1e-30))


# Tolerances, fixed before the first run.  float32: every value is a sum of at most a few thousand float32
# products whose order differs between the engine and the yardstick; 2e-5 of the largest logit covers that with
# room and is far below any real fault.  bfloat16: activations are rounded to 8 bits of mantissa (relative
# 2^-9) about eight times a layer; for at most 16 layers the errors add up to about 1e-2 of the logits' norm.
TOL_F32 = 2e-5
TOL_BF16 = 2e-2


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def check_greedy_tokens(prompt: List[int], tokens: List[int], chosen_logits: List[float], w, cfg, tol: float) -> None:
    """Greedy tokens of an engine whose logits carry rounding noise, against the plain model run on the sequence the
    engine produced: at every step the logit the engine reports for its token must be the plain one within ``tol``
    of the row's largest magnitude, and the token must be the plain argmax up to twice that (a flipped argmax
    between two nearly equal logits is rounding; a token from a wrong row of logits is not)."""
    import plain_llama
    rows = plain_llama.forward(list(prompt) + list(tokens), w, cfg)[len(prompt) - 1:-1]
    assert len(tokens) == len(chosen_logits) == rows.shape[0]
    for step, (tok, lg) in enumerate(zip(tokens, chosen_logits)):
        row = rows[step]
        scale = float(row.abs().max())
        assert abs(float(row[tok]) - lg) <= tol * scale, \
            f"step {step}: the engine's logit {lg:.5f} of token {tok} is not the plain model's {float(row[tok]):.5f}"
        assert float(row.max() - row[tok]) <= 2 * tol * scale, \
            f"step {step}: token {tok} is no argmax of the plain model ({float(row[tok]):.5f} < {float(row.max()):.5f})"


def force_chunked_decode(monkeypatch, second_kernel: bool = False):
    """Make the bfloat16 attention cut the keys of decoded tokens into chunks, as it does at long contexts with few
    requests; at the tiny contexts of tests its planner would let eight waves walk whole key ranges instead.  The
    chunks are merged by the wave that finishes the last one, as at contexts up to about 2,000 keys, or with
    ``second_kernel`` by the merging kernel, as beyond."""
    from atoma_infer_amd.kernels import attention_bf16
    monkeypatch.setattr(attention_bf16, "WHOLE_MIN_PAIRS", 10 ** 9)
    monkeypatch.setattr(attention_bf16, "WHOLE_SHORT_WALKS", ())
    monkeypatch.setattr(attention_bf16, "MERGE_WHOLE_MAX_KEYS", 0)
    if second_kernel:
        monkeypatch.setattr(attention_bf16, "MERGE_IN_KERNEL", False)
