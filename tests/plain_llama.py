"""A plain, slow Llama decoder in float32 on the CPU: the yardstick of every engine test.

Whole sequences, no cache, no batching, one function for each part.  Nothing
here is imported from the framework: the formulas are written from the
reference's text, and each function cites the lines it follows.  Weights are a
``dict`` from the checkpoint's tensor names to float32 CPU tensors; the
configuration is the plain ``dict`` of config.json.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def head_size(cfg: dict) -> int:
    """models/src/llama.rs:326 -- the head size is hidden_size / num_attention_heads, nothing else."""
    return cfg["hidden_size"] // cfg["num_attention_heads"]


def kv_heads(cfg: dict) -> int:
    """models/src/llama.rs:55-57 -- num_key_value_heads defaults to the number of attention heads."""
    v = cfg.get("num_key_value_heads")
    return cfg["num_attention_heads"] if v is None else v


def rope_inv_freq(cfg: dict) -> torch.Tensor:
    """Inverse frequencies, float32.

    Default: models/src/llama.rs:146-152, ``1 / theta^(i/hd)`` for even i < hd, computed with f32 powf.
    llama3 scaling: models/src/llama.rs:163-186 (three branches on the wavelength 2*pi/f, PI as f32).
    ``rope_scaling`` absent or of type "default" leaves the frequencies unscaled (:157-162).
    """
    hd = head_size(cfg)
    theta = torch.tensor(float(cfg.get("rope_theta", 10000.0)), dtype=torch.float32)
    exps = torch.arange(0, hd, 2, dtype=torch.float32) / torch.tensor(float(hd), dtype=torch.float32)
    freqs = 1.0 / torch.pow(theta, exps)  # float32 throughout
    rs = cfg.get("rope_scaling")
    if rs is None or rs.get("rope_type", rs.get("type")) == "default":
        return freqs
    f32 = lambda v: torch.tensor(float(v), dtype=torch.float32)
    orig = f32(rs["original_max_position_embeddings"])
    low_wl = orig / f32(rs["low_freq_factor"])
    high_wl = orig / f32(rs["high_freq_factor"])
    pi = f32(math.pi)
    out = []
    for f in freqs:
        wl = f32(2.0) * pi / f
        if wl < high_wl:
            out.append(f)
        elif wl > low_wl:
            out.append(f / f32(rs["factor"]))
        else:
            smooth = (orig / wl - f32(rs["low_freq_factor"])) / (f32(rs["high_freq_factor"]) - f32(rs["low_freq_factor"]))
            out.append((f32(1.0) - smooth) * f / f32(rs["factor"]) + smooth * f)
    return torch.stack(out)


def rope_tables(cfg: dict, positions: torch.Tensor):
    """cos and sin of position x inv_freq, [len(positions), hd/2], float32 (models/src/llama.rs:189-199).

    The reference builds the table for every position below max_position_embeddings and gathers rows by
    position (:241-248); building only the gathered rows gives the same numbers.  The reference rounds the table
    to the model's dtype (:197-198); the yardstick keeps float32.
    """
    ang = positions.to(torch.float32)[:, None] * rope_inv_freq(cfg)[None, :]
    return torch.cos(ang), torch.sin(ang)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate ``x`` [tokens, heads, hd] by half-split pairs (i, i + hd/2).

    The reference calls candle's ``rope`` (models/src/llama.rs:250); the pairing and signs it means are spelled out
    in csrc/kernels/rotary.h:116-131: the left half gets ``x1*cos - x2*sin``, the right half ``x2*cos + x1*sin``,
    with the same cos/sin column for both members of a pair.
    """
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x * rsqrt(mean(x^2) + eps) * w`` over the last axis.

    The reference calls candle's RmsNorm with (hidden_size, rms_norm_eps, weight) (models/src/llama.rs:416-421, 487);
    its text fixes where the norm sits and where eps comes from, the formula is the standard one.
    """
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def attention_scores_softmax_pv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                                causal: bool, window: Optional[int] = None) -> torch.Tensor:
    """softmax(scale * q k^T + mask) v for one head group layout: q [nh, Tq, hd], k and v [nh, Tk, hd].

    Unmasked it is the reference's own oracle ``fa_acausal`` (csrc/tests/flash_attn_tests.rs:19-29).  The causal mask is
    aligned to the bottom right: query row i of Tq sees key j iff ``j <= i + (Tk - Tq)``
    (csrc/kernels/mask.h:171-172, 187-192).  ``window`` w keeps only the last w keys up to and including the
    query's own position (csrc/kernels/mask.h:171-176 with window_size_left = w - 1).
    """
    tq, tk = q.shape[1], k.shape[1]
    att = torch.matmul(q, k.transpose(1, 2)) * scale
    if causal or window is not None:
        i = torch.arange(tq)[:, None] + (tk - tq)
        j = torch.arange(tk)[None, :]
        keep = torch.ones(tq, tk, dtype=torch.bool)
        if causal:
            keep &= j <= i
        if window is not None:
            keep &= j > i - window
        att = att.masked_fill(~keep[None], float("-inf"))
    att = torch.softmax(att, dim=-1)
    return torch.matmul(att, v)


def self_attention(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, cfg: dict,
                   positions: torch.Tensor, window: Optional[int] = None) -> torch.Tensor:
    """One attention layer over a whole sequence ``x`` [T, H] (models/src/llama.rs:253-314).

    q/k/v projections without bias (:269-271, 322-324), split into heads of hd columns (:273-296), rotation of q
    and k only (:298-299), query head h reads KV head ``h // (nh/nkv)`` (csrc/kernels/flash_fwd_kernel.h:593),
    scale ``1/sqrt(hd)`` (:342), causal softmax, output projection (:311).
    """
    nh, nkv, hd = cfg["num_attention_heads"], kv_heads(cfg), head_size(cfg)
    t = x.shape[0]
    q = (x @ w[prefix + "q_proj.weight"].T).view(t, nh, hd)
    k = (x @ w[prefix + "k_proj.weight"].T).view(t, nkv, hd)
    v = (x @ w[prefix + "v_proj.weight"].T).view(t, nkv, hd)
    cos, sin = rope_tables(cfg, positions)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    group = nh // nkv
    k = k.repeat_interleave(group, dim=1)
    v = v.repeat_interleave(group, dim=1)
    o = attention_scores_softmax_pv(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                    1.0 / math.sqrt(hd), causal=True, window=window)
    o = o.transpose(0, 1).reshape(t, nh * hd)
    return o @ w[prefix + "o_proj.weight"].T


def swiglu_mlp(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """``down(silu(gate(x)) * up(x))``, no biases (models/src/llama.rs:362-366, 372-374)."""
    g = x @ w[prefix + "gate_proj.weight"].T
    u = x @ w[prefix + "up_proj.weight"].T
    return ((g * torch.sigmoid(g)) * u) @ w[prefix + "down_proj.weight"].T


def block(x: torch.Tensor, w: Dict[str, torch.Tensor], i: int, cfg: dict, positions: torch.Tensor) -> torch.Tensor:
    """Pre-norm block with two residual sums (models/src/llama.rs:393-410).  A ``sliding_window`` in ``cfg`` (the
    reference's models report one through ``sliding_window()``, backends/vllm/src/model_executor.rs:116-140, and
    hand it to the attention kernel as its left window) limits every layer's attention to that many keys."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    h = x + self_attention(rms_norm(x, w[p + "input_layernorm.weight"], eps), w, p + "self_attn.", cfg, positions,
                           window=cfg.get("sliding_window"))
    return h + swiglu_mlp(rms_norm(h, w[p + "post_attention_layernorm.weight"], eps), w, p + "mlp.")


def forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict, start: int = 0) -> torch.Tensor:
    """Logits [T, V] (float32) at every position of one whole sequence (models/src/llama.rs:456-478).

    Embedding gather (:470), the blocks in order (:471-473), the final norm on every row (:474), the output head:
    the embedding matrix when ``tie_word_embeddings`` else ``lm_head.weight`` (:482-486), no bias.  ``start`` shifts
    all positions (used only by the test that relative distances alone matter).
    """
    ids = torch.tensor(tokens, dtype=torch.long)
    positions = torch.arange(start, start + len(tokens))
    x = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        x = block(x, w, i, cfg, positions)
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x @ head.T


def greedy_generate(prompt: List[int], n: int, w: Dict[str, torch.Tensor], cfg: dict) -> List[int]:
    """Greedy continuation by re-running the whole sequence for every new token (argmax, lowest index on ties)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(toks, w, cfg)[-1])))
    return toks[len(prompt):]


# ---------------------------------------------------------------------------------------------------------
# sampling


def repeat_penalty(logits: torch.Tensor, penalty: float, context: List[int]) -> torch.Tensor:
    """Divide positive, multiply negative logits of tokens in ``context`` by ``penalty``, each token once.

    The reference applies candle's ``apply_repeat_penalty`` to the last ``repeat_last_n`` tokens
    (backends/vllm/src/model_executor.rs:211-225).
    """
    out = logits.clone()
    for t in set(context):
        out[t] = out[t] / penalty if out[t] >= 0 else out[t] * penalty
    return out


def sampling_distribution(logits: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 1.0,
                          ) -> torch.Tensor:
    """Probabilities the sampler draws from.

    softmax(logits / T) (mode ``All``), then keep the k most probable (``TopK``), then the smallest set of most
    probable tokens whose mass reaches p (``TopP``); both in that order for ``TopKThenTopP``
    (backends/vllm/src/llm_service.rs:349-372).  The kept probabilities are used unnormalised as weights.
    Ties are broken towards the lower token id.
    """
    p = torch.softmax(logits.to(torch.float32) / temperature, dim=-1)
    order = sorted(range(p.numel()), key=lambda i: (-float(p[i]), i))
    keep = order
    if top_k and top_k < len(keep):
        keep = keep[:top_k]
    if top_p < 1.0:
        acc, cut = 0.0, len(keep)
        for n, i in enumerate(keep):
            acc += float(p[i])
            if acc >= top_p:
                cut = n + 1
                break
        keep = keep[:cut]
    out = torch.zeros_like(p)
    idx = torch.tensor(keep, dtype=torch.long)
    out[idx] = p[idx]
    return out


def draw(weights: torch.Tensor, u: float) -> int:
    """Inverse-CDF draw in token order: the first index whose running sum exceeds ``u`` x total."""
    c = torch.cumsum(weights.to(torch.float64), 0)
    target = u * float(c[-1])
    idx = int(torch.searchsorted(c, torch.tensor(target, dtype=torch.float64), right=True))
    return min(idx, weights.numel() - 1)
