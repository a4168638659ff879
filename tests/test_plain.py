"""What fixes the plain implementation beside the reference's text: the reference's own vectors, special cases
that reduce to a library routine, and invariants, each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch

import plain_llama as P
from util import TINY_A, TINY_B, random_tokens


def random_weights(cfg, seed=0, jitter=0.1):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd = cfg["num_attention_heads"], P.kv_heads(cfg), P.head_size(cfg)
    w = {"model.embed_tokens.weight": torch.randn(V, H, generator=g) * 0.02,
         "model.norm.weight": 1 + torch.randn(H, generator=g) * jitter}
    if not cfg.get("tie_word_embeddings"):
        w["lm_head.weight"] = torch.randn(V, H, generator=g) * 0.02
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        for n, shape in (("self_attn.q_proj", (nh * hd, H)), ("self_attn.k_proj", (nkv * hd, H)),
                         ("self_attn.v_proj", (nkv * hd, H)), ("self_attn.o_proj", (H, nh * hd)),
                         ("mlp.gate_proj", (I, H)), ("mlp.up_proj", (I, H)), ("mlp.down_proj", (H, I))):
            w[p + n + ".weight"] = torch.randn(*shape, generator=g) * 0.02
        w[p + "input_layernorm.weight"] = 1 + torch.randn(H, generator=g) * jitter
        w[p + "post_attention_layernorm.weight"] = 1 + torch.randn(H, generator=g) * jitter
    return w


def test_attention_equals_the_references_vectors():
    """csrc/tests/flash_attn_tests.rs:31-93 (no mask) and models/src/flash_attention.rs:632-705 (causal): q =
    arange(48)/30, k = /40, v = /50 in float16, 3 heads x 2 tokens x 8, scale 0.5, goldens to 4 places."""
    base = torch.arange(48, dtype=torch.float32).reshape(3, 2, 8).half()
    q, k, v = (base / 30).float(), (base / 40).float(), (base / 50).float()
    acausal = torch.tensor([
        [[0.0837, 0.1038, 0.1238, 0.1438, 0.1637, 0.1837, 0.2037, 0.2238],
         [0.0922, 0.1122, 0.1322, 0.1522, 0.1721, 0.1921, 0.2122, 0.2322]],
        [[0.4204, 0.4404, 0.4604, 0.4805, 0.5005, 0.5205, 0.5405, 0.5605],
         [0.428, 0.448, 0.468, 0.488, 0.5083, 0.5283, 0.5483, 0.5684]],
        [[0.7554, 0.7754, 0.7954, 0.8154, 0.8354, 0.8555, 0.8755, 0.8955],
         [0.7622, 0.7822, 0.8022, 0.8223, 0.8423, 0.8623, 0.8823, 0.9023]]])
    got = P.attention_scores_softmax_pv(q, k, v, 0.5, causal=False)
    assert (got - acausal).abs().max() < 1.5e-3          # the goldens carry float16 rounding
    causal = acausal.clone()
    causal[:, 0] = v[:, 0]                                # row 0 sees only key 0
    got = P.attention_scores_softmax_pv(q, k, v, 0.5, causal=True)
    assert (got - causal).abs().max() < 1.5e-3
    assert torch.allclose(got[:, 0], v[:, 0], atol=1e-6)


def test_attention_reduces_to_the_library_routine():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(2, 5, 16, generator=g) for _ in range(3))
    want = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    assert torch.allclose(P.attention_scores_softmax_pv(q, k, v, 1 / 4.0, causal=True), want, atol=1e-6)
    want = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None])[0]
    assert torch.allclose(P.attention_scores_softmax_pv(q, k, v, 1 / 4.0, causal=False), want, atol=1e-6)
    # bottom-right alignment: 2 query rows over 5 keys are the last two rows of the square case
    full = P.attention_scores_softmax_pv(q, k, v, 0.25, causal=True)
    assert torch.allclose(P.attention_scores_softmax_pv(q[:, 3:], k, v, 0.25, causal=True), full[:, 3:], atol=1e-6)
    # a window of w keeps the last w keys including the query's own
    win = P.attention_scores_softmax_pv(q, k, v, 0.25, causal=True, window=2)
    assert torch.allclose(win[:, 4], P.attention_scores_softmax_pv(q[:, 4:], k[:, 3:], v[:, 3:], 0.25, causal=True)[:, 0],
                          atol=1e-6)
    # rows of the softmax sum to one: constant values give constant output
    const = torch.full_like(v, 0.37)
    assert torch.allclose(P.attention_scores_softmax_pv(q, k, const, 0.25, causal=True), const, atol=1e-6)


def test_rope_pairing_signs_and_invariants():
    cfg = dict(TINY_A)
    hd = P.head_size(cfg)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 3, hd, generator=g)
    pos = torch.tensor([0, 1, 2, 10, 50, 127])
    cos, sin = P.rope_tables(cfg, pos)
    y = P.apply_rope(x, cos, sin)
    # position 0 is the identity; each pair (i, i + hd/2) keeps its norm
    assert torch.allclose(y[0], x[0], atol=1e-7)
    half = hd // 2
    assert torch.allclose(y[..., :half] ** 2 + y[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2, atol=1e-5)
    # equals the rotate-half routine with duplicated tables (a wrong sign or an interleaved pairing fails here)
    c2, s2 = torch.cat([cos, cos], -1)[:, None], torch.cat([sin, sin], -1)[:, None]
    rot = torch.cat([-x[..., half:], x[..., :half]], -1)
    assert torch.allclose(y, x * c2 + rot * s2, atol=1e-6)
    # a unit vector on axis 0 turns towards axis hd/2 by +angle
    e = torch.zeros(1, 1, hd)
    e[..., 0] = 1.0
    c1, s1 = P.rope_tables(cfg, torch.tensor([1]))
    r = P.apply_rope(e, c1, s1)
    assert math.isclose(float(r[0, 0, 0]), math.cos(1.0), abs_tol=1e-6)
    assert math.isclose(float(r[0, 0, half]), math.sin(1.0), abs_tol=1e-6)
    # scores depend only on distances
    q, k = torch.randn(1, 1, hd, generator=g), torch.randn(1, 1, hd, generator=g)
    def score(m, n):
        cm, sm = P.rope_tables(cfg, torch.tensor([m]))
        cn, sn = P.rope_tables(cfg, torch.tensor([n]))
        return float((P.apply_rope(q, cm, sm) * P.apply_rope(k, cn, sn)).sum())
    assert math.isclose(score(7, 3), score(57, 53), rel_tol=1e-4, abs_tol=1e-5)
    assert not math.isclose(score(7, 3), score(7, 4), rel_tol=1e-3)


def test_llama3_frequency_scaling_branches():
    """models/src/llama.rs:163-186.  Tiny B (theta 5e5, hd 32, original 64, low 1, high 4) hits all three
    branches: wavelengths below 16 stay, above 64 are divided by the factor, those between are blended."""
    inv = P.rope_inv_freq(TINY_B)
    base = P.rope_inv_freq({k: v for k, v in TINY_B.items() if k != "rope_scaling"})
    wl = 2 * math.pi / base
    lo, mid, hi = wl < 16, (wl >= 16) & (wl <= 64), wl > 64
    assert lo.any() and mid.any() and hi.any()
    assert torch.equal(inv[lo], base[lo])
    assert torch.allclose(inv[hi], base[hi] / 8)
    assert ((inv[mid] < base[mid]) & (inv[mid] > base[mid] / 8)).all()
    # factor 1 changes nothing; type "default" means unscaled (models/src/llama.rs:157-162)
    one = dict(TINY_B, rope_scaling=dict(TINY_B["rope_scaling"], factor=1.0))
    assert torch.allclose(P.rope_inv_freq(one), base, rtol=1e-6)
    dflt = dict(TINY_B, rope_scaling=dict(TINY_B["rope_scaling"], rope_type="default"))
    assert torch.equal(P.rope_inv_freq(dflt), base)
    # the default frequencies themselves
    assert torch.allclose(base, torch.tensor([500000.0 ** (-i / 32) for i in range(0, 32, 2)]), rtol=1e-5)


def _one_frequency_cfg(wavelen, **scaling):
    """A configuration whose second inverse frequency has the given wavelength: head size 4, so the frequencies are
    1 and theta^(-1/2), and theta = (wavelen / 2 pi)^2."""
    return {"hidden_size": 4, "num_attention_heads": 1, "rope_theta": (wavelen / (2 * math.pi)) ** 2,
            "rope_scaling": dict({"rope_type": "llama3"}, **scaling)}


def test_llama3_blend_by_hand_and_at_the_edges_of_its_band():
    """models/src/llama.rs:177-182: smooth = (orig / wavelen - low) / (high - low), and the blended frequency is
    (1 - smooth) * f / factor + smooth * f.  With orig 64, low 1, high 4, factor 8 a wavelength of 32 gives
    smooth = (2 - 1) / 3 = 1/3 and f * (2/3 / 8 + 1/3) = f * 5/12 (swapping smooth and 1 - smooth gives f * 17/24).
    The blend is continuous with its neighbours: towards wavelength orig / high it tends to f, towards orig / low
    to f / factor (:173-176); a frequency placed just inside either edge must lie within a fraction of a percent of
    the branch outside it, and a swapped blend is off by the factor there."""
    sc = dict(original_max_position_embeddings=64, low_freq_factor=1.0, high_freq_factor=4.0, factor=8.0)
    f = 2 * math.pi / 32
    inv = P.rope_inv_freq(_one_frequency_cfg(32.0, **sc))
    assert math.isclose(float(inv[0]), 1.0, rel_tol=1e-6)                  # wavelength 6.28 < 16: untouched
    assert math.isclose(float(inv[1]), f * 5 / 12, rel_tol=1e-5)
    assert math.isclose(float(inv[1]), 0.0818123, rel_tol=1e-5)
    # the two edges, from inside and from outside the band; other constants than above, none of them 1
    sc = dict(original_max_position_embeddings=96, low_freq_factor=1.5, high_freq_factor=6.0, factor=5.0)
    high_wl, low_wl = 96 / 6.0, 96 / 1.5
    for wl, want_ratio in ((high_wl * (1 - 5e-4), 1.0), (high_wl * (1 + 5e-4), 1.0),
                           (low_wl * (1 - 5e-4), 1 / 5.0), (low_wl * (1 + 5e-4), 1 / 5.0)):
        inv = P.rope_inv_freq(_one_frequency_cfg(wl, **sc))
        assert math.isclose(float(inv[1]) / (2 * math.pi / wl), want_ratio, rel_tol=5e-3), (wl, float(inv[1]))
    # and halfway in terms of orig / wavelen (here 3.75, smooth 1/2) the two branches weigh the same
    wl = 96 / 3.75
    inv = P.rope_inv_freq(_one_frequency_cfg(wl, **sc))
    assert math.isclose(float(inv[1]) / (2 * math.pi / wl), 0.5 * (1 + 1 / 5.0), rel_tol=1e-5)
    # a quarter of the way (orig / wavelen = 2.625, smooth 1/4): 3/4 of f / factor and 1/4 of f
    wl = 96 / 2.625
    inv = P.rope_inv_freq(_one_frequency_cfg(wl, **sc))
    assert math.isclose(float(inv[1]) / (2 * math.pi / wl), 0.75 / 5.0 + 0.25, rel_tol=1e-5)


def test_rms_norm_and_swiglu_reduce_to_library_routines():
    g = torch.Generator().manual_seed(2)
    x, w = torch.randn(4, 96, generator=g), torch.randn(96, generator=g)
    assert torch.allclose(P.rms_norm(x, w, 1e-6), torch.nn.functional.rms_norm(x, (96,), w, 1e-6), atol=1e-6)
    y = P.rms_norm(x, torch.ones(96), 1e-12)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(4), atol=1e-5)
    assert torch.allclose(P.rms_norm(3.0 * x, w, 1e-12), P.rms_norm(x, w, 1e-12), atol=1e-5)
    wts = {"gate_proj.weight": torch.randn(10, 96, generator=g), "up_proj.weight": torch.randn(10, 96, generator=g),
           "down_proj.weight": torch.randn(96, 10, generator=g)}
    want = (torch.nn.functional.silu(x @ wts["gate_proj.weight"].T) * (x @ wts["up_proj.weight"].T)) @ \
        wts["down_proj.weight"].T
    assert torch.allclose(P.swiglu_mlp(x, wts, ""), want, atol=1e-5)
    wts["gate_proj.weight"] = torch.zeros(10, 96)
    assert torch.count_nonzero(P.swiglu_mlp(x, wts, "")) == 0


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_whole_model_invariants(cfg):
    w = random_weights(cfg, seed=4)
    toks = random_tokens(24, cfg["vocab_size"], 5)
    full = P.forward(toks, w, cfg)
    assert full.shape == (24, cfg["vocab_size"])
    # causal: a prefix gives the same logits at its positions
    assert torch.allclose(P.forward(toks[:9], w, cfg), full[:9], atol=1e-5)
    # only distances count: shifting all positions changes nothing (fails if rope used absolute positions wrongly)
    assert torch.allclose(P.forward(toks, w, cfg, start=17), full, atol=2e-5)
    # the head: tied uses the embedding matrix, untied its own
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    w2 = dict(w)
    key = "model.embed_tokens.weight" if cfg.get("tie_word_embeddings") else "lm_head.weight"
    w2[key] = head * 2
    if not cfg.get("tie_word_embeddings"):
        assert torch.allclose(P.forward(toks, w2, cfg), 2 * full, atol=1e-5)
    # the norm sits before the mixer: scaling one layer's input norm weight scales nothing linearly
    # (a post-norm arrangement would); and zeroing o_proj and down_proj of every layer leaves embed -> norm -> head
    w3 = dict(w)
    for i in range(cfg["num_hidden_layers"]):
        w3[f"model.layers.{i}.self_attn.o_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.self_attn.o_proj.weight"])
        w3[f"model.layers.{i}.mlp.down_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.mlp.down_proj.weight"])
    x = w["model.embed_tokens.weight"][torch.tensor(toks)]
    want = P.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]) @ head.T
    assert torch.allclose(P.forward(toks, w3, cfg), want, atol=1e-6)


def test_one_token_block_in_closed_form():
    """A sequence of one token: the softmax over one key is 1, so attention returns v whatever q, k and the rotation
    are, and the block is h + mlp(norm2(h)) with h = x + Wo . repeat(Wv . norm1(x)) (models/src/llama.rs:401-409).
    Written out here with matrix products only; a block that adds the feed-forward to x instead of h, norms after
    the mixer, or feeds the mixer the unnormed rows fails it."""
    cfg = {"hidden_size": 24, "num_attention_heads": 3, "num_key_value_heads": 1, "rope_theta": 1e4,
           "rms_norm_eps": 1e-5}
    g = torch.Generator().manual_seed(21)
    r = lambda *shape: torch.randn(*shape, generator=g) * 0.5
    p = "model.layers.0."
    w = {p + "input_layernorm.weight": 1 + r(24), p + "post_attention_layernorm.weight": 1 + r(24),
         p + "self_attn.q_proj.weight": r(24, 24), p + "self_attn.k_proj.weight": r(8, 24),
         p + "self_attn.v_proj.weight": r(8, 24), p + "self_attn.o_proj.weight": r(24, 24),
         p + "mlp.gate_proj.weight": r(40, 24), p + "mlp.up_proj.weight": r(40, 24), p + "mlp.down_proj.weight": r(24, 40)}
    x = r(1, 24)

    def norm(t, gamma):
        return t / torch.sqrt((t * t).sum() / 24 + 1e-5) * gamma

    v = norm(x, w[p + "input_layernorm.weight"]) @ w[p + "self_attn.v_proj.weight"].T          # [1, 8]: the one KV head
    h = x + v.repeat(1, 3) @ w[p + "self_attn.o_proj.weight"].T                                  # all three heads read it
    n2 = norm(h, w[p + "post_attention_layernorm.weight"])
    gate, up = n2 @ w[p + "mlp.gate_proj.weight"].T, n2 @ w[p + "mlp.up_proj.weight"].T
    want = h + (gate / (1 + torch.exp(-gate)) * up) @ w[p + "mlp.down_proj.weight"].T
    for pos in (0, 5):      # one key: the position cannot matter either
        got = P.block(x, w, 0, cfg, torch.tensor([pos]))
        assert torch.allclose(got, want, atol=1e-5), (got - want).abs().max()
    # the pin bites: the feed-forward's share and the mixer's share are both far from nothing
    assert (want - h).abs().max() > 1e-2 and (h - x).abs().max() > 1e-2


def test_two_token_attention_by_hand():
    """Two tokens, one head of four columns.  Columns 0 and 2 (the pair that turns by one radian a position whatever
    theta is) are zero in q and k, and theta is so large that the other pair's angle at position 1 is below 1e-14, so
    the rotation changes nothing and token 1's weights are softmax([q1.k0, q1.k1] / sqrt(4)), worked out with exp
    by hand (models/src/llama.rs:342).  A scale of 1/hd, no scale, or a scale applied after the softmax fails it."""
    cfg = {"hidden_size": 4, "num_attention_heads": 1, "num_key_value_heads": 1, "rope_theta": 1e30}
    eye = torch.eye(4)
    wv = torch.tensor([[1.0, 0.5, 0.0, 0.0], [0.0, 1.0, 0.0, 2.0], [3.0, 0.0, 1.0, 0.0], [0.0, -1.0, 0.0, 1.0]])
    w = {"q_proj.weight": eye, "k_proj.weight": eye, "v_proj.weight": wv, "o_proj.weight": eye}
    x = torch.tensor([[0.0, 2.0, 0.0, -1.0], [0.0, 1.0, 0.0, 3.0]])
    out = P.self_attention(x, w, "", cfg, torch.arange(2))
    v = x @ wv.T
    # token 0 sees itself only
    assert torch.allclose(out[0], v[0], atol=1e-6)
    s0, s1 = float(x[1] @ x[0]) / 2.0, float(x[1] @ x[1]) / 2.0          # (2 - 3) / 2 = -0.5, (1 + 9) / 2 = 5
    assert (s0, s1) == (-0.5, 5.0)
    a0 = math.exp(s0) / (math.exp(s0) + math.exp(s1))
    want = a0 * v[0] + (1 - a0) * v[1]
    assert torch.allclose(out[1], want, atol=1e-6)
    # what the plausible slips would give is far from it
    for wrong_scale in (1.0 / 4.0, 1.0):
        t0, t1 = float(x[1] @ x[0]) * wrong_scale, float(x[1] @ x[1]) * wrong_scale
        b0 = math.exp(t0) / (math.exp(t0) + math.exp(t1))
        assert float(((b0 - a0) * (v[0] - v[1])).abs().max()) > 1e-3


def test_grouping_maps_query_heads_to_kv_heads_in_blocks():
    """Query head h reads KV head h // (nh/nkv) (csrc/kernels/flash_fwd_kernel.h:593), not h % nkv."""
    cfg = {"hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2, "rope_theta": 1e4}
    g = torch.Generator().manual_seed(6)
    w = {"q_proj.weight": torch.randn(64, 64, generator=g), "k_proj.weight": torch.randn(32, 64, generator=g),
         "v_proj.weight": torch.randn(32, 64, generator=g), "o_proj.weight": torch.eye(64)}
    x = torch.randn(5, 64, generator=g)
    out = P.self_attention(x, w, "", cfg, torch.arange(5)).view(5, 4, 16)
    # with one token-0-only view: every head's output at position 0 is its KV head's v[0]
    v0 = (x[0] @ w["v_proj.weight"].T).view(2, 16)
    assert torch.allclose(out[0, 0], v0[0], atol=1e-5) and torch.allclose(out[0, 1], v0[0], atol=1e-5)
    assert torch.allclose(out[0, 2], v0[1], atol=1e-5) and torch.allclose(out[0, 3], v0[1], atol=1e-5)


def test_sampling_functions():
    logits = torch.tensor([0.1, 2.0, -1.0, 2.0, 0.5])
    p = P.sampling_distribution(logits, 1.0)
    assert torch.allclose(p, torch.softmax(logits, 0))
    p = P.sampling_distribution(logits, 0.5, top_k=2)
    assert torch.count_nonzero(p) == 2 and p[1] > 0 and p[3] > 0
    p = P.sampling_distribution(logits, 1.0, top_k=1)
    assert torch.count_nonzero(p) == 1 and p[1] > 0           # ties go to the lower id
    p = P.sampling_distribution(logits, 1.0, top_p=0.5)
    assert torch.count_nonzero(p) == 2                          # 0.37 + 0.37 reaches 0.5
    assert P.draw(torch.tensor([0.0, 0.5, 0.0, 0.5]), 0.0) == 1
    assert P.draw(torch.tensor([0.0, 0.5, 0.0, 0.5]), 0.49) == 1
    assert P.draw(torch.tensor([0.0, 0.5, 0.0, 0.5]), 0.51) == 3
    out = P.repeat_penalty(torch.tensor([1.0, -1.0, 2.0]), 2.0, [0, 1, 1])
    assert out.tolist() == [0.5, -2.0, 2.0]
