"""Each part alone, and the generality of their arrangement: a toy architecture, defined here, whose layers
differ (attention with and without a window, a mixer with per-request state of its own, another position
encoding), whose run order names a layer twice and lets a layer read another layer's cache.  It is registered,
written with random weights, built and stepped without a change to the framework's files."""
import dataclasses
import math
from typing import Dict, List

import pytest
import torch

import plain_llama as P
from util import TINY_B, TOL_BF16, TOL_F32, frob_err, plain_weights, random_tokens, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ----------------------------------------------------------------------------------------------------------
# parts alone


def getter(tensors):
    return lambda name: tensors[name]


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(act):
    from atoma_infer_amd.parts import RMSNorm
    g = torch.Generator().manual_seed(0)
    w = (1 + 0.1 * torch.randn(100, generator=g)).to(torch.bfloat16)
    part = RMSNorm(100, 1e-6)
    assert part.weight_specs()["weight"].shape == (100,)
    part.load(getter({"weight": w}), torch.device(DEV), act)
    resid, delta = torch.randn(5, 100, generator=g), torch.randn(5, 100, generator=g).to(act)
    r = resid.to(DEV)
    out = part.add_norm(r, delta.to(DEV))
    want_r = resid + delta.float()
    assert torch.allclose(r.cpu(), want_r)
    want = P.rms_norm(want_r, w.float(), 1e-6)
    assert out.dtype is act
    assert torch.allclose(out.float().cpu(), want, atol=1e-5 if act is torch.float32 else 2e-2, rtol=1e-2)


def test_rotary_part_tables_equal_the_plain_ones():
    from atoma_infer_amd.parts import RotaryEncoding
    rs = {k: v for k, v in TINY_B["rope_scaling"].items() if k != "rope_type"}
    part = RotaryEncoding(32, 500000.0, 256, rs)
    part.prepare(torch.device(DEV))
    cos, sin, rd = part.rotary_tables()
    pc, ps = P.rope_tables(TINY_B, torch.arange(256))
    assert rd == 32 and torch.equal(cos.cpu(), pc) and torch.equal(sin.cpu(), ps)
    # apply: equals the plain rotation
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(4, 3, 32, generator=g), torch.randn(4, 2, 32, generator=g)
    pos = torch.tensor([0, 5, 200, 255], dtype=torch.int32)
    dq, dk = q.to(DEV), k.to(DEV)
    part.apply(dq, dk, pos.to(DEV))
    assert torch.allclose(dq.cpu(), P.apply_rope(q, pc[pos.long()], ps[pos.long()]), atol=1e-6)
    assert torch.allclose(dk.cpu(), P.apply_rope(k, pc[pos.long()], ps[pos.long()]), atol=1e-6)


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,inter", [(64, 96), (96, 250)])
def test_swiglu_part(act, width, inter):
    from atoma_infer_amd.parts import SwiGLU
    g = torch.Generator().manual_seed(2)
    ws = {n: (torch.randn(*s, generator=g) * 0.1).to(torch.bfloat16) for n, s in
          (("gate_proj.weight", (inter, width)), ("up_proj.weight", (inter, width)),
           ("down_proj.weight", (width, inter)))}
    part = SwiGLU(width, inter)
    assert {k: v.shape for k, v in part.weight_specs().items()} == {k: tuple(v.shape) for k, v in ws.items()}
    part.load(getter(ws), torch.device(DEV), act)
    x = torch.randn(7, width, generator=g).to(act)
    y = part.forward(x.to(DEV), None)
    if y.dim() == 3:
        y = y.sum(0)
    want = P.swiglu_mlp(x.float(), {k: v.float() for k, v in ws.items()}, "")
    err = frob_err(y.float(), want)
    assert err < (1e-5 if act is torch.float32 else 1e-2), err


def test_embedding_and_head_parts():
    from atoma_infer_amd.parts import OutputHead, TokenEmbedding
    g = torch.Generator().manual_seed(3)
    table = (torch.randn(50, 32, generator=g)).to(torch.bfloat16)
    emb = TokenEmbedding(50, 32)
    emb.load(getter({"weight": table}), torch.device(DEV), torch.bfloat16)
    tied = OutputHead(32, 50, tied_to=emb)
    assert tied.weight_specs() == {}
    tied.load(getter({}), torch.device(DEV), torch.bfloat16)
    x = torch.randn(3, 32, generator=g).to(torch.bfloat16)
    logits = tied.forward(x.to(DEV))
    assert logits.dtype is torch.float32 and rel_err(logits, x.float() @ table.float().T) < 1e-5
    own = (torch.randn(50, 32, generator=g)).to(torch.bfloat16)
    untied = OutputHead(32, 50)
    assert untied.weight_specs()["weight"].shape == (50, 32)
    untied.load(getter({"weight": own}), torch.device(DEV), torch.bfloat16)
    assert rel_err(untied.forward(x.to(DEV)), x.float() @ own.float().T) < 1e-5
    assert torch.equal(emb.forward(torch.tensor([4, 0, 49], dtype=torch.int32, device=DEV)).cpu(),
                       table.float()[[4, 0, 49]])


class PartCtx:
    """What a mixer reads of a step's context, for one request that brings tokens start .. start + count - 1."""

    def __init__(self, start, count):
        import numpy as np
        self.h_starts, self.h_counts = np.asarray([start], dtype=np.int32), np.asarray([count], dtype=np.int32)
        self.positions = torch.arange(start, start + count, dtype=torch.int32, device=DEV)
        self.token_seq = torch.zeros(count, dtype=torch.int32, device=DEV)
        self.scratch, self.plans = {}, {}


def attention_part(act, nh, nkv, hd, width, window, seed):
    from atoma_infer_amd.parts import PagedAttention, RotaryEncoding
    g = torch.Generator().manual_seed(seed)
    ws = {n: (torch.randn(*sh, generator=g) * 0.2).to(torch.bfloat16) for n, sh in
          (("q_proj.weight", (nh * hd, width)), ("k_proj.weight", (nkv * hd, width)),
           ("v_proj.weight", (nkv * hd, width)), ("o_proj.weight", (width, nh * hd)))}
    part = PagedAttention(width, nh, nkv, hd, RotaryEncoding(hd, 10000.0, 256), window)
    assert {k: v.shape for k, v in part.weight_specs().items()} == {k: tuple(v.shape) for k, v in ws.items()}
    assert part.cache_spec().kv_heads == nkv and part.cache_spec().head_size == hd and part.cache_spec().window == window
    part.load(getter(ws), torch.device(DEV), act)
    return part, ws


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,width,window", [(4, 2, 16, 48, None), (3, 3, 32, 96, 20), (8, 2, 64, 64, None)])
def test_attention_part(act, nh, nkv, hd, width, window):
    """The mixer alone over a cache of its own: a prompt in two portions, then tokens one by one, against the plain
    attention of the whole sequence (projections, rotation, grouped heads, window, output projection)."""
    from atoma_infer_amd.cache.pool import LayerCache
    part, ws = attention_part(act, nh, nkv, hd, width, window, seed=nh + hd)
    page, pages, n = 16, 8, 70
    g = torch.Generator().manual_seed(4)
    x = torch.randn(n, width, generator=g).to(act)
    cfg = {"hidden_size": nh * hd, "num_attention_heads": nh, "num_key_value_heads": nkv, "rope_theta": 10000.0}
    fw = {"p.self_attn." + k: v.float() for k, v in ws.items()}
    # the plain function projects from width to nh * hd itself; it reads hidden_size only for the head size
    want = P.self_attention(x.float(), fw, "p.self_attn.", cfg, torch.arange(n), window)
    order = torch.randperm(pages, generator=g)[: -(-n // page)]
    bt = order.int().view(1, -1).to(DEV)
    k = torch.zeros(pages, nkv, page * hd, dtype=act, device=DEV)
    v = torch.zeros(pages, nkv, page * hd, dtype=act, device=DEV)
    got = []
    for start, count in [(0, 37), (37, 20)] + [(i, 1) for i in range(57, n)]:
        pos = torch.arange(start, start + count)
        slots = (order[pos // page] * page + pos % page).int().to(DEV)
        cache = LayerCache(k=k, v=v, page_size=page, writable=True, group=0, slot_mapping=slots, block_tables=bt)
        y = part.forward(x[start:start + count].to(DEV), PartCtx(start, count), cache)
        got.append((y.sum(0) if y.dim() == 3 else y).float().cpu())
    err = frob_err(torch.cat(got), want)
    assert err < (TOL_F32 if act is torch.float32 else TOL_BF16), err


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 24])
def test_an_encoding_that_biases_scores_by_distance(act, window):
    """A position encoding defined here that rotates nothing and gives each head a slope: the score of the key at j
    for the query at p gains slope * (j - p).  The framework's attention takes it through its general kernel; the
    plain formula is written out below (softmax over the visible keys of q.k * scale + slope * (j - p))."""
    from atoma_infer_amd.cache.pool import LayerCache
    from atoma_infer_amd.parts import PagedAttention, PositionEncoding

    class Slopes(PositionEncoding):
        def graph_safe(self):
            return True

        def apply(self, q, k, positions):
            pass

        def score_slopes(self, num_heads):
            return torch.tensor([2.0 ** (-8.0 * (h + 1) / num_heads) for h in range(num_heads)])

    nh, nkv, hd, width, n, page, pages = 6, 2, 32, 80, 70, 16, 8
    g = torch.Generator().manual_seed(11)
    ws = {name: (torch.randn(*sh, generator=g) * 0.2).to(torch.bfloat16) for name, sh in
          (("q_proj.weight", (nh * hd, width)), ("k_proj.weight", (nkv * hd, width)),
           ("v_proj.weight", (nkv * hd, width)), ("o_proj.weight", (width, nh * hd)))}
    part = PagedAttention(width, nh, nkv, hd, Slopes(), window)
    part.load(getter(ws), torch.device(DEV), act)
    assert part.step_planner(page, act) is None              # the general kernel needs no plan
    x = torch.randn(n, width, generator=g).to(act)
    xf, w = x.double(), {k: v.double() for k, v in ws.items()}
    q = (xf @ w["q_proj.weight"].T).view(n, nh, hd)
    k = (xf @ w["k_proj.weight"].T).view(n, nkv, hd).repeat_interleave(nh // nkv, 1)
    v = (xf @ w["v_proj.weight"].T).view(n, nkv, hd).repeat_interleave(nh // nkv, 1)
    slopes = Slopes().score_slopes(nh).double()
    dist = torch.arange(n)[None, :] - torch.arange(n)[:, None]                  # j - p
    scores = torch.einsum("phd,jhd->hpj", q, k) / math.sqrt(hd) + slopes[:, None, None] * dist[None]
    hidden = (dist > 0) | ((dist <= -window) if window else torch.zeros_like(dist, dtype=torch.bool))
    probs = torch.softmax(scores.masked_fill(hidden[None], float("-inf")), dim=-1)
    want = (torch.einsum("hpj,jhd->phd", probs, v).reshape(n, nh * hd) @ w["o_proj.weight"].T).float()
    # the bias matters: without it the result is another
    plain = torch.softmax((scores - slopes[:, None, None] * dist[None]).masked_fill(hidden[None], float("-inf")), dim=-1)
    assert frob_err((torch.einsum("hpj,jhd->phd", plain, v).reshape(n, nh * hd) @ w["o_proj.weight"].T).float(), want) > 0.05
    order = torch.randperm(pages, generator=g)[: -(-n // page)]
    bt = order.int().view(1, -1).to(DEV)
    kc = torch.zeros(pages, nkv, page * hd, dtype=act, device=DEV)
    vc = torch.zeros(pages, nkv, page * hd, dtype=act, device=DEV)
    got = []
    for start, count in [(0, 37), (37, 20)] + [(i, 1) for i in range(57, n)]:
        pos = torch.arange(start, start + count)
        slots = (order[pos // page] * page + pos % page).int().to(DEV)
        cache = LayerCache(k=kc, v=vc, page_size=page, writable=True, group=0, slot_mapping=slots, block_tables=bt)
        y = part.forward(x[start:start + count].to(DEV), PartCtx(start, count), cache)
        got.append((y.sum(0) if y.dim() == 3 else y).float().cpu())
    err = frob_err(torch.cat(got), want)
    assert err < (TOL_F32 if act is torch.float32 else TOL_BF16), err


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_pre_norm_block_part(act):
    """The arrangement alone: h = x + mixer(norm(x)), y = h + ffn(norm(h)), with the sums left to the next norm."""
    from atoma_infer_amd.cache.pool import LayerCache
    from atoma_infer_amd.parts import PreNormBlock, RMSNorm, SwiGLU
    nh, nkv, hd, width, inter, eps = 4, 2, 16, 64, 96, 1e-5
    mixer, ws = attention_part(act, nh, nkv, hd, width, None, seed=7)
    g = torch.Generator().manual_seed(8)
    fw = {n: (torch.randn(*sh, generator=g) * 0.1).to(torch.bfloat16) for n, sh in
          (("gate_proj.weight", (inter, width)), ("up_proj.weight", (inter, width)), ("down_proj.weight", (width, inter)))}
    n1, n2 = (1 + 0.1 * torch.randn(width, generator=g)).bfloat16(), (1 + 0.1 * torch.randn(width, generator=g)).bfloat16()
    block = PreNormBlock(RMSNorm(width, eps), mixer, RMSNorm(width, eps), SwiGLU(width, inter))
    tensors = {"input_layernorm.weight": n1, "post_attention_layernorm.weight": n2}
    tensors.update({"self_attn." + k: v for k, v in ws.items()})
    tensors.update({"mlp." + k: v for k, v in fw.items()})
    assert set(block.weight_specs()) == set(tensors)
    block.load(getter(tensors), torch.device(DEV), act)
    n, page = 21, 16
    x = torch.randn(n, width, generator=g)
    cfg = {"hidden_size": width, "num_attention_heads": nh, "num_key_value_heads": nkv, "rope_theta": 10000.0,
           "rms_norm_eps": eps}
    pw = {"model.layers.0." + k: v.float() for k, v in tensors.items()}
    want = P.block(x, pw, 0, cfg, torch.arange(n))
    resid = x.clone().to(DEV)
    cache = LayerCache(k=torch.zeros(2, nkv, page * hd, dtype=act, device=DEV),
                       v=torch.zeros(2, nkv, page * hd, dtype=act, device=DEV), page_size=page, writable=True, group=0,
                       slot_mapping=torch.arange(n, dtype=torch.int32, device=DEV),
                       block_tables=torch.tensor([[0, 1]], dtype=torch.int32, device=DEV))
    delta = block.forward(resid, None, PartCtx(0, n), cache)
    y = resid.cpu() + (delta.sum(0) if delta.dim() == 3 else delta).float().cpu()
    err = frob_err(y, want)
    assert err < (TOL_F32 if act is torch.float32 else TOL_BF16), err


def test_part_registries():
    from atoma_infer_amd.parts import make_part, registered_kinds
    assert "attention" in registered_kinds("mixer") and "swiglu" in registered_kinds("feed_forward")
    assert "rmsnorm" in registered_kinds("norm") and {"rotary", "none"} <= set(registered_kinds("position"))
    with pytest.raises(KeyError):
        make_part("mixer", "no-such-mixer")
    with pytest.raises(ValueError):
        make_part("mixer", "attention", width=64, num_heads=4, num_kv_heads=3, head_size=16)
    with pytest.raises(ValueError):
        make_part("mixer", "attention", width=40, num_heads=4, num_kv_heads=4, head_size=10)   # head size refused


# ----------------------------------------------------------------------------------------------------------
# a toy architecture, defined here


def _toy_parts():
    """Parts that exist only in this test: a mixer with state of its own, another position encoding and a
    feed-forward that routes every token to some of its experts."""
    from atoma_infer_amd.parts import (FeedForward, Mixer, PositionEncoding, StateSpec, WeightSpec,
                                       register_feed_forward, register_mixer, register_position)

    class DecayMixer(Mixer):
        """state <- decay * state + x W_in (per token, in order); y = state W_out.  State: [inner] per request."""

        #: (start, tokens) of every entry a mixer with ``align`` > 1 has seen
        seen = []

        def __init__(self, width: int, inner: int, decay: float, align: int = 1):
            self.width, self.inner, self.decay, self.align = width, inner, decay, align

        def weight_specs(self):
            return {"in_proj.weight": WeightSpec((self.inner, self.width)),
                    "out_proj.weight": WeightSpec((self.width, self.inner))}

        def state_spec(self):
            return StateSpec((self.inner,))

        def load(self, get, device, act_dtype):
            self.w_in = get("in_proj.weight").to(device)
            self.w_out = get("out_proj.weight").to(device)
            self.act_dtype = act_dtype

        def forward(self, x, ctx, cache):
            from atoma_infer_amd.parts import linear
            u = linear(x, self.w_in, torch.float32)
            out = torch.empty_like(u)
            row = 0
            for e in range(ctx.n_entries):
                slot, n = int(ctx.h_state_slots[e]), int(ctx.h_counts[e])
                if self.align > 1:
                    # a mixer that scans its tokens in blocks: portions of several tokens must start on a block
                    assert n == 1 or int(ctx.h_starts[e]) % self.align == 0, (int(ctx.h_starts[e]), n)
                    DecayMixer.seen.append((int(ctx.h_starts[e]), n))
                st = cache.state[slot]
                for i in range(n):
                    st.mul_(self.decay).add_(u[row + i])
                    out[row + i] = st
                row += n
            return linear(out.to(self.act_dtype), self.w_out)

    class InterleavedRotary(PositionEncoding):
        """Rotates neighbouring pairs (2i, 2i+1) instead of half-split ones; no tables for the fused kernel."""

        def __init__(self, head_size: int, theta: float):
            self.inv = 1.0 / (theta ** (torch.arange(0, head_size, 2).float() / head_size))

        def load(self, get, device, act_dtype):
            self.inv = self.inv.to(device)

        def apply(self, q, k, positions):
            ang = positions.float()[:, None] * self.inv[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            for x in (q, k):
                if x.numel() == 0:
                    continue
                xf = x.float().clone()   # float() of a float32 tensor is the tensor itself
                a, b = xf[..., 0::2], xf[..., 1::2]
                x[..., 0::2] = (a * c - b * s).to(x.dtype)
                x[..., 1::2] = (b * c + a * s).to(x.dtype)

    class RoutedFeedForward(FeedForward):
        """Every token goes to the ``top`` experts with its largest router logits (float32); their outputs are
        weighted by the softmax over those logits.  An expert is a small gate/up/down feed-forward."""

        def __init__(self, width: int, inter: int, experts: int, top: int):
            self.width, self.inter, self.n, self.top = width, inter, experts, top

        def weight_specs(self):
            d = {"router.weight": WeightSpec((self.n, self.width))}
            for e in range(self.n):
                d[f"experts.{e}.gate_proj.weight"] = WeightSpec((self.inter, self.width))
                d[f"experts.{e}.up_proj.weight"] = WeightSpec((self.inter, self.width))
                d[f"experts.{e}.down_proj.weight"] = WeightSpec((self.width, self.inter))
            return d

        def load(self, get, device, act_dtype):
            self.router = get("router.weight").to(device)
            self.experts = [(torch.cat([get(f"experts.{e}.gate_proj.weight"), get(f"experts.{e}.up_proj.weight")]).to(device),
                             get(f"experts.{e}.down_proj.weight").to(device)) for e in range(self.n)]

        def forward(self, x, ctx):
            from atoma_infer_amd.kernels import ops
            from atoma_infer_amd.parts import linear
            logits = linear(x, self.router, torch.float32)
            val, idx = torch.topk(logits, self.top, dim=-1)
            gate = torch.softmax(val, dim=-1)
            out = torch.zeros(x.shape[0], self.width, dtype=torch.float32, device=x.device)
            for e, (w_gate_up, w_down) in enumerate(self.experts):
                hit = idx == e
                rows = hit.any(-1).nonzero().flatten()        # read on the host: this part is not graph-safe
                if rows.numel() == 0:
                    continue
                y = linear(ops.swiglu(linear(x[rows], w_gate_up)), w_down, torch.float32)
                out.index_add_(0, rows, y * (gate * hit)[rows].sum(-1, keepdim=True))
            return out

    register_mixer("toy_decay", DecayMixer, replace=True)
    register_feed_forward("toy_routed", RoutedFeedForward, replace=True)
    register_position("toy_interleaved", InterleavedRotary, replace=True)


def _toy_architecture():
    from atoma_infer_amd.config import ModelConfig, key, register_architecture
    from atoma_infer_amd.config.base import as_float, as_positive_int
    from atoma_infer_amd.models import LayerCall, ModelSpec
    from atoma_infer_amd.parts import OutputHead, TokenEmbedding, make_part

    @dataclasses.dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architectures = ("ToyMixedForCausalLM",)
        width: int = key(convert=as_positive_int)
        vocab: int = key(convert=as_positive_int)
        heads: int = key(convert=as_positive_int)
        kv_heads: int = key(convert=as_positive_int)
        inter: int = key(convert=as_positive_int)
        eps: float = key(convert=as_float)
        max_positions: int = key(convert=as_positive_int)
        layers: tuple = key(convert=lambda v: tuple(dict(x) for x in v))
        order: tuple = key(convert=lambda v: tuple(dict(x) for x in v))
        align: int = key(convert=as_positive_int, default=1)

        def to_dict(self):
            d = {f.name: getattr(self, f.name) for f in dataclasses.fields(self)}
            d["layers"], d["order"] = [dict(x) for x in self.layers], [dict(x) for x in self.order]
            d["architectures"] = ["ToyMixedForCausalLM"]
            return d

    def build(cfg: ToyConfig) -> ModelSpec:
        hd = cfg.width // cfg.heads
        layers = []
        for i, ld in enumerate(cfg.layers):
            if ld["mixer"] == "attention":
                pos = None
                if ld.get("position") == "rotary":
                    pos = make_part("position", "rotary", head_size=hd, theta=10000.0, max_positions=cfg.max_positions)
                elif ld.get("position") == "interleaved":
                    pos = make_part("position", "toy_interleaved", head_size=hd, theta=100.0)
                mixer = make_part("mixer", "attention", width=cfg.width, num_heads=cfg.heads,
                                  num_kv_heads=cfg.kv_heads, head_size=hd, position=pos, window=ld.get("window"))
            else:
                mixer = make_part("mixer", "toy_decay", width=cfg.width, inner=ld["inner"], decay=ld["decay"],
                                  align=cfg.align)
            if "experts" in ld:
                ffn = make_part("feed_forward", "toy_routed", width=cfg.width, inter=ld["expert_inter"],
                                experts=ld["experts"], top=ld["top"])
            else:
                ffn = make_part("feed_forward", "swiglu", width=cfg.width, intermediate=cfg.inter)
            block = make_part("block", "pre_norm", norm1=make_part("norm", "rmsnorm", width=cfg.width, eps=cfg.eps),
                              mixer=mixer, norm2=make_part("norm", "rmsnorm", width=cfg.width, eps=cfg.eps),
                              feed_forward=ffn,
                              names=("norm_a", "mixer", "norm_b", "ffn"))
            layers.append((f"toy.layers.{i}", block))
        emb = TokenEmbedding(cfg.vocab, cfg.width)
        return ModelSpec(width=cfg.width, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
                         embedding=("toy.embed", emb), layers=layers,
                         final_norm=("toy.final_norm", make_part("norm", "rmsnorm", width=cfg.width, eps=cfg.eps)),
                         head=("toy.head", OutputHead(cfg.width, cfg.vocab)),
                         run_order=[LayerCall(o["layer"], o.get("kv_from")) for o in cfg.order],
                         chunk_alignment=cfg.align)

    register_architecture("ToyMixedForCausalLM", ToyConfig, build, replace=True)


TOY = {
    "architectures": ["ToyMixedForCausalLM"], "width": 64, "vocab": 211, "heads": 4, "kv_heads": 2, "inter": 96,
    "eps": 1e-5, "max_positions": 512,
    "layers": [
        {"mixer": "attention", "position": "rotary"},                       # 0: all keys
        {"mixer": "toy_decay", "inner": 40, "decay": 0.9},                  # 1: state of its own
        {"mixer": "attention", "position": "rotary", "window": 24},         # 2: a window of 24 keys
        {"mixer": "attention", "position": "interleaved"},                  # 3: another position encoding
        {"mixer": "attention"},                                             # 4: no position encoding
    ],
    # layer 1 runs twice (two states), call 6 reads the cache that call 0 wrote, with layer 4's queries
    "order": [{"layer": 0}, {"layer": 1}, {"layer": 2}, {"layer": 3}, {"layer": 1}, {"layer": 4},
              {"layer": 4, "kv_from": 0}],
}


# the same kinds of layers with routed feed-forwards of different sizes.  Compared with the plain model in float32
# only: where two router logits nearly tie, bfloat16 rounding may pick the other expert, which is no fault
TOY_ROUTED = dict(TOY, vocab=157, layers=[
    {"mixer": "attention", "position": "rotary", "experts": 3, "top": 2, "expert_inter": 48},
    {"mixer": "toy_decay", "inner": 24, "decay": 0.8},
    {"mixer": "attention", "position": "rotary", "window": 24, "experts": 5, "top": 1, "expert_inter": 32},
], order=[{"layer": 0}, {"layer": 1}, {"layer": 2}])


def toy_plain_forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    """The toy model on a whole sequence, from the plain implementation's functions."""
    H, nh, nkv = cfg["width"], cfg["heads"], cfg["kv_heads"]
    hd, t = H // nh, len(tokens)
    pos = torch.arange(t)
    x = w["toy.embed.weight"][torch.tensor(tokens)]
    kv_of_call = {}

    def encode(ld, q, k):
        if ld.get("position") == "rotary":
            c, s = P.rope_tables({"hidden_size": H, "num_attention_heads": nh, "rope_theta": 10000.0}, pos)
            return P.apply_rope(q, c, s), (P.apply_rope(k, c, s) if k is not None else None)
        if ld.get("position") == "interleaved":
            inv = 1.0 / (100.0 ** (torch.arange(0, hd, 2).float() / hd))
            ang = pos.float()[:, None] * inv[None]
            c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
            def rot(z):
                a, b = z[..., 0::2], z[..., 1::2]
                out = torch.empty_like(z)
                out[..., 0::2], out[..., 1::2] = a * c - b * s, b * c + a * s
                return out
            return rot(q), (rot(k) if k is not None else None)
        return q, k

    for ci, call in enumerate(cfg["order"]):
        li, ld = call["layer"], cfg["layers"][call["layer"]]
        p = f"toy.layers.{li}."
        h = P.rms_norm(x, w[p + "norm_a.weight"], cfg["eps"])
        if ld["mixer"] == "attention":
            q = (h @ w[p + "mixer.q_proj.weight"].T).view(t, nh, hd)
            if call.get("kv_from") is None:
                k = (h @ w[p + "mixer.k_proj.weight"].T).view(t, nkv, hd)
                v = (h @ w[p + "mixer.v_proj.weight"].T).view(t, nkv, hd)
                q, k = encode(ld, q, k)
                kv_of_call[ci] = (k, v)
            else:
                q, _ = encode(ld, q, None)
                k, v = kv_of_call[call["kv_from"]]
            kk, vv = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
            o = P.attention_scores_softmax_pv(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                              1 / math.sqrt(hd), True, ld.get("window"))
            a = o.transpose(0, 1).reshape(t, H) @ w[p + "mixer.o_proj.weight"].T
        else:
            u = h @ w[p + "mixer.in_proj.weight"].T
            st, ys = torch.zeros(ld["inner"]), []
            for i in range(t):
                st = ld["decay"] * st + u[i]
                ys.append(st)
            a = torch.stack(ys) @ w[p + "mixer.out_proj.weight"].T
        x = x + a
        h = P.rms_norm(x, w[p + "norm_b.weight"], cfg["eps"])
        if "experts" in ld:
            val, idx = torch.topk(h @ w[p + "ffn.router.weight"].T, ld["top"], dim=-1)
            gate = torch.softmax(val, dim=-1)
            y = torch.zeros_like(x)
            for i in range(t):
                for j in range(ld["top"]):
                    y[i] += gate[i, j] * P.swiglu_mlp(h[i:i + 1], w, p + f"ffn.experts.{int(idx[i, j])}.")[0]
            x = x + y
        else:
            x = x + P.swiglu_mlp(h, w, p + "ffn.")
    return P.rms_norm(x, w["toy.final_norm.weight"], cfg["eps"]) @ w["toy.head.weight"].T


@pytest.fixture(scope="module")
def toy_dir(tmp_path_factory):
    _toy_parts()
    _toy_architecture()
    from atoma_infer_amd.weights import write_random_model
    d = str(tmp_path_factory.mktemp("toy"))
    write_random_model(d, TOY, seed=5, dtype="bfloat16", norm_jitter=0.1)
    yield d
    from atoma_infer_amd.config import unregister_architecture
    unregister_architecture("ToyMixedForCausalLM")


def test_toy_cache_plan(toy_dir):
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.config import load_model_config
    arch, cfg = load_model_config(toy_dir)
    plan = plan_cache(arch.build(cfg))
    # attention calls 0, 3, 5 keep all keys (one group), call 2 keeps a window (a group of its own),
    # call 6 reads call 0's entry, calls 1 and 4 each have their own state
    assert [(g.spec.window, g.calls) for g in plan.groups] == [(None, [0, 3, 5]), (24, [2])]
    assert plan.where[6] == (0, 0, False) and sorted(plan.states) == [1, 4] and plan.states[1] == ((40,), "float32")


def _toy_run(model, plan, reqs, schedule, pages):
    """Step ``schedule`` ([(request name, tokens), ...], [names that end]) and collect the logits of every position."""
    from atoma_infer_amd.cache import CachePool
    from atoma_infer_amd.engine import ModelRunner, StepEntry
    pool = CachePool(plan, 16, pages, 3, model.act_dtype, model.device)
    runner = ModelRunner(model, pool)
    ids, got = {}, {}
    for entries, end in schedule:
        batch, places = [], []
        for name, n in entries:
            if name not in ids:
                ids[name] = len(ids)
                runner.add_request(ids[name])
            s = runner.computed_len(ids[name])
            batch.append(StepEntry(ids[name], reqs[name][s:s + n], s, list(range(n))))
            places += [(name, s + i) for i in range(n)]
        logits = runner.step(batch).cpu()
        for r, key in enumerate(places):
            got[key] = logits[r].clone()
        for name in end:
            runner.free_request(ids[name])
        runner.manager.check()
    return got, runner


def _toy_check(got, want, dtype):
    for n in want:
        rows = sorted(p for (m, p) in got if m == n)
        mine, ref = torch.stack([got[(n, p)] for p in rows]), want[n][rows]
        if dtype == "float32":
            assert rel_err(mine, ref) < TOL_F32, n
        else:
            assert frob_err(mine, ref) < TOL_BF16, n


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_steps_like_its_plain_model(toy_dir, dtype):
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.models import load_model
    model = load_model(toy_dir, dtype)
    plan = plan_cache(model.spec)
    w = plain_weights(toy_dir)
    reqs = {n: random_tokens(ln, TOY["vocab"], 60 + i) for i, (n, ln) in enumerate([("a", 120), ("b", 75), ("c", 90)])}
    want = {n: toy_plain_forward(t, w, TOY) for n, t in reqs.items()}

    # whole prompts, one request at a time
    got, _ = _toy_run(model, plan, reqs, [([(n, len(t))], [n]) for n, t in reqs.items()], [8, 8])
    _toy_check(got, want, dtype)
    # portions of changing size beside decoded tokens of other requests; the windowed group has so few pages
    # (12 of 16 tokens, where the three requests would need 19 without giving any back) that it only works because passed pages return
    sched = [([("a", 50), ("b", 2)], []), ([("a", 1), ("b", 33), ("c", 17)], []), ([("a", 30), ("c", 2)], []),
             ([("b", 40), ("a", 1), ("c", 1)], ["b"]), ([("a", 38), ("c", 3)], ["a"]), ([("c", 60)], []),
             ([("c", 1)], []), ([("c", 1)], []), ([("c", 5)], ["c"])]
    got, runner = _toy_run(model, plan, reqs, sched, [19, 12])
    _toy_check(got, want, dtype)
    assert runner.manager.num_free_pages(0) == 19 and runner.manager.num_free_pages(1) == 12


@pytest.fixture(scope="module")
def routed_dir(tmp_path_factory, toy_dir):
    from atoma_infer_amd.weights import write_random_model
    d = str(tmp_path_factory.mktemp("toy_routed"))
    write_random_model(d, TOY_ROUTED, seed=9, dtype="bfloat16", norm_jitter=0.1)
    return d


def test_routed_feed_forward_and_steps_that_cannot_be_replayed(routed_dir):
    """A feed-forward with routing, and single decoded tokens of requests that take turns: the toy parts read the
    step on the host, so such steps must not be recorded into a graph with one request's state slot in it."""
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.models import load_model, random_model
    w = plain_weights(routed_dir)
    reqs = {n: random_tokens(ln, TOY_ROUTED["vocab"], 80 + i) for i, (n, ln) in enumerate([("a", 70), ("b", 41)])}
    want = {n: toy_plain_forward(t, w, TOY_ROUTED) for n, t in reqs.items()}
    turns = [([("a", 60), ("b", 32)], [])] + [([(n, 1)], []) for _ in range(8) for n in ("a", "b")] \
        + [([("a", 2), ("b", 1)], ["a", "b"])]
    model = load_model(routed_dir, "float32")
    assert not model.spec.graph_safe()
    plan = plan_cache(model.spec)
    got, runner = _toy_run(model, plan, reqs, [([(n, len(t))], [n]) for n, t in reqs.items()], [8, 8])
    _toy_check(got, want, "float32")
    assert not runner.use_graphs
    got, _ = _toy_run(model, plan, reqs, turns, [8, 8])
    _toy_check(got, want, "float32")
    # bfloat16: the same steps against whole prompts of the same engine
    model = load_model(routed_dir, "bfloat16")
    whole, _ = _toy_run(model, plan, reqs, [([(n, len(t))], [n]) for n, t in reqs.items()], [8, 8])
    got, _ = _toy_run(model, plan, reqs, turns, [8, 8])
    for key, row in got.items():
        assert frob_err(row[None], whole[key][None]) < TOL_BF16, key
    # the architecture this framework serves is made of parts that can be replayed
    assert random_model(TINY_B, seed=1, dtype="bfloat16").spec.graph_safe()


def test_toy_architecture_generates_through_the_engine(toy_dir):
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    w = plain_weights(toy_dir)
    prompts = [random_tokens(19, TOY["vocab"], 1), random_tokens(3, TOY["vocab"], 2)]
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(5):
            seq.append(int(torch.argmax(toy_plain_forward(seq, w, TOY)[-1])))
        want.append(seq[len(p):])
    eng = LlmEngine(toy_dir, "float32", cache=CacheConfig(block_size=16, num_gpu_blocks_override=8),
                    scheduler=SchedulerConfig(max_num_batched_tokens=8, max_num_sequences=2, max_model_len=64))
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=5, ignore_eos_token=True))
    assert [o.inference_outputs[0].token_ids for o in outs] == want


def test_prompts_are_cut_where_the_model_allows(tmp_path):
    """The toy model with ``chunk_alignment`` 8 (its state mixer asserts that portions of several tokens start on a
    multiple of 8): prompts of 45 and 30 tokens under a budget of 21 tokens a step, a pool so small that one request
    is preempted and computed again, against the plain model."""
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    from atoma_infer_amd.weights import write_random_model
    _toy_parts()
    _toy_architecture()
    cfg = dict(TOY, align=8)
    d = write_random_model(str(tmp_path / "toy8"), cfg, seed=5, dtype="bfloat16", norm_jitter=0.1)
    w = plain_weights(d)
    prompts = [random_tokens(45, TOY["vocab"], 7), random_tokens(30, TOY["vocab"], 8)]
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(12):
            seq.append(int(torch.argmax(toy_plain_forward(seq, w, cfg)[-1])))
        want.append(seq[len(p):])
    eng = LlmEngine(d, "float32", cache=CacheConfig(block_size=16, num_gpu_blocks_override=6),
                    scheduler=SchedulerConfig(max_num_batched_tokens=21, max_num_sequences=2, max_model_len=64))
    assert eng.model.spec.chunk_alignment == 8
    mixer_cls = type(eng.model.spec.layers[1][1].mixer)
    del mixer_cls.seen[:]
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=12, ignore_eos_token=True))
    assert [o.inference_outputs[0].token_ids for o in outs] == want
    portions = [(s0, n) for s0, n in mixer_cls.seen if n > 1]
    assert portions and all(s0 % 8 == 0 for s0, _ in portions)
    assert any(n == 16 for _, n in portions) and any(n % 8 for _, n in portions)    # 21 -> 16; the last is ragged
    assert eng.stats["preemptions"] > 0


# ----------------------------------------------------------------------------------------------------------
# a second toy architecture: another norm and another arrangement of a block


def _parallel_parts():
    """A norm that subtracts the mean and has a bias, and a block whose mixer and feed-forward both read the same
    normed input and whose outputs are added to the residual stream together."""
    from atoma_infer_amd.parts import Block, Norm, WeightSpec, register_block, register_norm

    class ShiftScaleNorm(Norm):
        def __init__(self, width: int, eps: float):
            self.width, self.eps = width, eps

        def weight_specs(self):
            return {"weight": WeightSpec((self.width,), "norm"), "bias": WeightSpec((self.width,))}

        def load(self, get, device, act_dtype):
            self.weight, self.bias = get("weight").to(device).float(), get("bias").to(device).float()
            self.act_dtype = act_dtype

        def add_norm(self, resid, delta, rows=None):
            if delta is not None:
                delta = delta.float().sum(0) if delta.dim() == 3 else delta.float()
            if rows is None:
                if delta is not None:
                    resid += delta
                x = resid
            else:
                sel = rows.long()
                x = resid[sel] if delta is None else resid[sel] + delta[sel]
            mu = x.mean(-1, keepdim=True)
            var = ((x - mu) ** 2).mean(-1, keepdim=True)
            return ((x - mu) * torch.rsqrt(var + self.eps) * self.weight + self.bias).to(self.act_dtype)

    class ParallelBlock(Block):
        def __init__(self, norm, mixer, feed_forward):
            self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward

        def _children(self):
            return (("norm", self.norm), ("mixer", self.mixer), ("ffn", self.feed_forward))

        def weight_specs(self):
            return {f"{n}.{k}": ws for n, part in self._children() for k, ws in part.weight_specs().items()}

        def load(self, get, device, act_dtype):
            for n, part in self._children():
                part.load(lambda rel, _n=n: get(f"{_n}.{rel}"), device, act_dtype)

        def forward(self, resid, delta, ctx, cache):
            x = self.norm.add_norm(resid, delta)
            outs = [self.mixer.forward(x, ctx, cache), self.feed_forward.forward(x, ctx)]
            # either may come as float32 planes of a split product; the next norm sums whatever it is given
            return torch.stack([o.float().sum(0) if o.dim() == 3 else o.float() for o in outs])

    register_norm("toy_shift_scale", ShiftScaleNorm, replace=True)
    register_block("toy_parallel", ParallelBlock, replace=True)


def _parallel_architecture():
    from atoma_infer_amd.config import ModelConfig, key, register_architecture
    from atoma_infer_amd.config.base import as_float, as_positive_int
    from atoma_infer_amd.models import ModelSpec
    from atoma_infer_amd.parts import OutputHead, TokenEmbedding, make_part

    @dataclasses.dataclass(frozen=True)
    class ParallelConfig(ModelConfig):
        architectures = ("ToyParallelForCausalLM",)
        width: int = key(convert=as_positive_int)
        vocab: int = key(convert=as_positive_int)
        heads: int = key(convert=as_positive_int)
        kv_heads: int = key(convert=as_positive_int)
        inter: int = key(convert=as_positive_int)
        depth: int = key(convert=as_positive_int)
        eps: float = key(convert=as_float)
        max_positions: int = key(convert=as_positive_int)

        def to_dict(self):
            d = {f.name: getattr(self, f.name) for f in dataclasses.fields(self)}
            d["architectures"] = ["ToyParallelForCausalLM"]
            return d

    def build(cfg: ParallelConfig) -> ModelSpec:
        hd = cfg.width // cfg.heads
        norm = lambda: make_part("norm", "toy_shift_scale", width=cfg.width, eps=cfg.eps)
        layers = []
        for i in range(cfg.depth):
            pos = make_part("position", "rotary", head_size=hd, theta=10000.0, max_positions=cfg.max_positions)
            mixer = make_part("mixer", "attention", width=cfg.width, num_heads=cfg.heads, num_kv_heads=cfg.kv_heads,
                              head_size=hd, position=pos)
            ffn = make_part("feed_forward", "swiglu", width=cfg.width, intermediate=cfg.inter)
            layers.append((f"par.layers.{i}", make_part("block", "toy_parallel", norm=norm(), mixer=mixer,
                                                        feed_forward=ffn)))
        return ModelSpec(width=cfg.width, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
                         embedding=("par.embed", TokenEmbedding(cfg.vocab, cfg.width)), layers=layers,
                         final_norm=("par.final_norm", norm()), head=("par.head", OutputHead(cfg.width, cfg.vocab)))

    register_architecture("ToyParallelForCausalLM", ParallelConfig, build, replace=True)


TOY_PARALLEL = {"architectures": ["ToyParallelForCausalLM"], "width": 96, "vocab": 173, "heads": 6, "kv_heads": 3,
                "inter": 136, "depth": 3, "eps": 1e-4, "max_positions": 256}


def parallel_plain_forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    H, nh, nkv = cfg["width"], cfg["heads"], cfg["kv_heads"]
    hd, t = H // nh, len(tokens)

    def norm(x, p):
        mu = x.mean(-1, keepdim=True)
        return (x - mu) / torch.sqrt(((x - mu) ** 2).mean(-1, keepdim=True) + cfg["eps"]) * w[p + "weight"] + w[p + "bias"]

    c, s = P.rope_tables({"hidden_size": H, "num_attention_heads": nh, "rope_theta": 10000.0}, torch.arange(t))
    x = w["par.embed.weight"][torch.tensor(tokens)]
    for i in range(cfg["depth"]):
        p = f"par.layers.{i}."
        h = norm(x, p + "norm.")
        q = P.apply_rope((h @ w[p + "mixer.q_proj.weight"].T).view(t, nh, hd), c, s)
        k = P.apply_rope((h @ w[p + "mixer.k_proj.weight"].T).view(t, nkv, hd), c, s)
        v = (h @ w[p + "mixer.v_proj.weight"].T).view(t, nkv, hd)
        kk, vv = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
        o = P.attention_scores_softmax_pv(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                          1 / math.sqrt(hd), True, None)
        x = x + o.transpose(0, 1).reshape(t, H) @ w[p + "mixer.o_proj.weight"].T + P.swiglu_mlp(h, w, p + "ffn.")
    return norm(x, "par.final_norm.") @ w["par.head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_another_norm_and_another_block_arrangement(tmp_path, dtype):
    """Registered here, built from config.json, loaded, stepped in portions beside decoded tokens: nothing in the
    framework's files knows of them."""
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.config import unregister_architecture
    from atoma_infer_amd.models import load_model
    from atoma_infer_amd.weights import write_random_model
    _parallel_parts()
    _parallel_architecture()
    try:
        d = write_random_model(str(tmp_path / "par"), TOY_PARALLEL, seed=4, dtype="bfloat16", norm_jitter=0.1)
        model = load_model(d, dtype)
        assert not model.spec.graph_safe()          # the toy parts do not say they can be replayed
        plan = plan_cache(model.spec)
        w = plain_weights(d)
        reqs = {n: random_tokens(ln, TOY_PARALLEL["vocab"], 30 + i) for i, (n, ln) in enumerate([("a", 100), ("b", 37)])}
        want = {n: parallel_plain_forward(t, w, TOY_PARALLEL) for n, t in reqs.items()}
        sched = [([("a", 64)], []), ([("a", 3), ("b", 30)], []), ([("a", 1), ("b", 1)], []), ([("b", 2), ("a", 1)], []),
                 ([("a", 31), ("b", 4)], ["a", "b"])]
        got, runner = _toy_run(model, plan, reqs, sched, [10])
        _toy_check(got, want, dtype)
        assert runner.manager.num_free_pages(0) == 10
    finally:
        unregister_architecture("ToyParallelForCausalLM")


def test_toy_state_survives_preemption(toy_dir):
    """Three requests in a pool that holds less than two at their full length (the window group admits only what
    it can carry, so the squeeze must come from growth): one is preempted and computed again later.  Its mixer state
    must start from zero then (the slot it gets may have been another request's), or its tokens change."""
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    w = plain_weights(toy_dir)
    prompts = [random_tokens(20 + 3 * i, TOY["vocab"], 40 + i) for i in range(3)]
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(20):
            seq.append(int(torch.argmax(toy_plain_forward(seq, w, TOY)[-1])))
        want.append(seq[len(p):])
    eng = LlmEngine(toy_dir, "float32", cache=CacheConfig(block_size=16, num_gpu_blocks_override=5),
                    scheduler=SchedulerConfig(max_num_batched_tokens=32, max_num_sequences=3, max_model_len=64))
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=20, ignore_eos_token=True))
    assert eng.stats["preemptions"] > 0
    assert [o.inference_outputs[0].token_ids for o in outs] == want
    assert eng.runner.manager.num_requests() == 0


# ----------------------------------------------------------------------------------------------------------
# a mixer whose cache is one latent vector per token, and whose state is a counter of integers


def _latent_parts():
    """Attention over cached latent vectors: a token leaves c = x Wc^T (``latent`` numbers, one head, no second
    tensor) in its page; a query head scores the latents themselves and sums them, and Wo maps the heads' sums back.
    The state counts, in int32, the tokens the request has brought."""
    from atoma_infer_amd.parts import CacheSpec, Mixer, StateSpec, WeightSpec, register_mixer

    class LatentMixer(Mixer):
        def __init__(self, width: int, latent: int, heads: int):
            self.width, self.latent, self.heads = width, latent, heads

        def weight_specs(self):
            return {"c_proj.weight": WeightSpec((self.latent, self.width)),
                    "q_proj.weight": WeightSpec((self.heads * self.latent, self.width)),
                    "o_proj.weight": WeightSpec((self.width, self.heads * self.latent))}

        def load(self, get, device, act_dtype):
            self.wc, self.wq, self.wo = (get(n + ".weight").to(device).float() for n in ("c_proj", "q_proj", "o_proj"))

        def cache_spec(self):
            return CacheSpec(kv_heads=1, head_size=self.latent, value_size=0)

        def state_spec(self):
            return StateSpec((1,), "int32")

        def forward(self, x, ctx, cache):
            assert cache.v is None and cache.state.dtype is torch.int32
            L, page = self.latent, cache.page_size
            xf = x.float()
            lat = cache.k.view(-1, L)                     # this mixer's tile order: token after token
            lat[cache.slot_mapping.long()] = (xf @ self.wc.T).to(lat.dtype)
            q = (xf @ self.wq.T).view(-1, self.heads, L)
            out = torch.empty_like(q)
            row = 0
            for e in range(ctx.n_entries):
                start, n = int(ctx.h_starts[e]), int(ctx.h_counts[e])
                slot = int(ctx.h_state_slots[e])
                assert int(cache.state[slot, 0]) == start, "the counter follows the request, whatever its slot was"
                cache.state[slot, 0] += n
                total = start + n
                pages = cache.block_tables[e, : -(-total // page)].long()
                seen = cache.k.view(-1, page, L)[pages].reshape(-1, L)[:total].float()
                s = torch.einsum("nhl,sl->hns", q[row: row + n], seen) / math.sqrt(L)
                far = torch.arange(total, device=x.device)[None, :] > (start + torch.arange(n, device=x.device))[:, None]
                p = torch.softmax(s.masked_fill(far[None], float("-inf")), dim=-1)
                out[row: row + n] = torch.einsum("hns,sl->nhl", p, seen)
                row += n
            return (out.reshape(-1, self.heads * L) @ self.wo.T).to(x.dtype)

    register_mixer("toy_latent", LatentMixer, replace=True)


TOY_LATENT = {"architectures": ["ToyLatentForCausalLM"], "width": 80, "vocab": 211, "latent": 24, "heads": 3,
              "attn_heads": 5, "attn_kv_heads": 1, "inter": 112, "depth": 3, "eps": 1e-5, "max_positions": 256}


def _latent_architecture():
    from atoma_infer_amd.config import ModelConfig, key, register_architecture
    from atoma_infer_amd.config.base import as_float, as_positive_int
    from atoma_infer_amd.models import ModelSpec
    from atoma_infer_amd.parts import OutputHead, TokenEmbedding, make_part

    @dataclasses.dataclass(frozen=True)
    class LatentConfig(ModelConfig):
        architectures = ("ToyLatentForCausalLM",)
        width: int = key(convert=as_positive_int)
        vocab: int = key(convert=as_positive_int)
        latent: int = key(convert=as_positive_int)
        heads: int = key(convert=as_positive_int)
        attn_heads: int = key(convert=as_positive_int)
        attn_kv_heads: int = key(convert=as_positive_int)
        inter: int = key(convert=as_positive_int)
        depth: int = key(convert=as_positive_int)
        eps: float = key(convert=as_float)
        max_positions: int = key(convert=as_positive_int)

        def to_dict(self):
            d = {f.name: getattr(self, f.name) for f in dataclasses.fields(self)}
            d["architectures"] = ["ToyLatentForCausalLM"]
            return d

    def build(cfg: LatentConfig) -> ModelSpec:
        norm = lambda: make_part("norm", "rmsnorm", width=cfg.width, eps=cfg.eps)
        hd = cfg.width // cfg.attn_heads
        layers = []
        for i in range(cfg.depth):
            if i % 2 == 0:
                mixer = make_part("mixer", "toy_latent", width=cfg.width, latent=cfg.latent, heads=cfg.heads)
            else:       # the framework's attention between them: its keys and values lie in a group of their own
                pos = make_part("position", "rotary", head_size=hd, theta=10000.0, max_positions=cfg.max_positions)
                mixer = make_part("mixer", "attention", width=cfg.width, num_heads=cfg.attn_heads,
                                  num_kv_heads=cfg.attn_kv_heads, head_size=hd, position=pos)
            ffn = make_part("feed_forward", "swiglu", width=cfg.width, intermediate=cfg.inter)
            layers.append((f"lat.layers.{i}", make_part("block", "pre_norm", norm1=norm(), mixer=mixer, norm2=norm(),
                                                        feed_forward=ffn, names=("n1", "mix", "n2", "ffn"))))
        return ModelSpec(width=cfg.width, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
                         embedding=("lat.embed", TokenEmbedding(cfg.vocab, cfg.width)), layers=layers,
                         final_norm=("lat.final_norm", norm()), head=("lat.head", OutputHead(cfg.width, cfg.vocab)))

    register_architecture("ToyLatentForCausalLM", LatentConfig, build, replace=True)


def latent_plain_forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    H, L, nh, t = cfg["width"], cfg["latent"], cfg["heads"], len(tokens)
    ah, akv = cfg["attn_heads"], cfg["attn_kv_heads"]
    hd = H // ah
    rms = lambda x, g: x / torch.sqrt((x * x).mean(-1, keepdim=True) + cfg["eps"]) * g
    c, s = P.rope_tables({"hidden_size": H, "num_attention_heads": ah, "rope_theta": 10000.0}, torch.arange(t))
    x = w["lat.embed.weight"][torch.tensor(tokens)]
    for i in range(cfg["depth"]):
        p = f"lat.layers.{i}."
        h = rms(x, w[p + "n1.weight"])
        if i % 2 == 0:
            lat = h @ w[p + "mix.c_proj.weight"].T
            q = (h @ w[p + "mix.q_proj.weight"].T).view(t, nh, L).transpose(0, 1)
            kv = lat[None].expand(nh, t, L)
            o = P.attention_scores_softmax_pv(q, kv, kv, 1 / math.sqrt(L), True, None)
            x = x + o.transpose(0, 1).reshape(t, nh * L) @ w[p + "mix.o_proj.weight"].T
        else:
            q = P.apply_rope((h @ w[p + "mix.q_proj.weight"].T).view(t, ah, hd), c, s)
            k = P.apply_rope((h @ w[p + "mix.k_proj.weight"].T).view(t, akv, hd), c, s)
            v = (h @ w[p + "mix.v_proj.weight"].T).view(t, akv, hd)
            kk, vv = k.repeat_interleave(ah // akv, 1), v.repeat_interleave(ah // akv, 1)
            o = P.attention_scores_softmax_pv(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                              1 / math.sqrt(hd), True, None)
            x = x + o.transpose(0, 1).reshape(t, H) @ w[p + "mix.o_proj.weight"].T
        x = x + P.swiglu_mlp(rms(x, w[p + "n2.weight"]), w, p + "ffn.")
    return rms(x, w["lat.final_norm.weight"]) @ w["lat.head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_cache_of_latent_vectors_and_a_state_of_integers(tmp_path, dtype):
    """A mixer that keeps one tensor per token, of a width of its own and in a tile order of its own, beside layers
    of the framework's attention: the pool gives it pages of its own group and no second tensor, its state is
    int32, and the steps (portions beside decoded tokens, pages reused) equal the whole-sequence formula."""
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.config import unregister_architecture
    from atoma_infer_amd.models import load_model
    from atoma_infer_amd.parts import CacheSpec
    from atoma_infer_amd.weights import write_random_model
    _latent_parts()
    _latent_architecture()
    try:
        d = write_random_model(str(tmp_path / "lat"), TOY_LATENT, seed=6, dtype="bfloat16", norm_jitter=0.1)
        model = load_model(d, dtype)
        plan = plan_cache(model.spec)
        assert [(g.spec, g.calls) for g in plan.groups] == [
            (CacheSpec(1, 24, None, 0), [0, 2]), (CacheSpec(1, 16, None), [1])]
        elem = 2
        assert plan.bytes_per_token(elem) == (2 * 24 + 2 * 16) * elem
        assert plan.states == {0: ((1,), "int32"), 2: ((1,), "int32")}
        w = plain_weights(d)
        reqs = {n: random_tokens(ln, TOY_LATENT["vocab"], 70 + i) for i, (n, ln) in enumerate([("a", 90), ("b", 41), ("c", 60)])}
        want = {n: latent_plain_forward(t, w, TOY_LATENT) for n, t in reqs.items()}
        sched = [([("a", 50)], []), ([("a", 3), ("b", 30)], []), ([("a", 1), ("b", 1)], []), ([("b", 10), ("a", 36)], ["a", "b"]),
                 ([("c", 17)], []), ([("c", 2)], []), ([("c", 1)], []), ([("c", 40)], ["c"])]
        got, runner = _toy_run(model, plan, reqs, sched, [9, 9])
        _toy_check(got, want, dtype)
        assert runner.pool.v[0] is None and runner.pool.v[1] is not None
        assert runner.manager.num_free_pages(0) == 9 and runner.manager.num_free_pages(1) == 9
    finally:
        unregister_architecture("ToyLatentForCausalLM")
