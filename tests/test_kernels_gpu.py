"""Each kernel alone against a plain float32 formula in PyTorch, at sizes other than the engine's."""
import ctypes
import math

import pytest
import torch

from util import force_chunked_decode

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_embed(wdt):
    from atoma_infer_amd.kernels import ops
    table = rnd(37, 24, dtype=wdt)
    tok = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = ops.embed(tok, table)
    assert out.dtype is torch.float32
    assert torch.equal(out, table.float()[tok.long()])


@pytest.mark.parametrize("width", [24, 96, 1000, 2048, 5000])
@pytest.mark.parametrize("ddt,wdt,odt", [(torch.float32, torch.float32, torch.float32),
                                         (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                         (torch.float32, torch.bfloat16, torch.bfloat16)])
def test_add_rmsnorm(width, ddt, wdt, odt):
    from atoma_infer_amd.kernels import ops
    eps = 3e-6
    resid, delta, w = rnd(7, width, seed=1), rnd(7, width, dtype=ddt, seed=2), rnd(width, dtype=wdt, seed=3)
    want_resid = resid + delta.float()
    want = want_resid * torch.rsqrt(want_resid.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    r = resid.clone()
    out = ops.add_rmsnorm(r, delta, w, eps, odt)
    assert torch.allclose(r, want_resid, rtol=0, atol=0)
    tol = 1e-5 if odt is torch.float32 else 1e-2
    assert torch.allclose(out.float(), want, rtol=tol, atol=tol)
    # selected rows: resid stays, rows come out in the order asked
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    r2 = resid.clone()
    out2 = ops.add_rmsnorm(r2, delta, w, eps, odt, rows=rows)
    assert torch.equal(r2, resid)
    assert torch.allclose(out2.float(), want[rows.long()], rtol=tol, atol=tol)
    # without delta, and with planes
    out3 = ops.add_rmsnorm(resid.clone(), None, w, eps, torch.float32)
    want3 = resid * torch.rsqrt(resid.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    assert torch.allclose(out3, want3, rtol=1e-5, atol=1e-5)
    planes = torch.stack([delta.float() * 0.25, delta.float() * 0.5, delta.float() * 0.25])
    r4 = resid.clone()
    ops.add_rmsnorm(r4, planes.contiguous(), w, eps, torch.float32)
    assert torch.allclose(r4, want_resid, rtol=1e-6, atol=1e-6)


def test_rmsnorm_properties():
    """weight 1 and eps -> 0 gives unit RMS; scaling the input leaves the output (nearly) unchanged."""
    from atoma_infer_amd.kernels import ops
    x = rnd(3, 333, seed=5)
    one = torch.ones(333, device=DEV)
    y = ops.add_rmsnorm(x.clone(), None, one, 1e-12, torch.float32)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(3, device=DEV), atol=1e-5)
    y2 = ops.add_rmsnorm((x * 7.5).clone(), None, one, 1e-12, torch.float32)
    assert torch.allclose(y, y2, atol=1e-5)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inter", [10, 100, 250, 1024])
def test_swiglu(dt, inter):
    from atoma_infer_amd.kernels import ops
    gu = rnd(5, 2 * inter, dtype=dt, seed=4, scale=3.0)
    out = ops.swiglu(gu)
    g, u = gu.float()[:, :inter], gu.float()[:, inter:]
    want = torch.nn.functional.silu(g) * u
    tol = 1e-6 if dt is torch.float32 else 2e-2
    assert torch.allclose(out.float(), want, rtol=tol, atol=tol)
    z = torch.zeros(2, 2 * inter, dtype=dt, device=DEV)
    z[:, inter:] = 3.0
    assert torch.count_nonzero(ops.swiglu(z)) == 0  # gate 0 -> 0


@pytest.mark.parametrize("m,n,k", [(1, 5, 7), (3, 64, 64), (65, 130, 33), (130, 70, 250), (17, 1000, 96)])
@pytest.mark.parametrize("adt,wdt,cdt", [(torch.float32, torch.float32, torch.float32),
                                         (torch.float32, torch.bfloat16, torch.float32),
                                         (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                         (torch.bfloat16, torch.float32, torch.float32)])
def test_gemm_generic(m, n, k, adt, wdt, cdt):
    from atoma_infer_amd.kernels import ops
    a, w = rnd(m, k, dtype=adt, seed=1), rnd(n, k, dtype=wdt, seed=2)
    c = ops.gemm_generic(a, w, cdt)
    want = (a.double().cpu() @ w.double().cpu().T)
    tol = 2e-6 * math.sqrt(k) * 10 if cdt is torch.float32 else 2e-2
    assert (c.double().cpu() - want).abs().max() <= tol * want.abs().max()
    # strided activations (a column slice of a wider matrix)
    wide = rnd(m, k + 9, dtype=adt, seed=3)
    c2 = ops.gemm_generic(wide[:, 4:4 + k], w, cdt)
    want2 = wide[:, 4:4 + k].double().cpu() @ w.double().cpu().T
    assert (c2.double().cpu() - want2).abs().max() <= tol * want2.abs().max()


@pytest.mark.parametrize("m", [1, 7, 16, 17, 48, 64])
@pytest.mark.parametrize("n,k", [(16, 32), (100, 64), (3072, 2048), (2048, 8192), (1000, 96), (40000, 128),
                                 (70000, 64)])
@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
def test_gemm_bf16_skinny(m, n, k, cdt):
    from atoma_infer_amd.kernels import gemm_bf16
    a, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2)
    want = a.double().cpu() @ w.double().cpu().T
    tol = 1e-5 if cdt is torch.float32 else 1e-2
    # the kernel itself, with the plan the engine would pick, whole and split along K
    c = torch.empty((m, n), dtype=cdt, device=DEV)
    gemm_bf16.skinny(a, w, c)
    assert (c.double().cpu() - want).abs().max() <= tol * want.abs().max()
    rt, wk, slices = gemm_bf16._plan(m, n, k, True)
    planes = torch.empty((slices, m, n), dtype=torch.float32, device=DEV)
    gemm_bf16.skinny(a, w, planes, slices, rt, wk)
    assert (planes.sum(0).double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()
    # the ways in which parts call it: this kernel or the library, whichever is quicker at the shape
    c = gemm_bf16.try_linear(a, w, cdt)
    assert c is not None and c.dtype is cdt
    assert (c.double().cpu() - want).abs().max() <= tol * want.abs().max()
    planes = gemm_bf16.linear_planes(a, w)
    assert planes.dim() == 3
    assert (planes.sum(0).double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()


@pytest.mark.parametrize("m", [3, 20, 33, 64])
@pytest.mark.parametrize("rt,wk,slices", [(1, 1, 1), (2, 1, 2), (4, 1, 1), (1, 4, 8), (2, 4, 4), (4, 4, 8), (4, 4, 1),
                                          (1, 8, 2), (2, 8, 1)])
@pytest.mark.parametrize("n,k", [(2048, 2048), (200, 4096), (72, 2048)])
def test_gemm_bf16_skinny_every_shape_of_wave(m, rt, wk, slices, n, k):
    """Every way of dealing the rows of W and the steps of K to waves gives the same product, whatever the plan
    would pick at the size."""
    from atoma_infer_amd.kernels import gemm_bf16
    a, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2)
    want = a.double().cpu() @ w.double().cpu().T
    planes = torch.full((slices, m, n), float("nan"), dtype=torch.float32, device=DEV)
    gemm_bf16.skinny(a, w, planes, slices, rt, wk)
    assert (planes.sum(0).double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()


def test_gemm_bf16_rows_do_not_depend_on_the_batch():
    from atoma_infer_amd.kernels import gemm_bf16
    a, w = rnd(64, 512, dtype=torch.bfloat16, seed=1), rnd(300, 512, dtype=torch.bfloat16, seed=2)
    full = torch.empty((64, 300), dtype=torch.float32, device=DEV)
    gemm_bf16.skinny(a, w, full)
    for lo, hi in [(0, 1), (5, 6), (10, 33), (63, 64)]:
        part = torch.empty((hi - lo, 300), dtype=torch.float32, device=DEV)
        gemm_bf16.skinny(a[lo:hi], w, part)
        assert torch.equal(part, full[lo:hi])


def test_gemm_bf16_float32_out_for_many_rows():
    from atoma_infer_amd.kernels import gemm_bf16
    a, w = rnd(150, 64, dtype=torch.bfloat16, seed=1), rnd(333, 64, dtype=torch.bfloat16, seed=2)
    c = gemm_bf16.try_linear(a, w, torch.float32)
    want = a.double().cpu() @ w.double().cpu().T
    assert (c.double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()
    cb = gemm_bf16.try_linear(a, w, torch.bfloat16)   # the library product
    assert (cb.double().cpu() - want).abs().max() <= 1e-2 * want.abs().max()
    # K no multiple of 32: the streaming kernel refuses; few rows then go to the float32 kernel, many to the library
    assert gemm_bf16.try_linear(a[:8, :40], w[:, :40], torch.float32) is None
    c = gemm_bf16.try_linear(a[:, :40], w[:, :40], torch.float32)
    if c is not None:
        want = a[:, :40].double().cpu() @ w[:, :40].double().cpu().T
        assert (c.double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()


# ----------------------------------------------------------------------------------------------------------
# attention kernels against plain softmax(QK^T)V


class FakeCtx:
    """Only what the attention wrappers read of a StepContext."""

    def __init__(self, starts, counts):
        import numpy as np
        self.h_starts = np.asarray(starts, dtype=np.int32)
        self.h_counts = np.asarray(counts, dtype=np.int32)
        qs = [0]
        for c in counts:
            qs.append(qs[-1] + c)
        self.q_start = torch.tensor(qs, dtype=torch.int32, device=DEV)
        pos, seq = [], []
        for e, (s, c) in enumerate(zip(starts, counts)):
            pos += list(range(s, s + c))
            seq += [e] * c
        self.positions = torch.tensor(pos, dtype=torch.int32, device=DEV)
        self.token_seq = torch.tensor(seq, dtype=torch.int32, device=DEV)
        self.scratch = {}


class FakeCache:
    def __init__(self, block_tables, page):
        self.block_tables, self.page_size = block_tables, page


def paged_setup(lens, nkv, hd, page, dtype, seed=0, edit=None):
    """Random keys/values for requests of the given lengths, laid into shuffled pages.  Returns
    (k list, v list as float32 [len, nkv, hd]), kcache, vcache, block_tables.  ``edit(ks, vs)`` may change them
    before they are laid out."""
    g = torch.Generator().manual_seed(seed)
    ks = [torch.randn(n, nkv, hd, generator=g).to(dtype) for n in lens]
    vs = [torch.randn(n, nkv, hd, generator=g).to(dtype) for n in lens]
    if edit is not None:
        edit(ks, vs)
    blocks = [-(-n // page) for n in lens]
    total = sum(blocks) + 3
    perm = torch.randperm(total, generator=g).tolist()
    from atoma_infer_amd.cache.layout import pack_keys, pack_values
    kc = torch.randn(total, nkv, page, hd, generator=g).to(dtype)    # unused slots hold noise, not zeros
    vc = torch.randn(total, nkv, hd, page, generator=g).to(dtype)
    bt = torch.zeros(len(lens), max(blocks), dtype=torch.int32)
    nxt = 0
    for e, n in enumerate(lens):
        for b in range(blocks[e]):
            pg = perm[nxt]
            nxt += 1
            bt[e, b] = pg
            lo, hi = b * page, min((b + 1) * page, n)
            kc[pg, :, : hi - lo, :] = ks[e][lo:hi].permute(1, 0, 2)
            vc[pg, :, :, : hi - lo] = vs[e][lo:hi].permute(1, 2, 0)
    return ks, vs, pack_keys(kc).to(DEV), pack_values(vc).to(DEV), bt.to(DEV)


def plain_attention(q, k, v, start, scale, window, group):
    """q [c, nh, hd] at positions start..start+c-1 over k, v [len, nkv, hd] (float64)."""
    c, nh, hd = q.shape
    k = k.double().repeat_interleave(group, dim=1)
    v = v.double().repeat_interleave(group, dim=1)
    att = torch.einsum("qhd,khd->hqk", q.double(), k) * scale
    pos = torch.arange(start, start + c)[:, None]
    key = torch.arange(k.shape[0])[None, :]
    keep = key <= pos
    if window:
        keep &= key > pos - window
    att = att.masked_fill(~keep[None], float("-inf")).softmax(-1)
    return torch.einsum("hqk,khd->qhd", att, v)


ATTN_CASES = [
    # (nh, nkv, hd, page, window, [(start, count), ...])
    (4, 1, 16, 16, 0, [(0, 40), (0, 1), (39, 1)]),
    (3, 3, 32, 16, 0, [(0, 70), (5, 9), (64, 2)]),
    (8, 2, 64, 16, 0, [(0, 130), (600, 1), (1030, 3), (511, 1), (512, 1)]),
    (6, 2, 48, 16, 0, [(0, 33), (100, 20)]),
    (4, 4, 80, 16, 0, [(10, 50)]),
    (16, 2, 128, 16, 0, [(0, 64), (700, 1)]),
    (2, 1, 256, 16, 0, [(0, 35), (520, 2)]),
    (8, 2, 64, 16, 48, [(0, 130), (600, 1), (1030, 3), (40, 20)]),
    (4, 2, 32, 16, 600, [(0, 100), (900, 1), (640, 5)]),
    # prompt tiles with so many keys that they are cut along the keys and merged
    (8, 2, 64, 16, 0, [(0, 1100), (900, 150), (2047, 1)]),
    (4, 2, 32, 16, 800, [(0, 1300), (1200, 40)]),
    (4, 1, 128, 16, 0, [(4000, 70)]),
    # decoded tokens with so many keys that their chunks are 512 keys long
    (8, 8, 64, 16, 0, [(20000, 1), (16500, 1), (3, 2)]),
    (4, 4, 128, 16, 9000, [(17000, 1), (30000, 1), (16385, 1)]),
    # pages of 32, 64 and 48 tokens (a block of 32 keys is then one page, half a page, or lies across two): prompts,
    # portions, decoded tokens whose keys are cut into chunks, a window
    (8, 2, 64, 32, 0, [(0, 130), (600, 1), (1030, 3), (511, 1), (512, 1)]),
    (8, 2, 64, 64, 0, [(0, 1100), (900, 150), (2047, 1)]),
    (6, 2, 48, 64, 0, [(0, 33), (100, 20), (77, 1)]),
    (4, 4, 80, 48, 0, [(10, 50), (0, 97), (200, 1)]),
    (16, 2, 128, 32, 0, [(0, 64), (700, 1), (4000, 70)]),
    (4, 2, 32, 64, 600, [(0, 100), (900, 1), (640, 5)]),
    (8, 2, 64, 48, 100, [(0, 300), (1500, 1), (95, 2)]),
]


@pytest.mark.parametrize("nh,nkv,hd,page,window,entries", ATTN_CASES)
@pytest.mark.parametrize("kind", ["generic_f32", "generic_bf16", "mfma"])
def test_paged_attention(nh, nkv, hd, page, window, entries, kind):
    from atoma_infer_amd.kernels import attention_bf16, ops
    dtype = torch.float32 if kind == "generic_f32" else torch.bfloat16
    starts, counts = [s for s, _ in entries], [c for _, c in entries]
    lens = [s + c for s, c in entries]
    ks, vs, kc, vc, bt = paged_setup(lens, nkv, hd, page, dtype, seed=hd + nh)
    t = sum(counts)
    g = torch.Generator().manual_seed(1)
    qkv = (torch.randn(t, (nh + 2 * nkv) * hd, generator=g) * 1.5).to(dtype).to(DEV)   # q lives inside a wider row
    out = torch.empty(t, nh * hd, dtype=dtype, device=DEV)
    ctx, cache = FakeCtx(starts, counts), FakeCache(bt, page)
    scale = 1.0 / math.sqrt(hd)
    if kind == "mfma":
        assert attention_bf16.try_attention(qkv, kc, vc, out, ctx, cache, scale, window, nh, nkv, hd)
        assert attention_bf16.lib(hd, page=page).atoma_attention_mfma_page_size() == page
    else:
        ops.paged_attention_generic(qkv, kc, vc, out, bt, ctx.token_seq, ctx.positions, scale, window, page, nh,
                                    nkv, hd)
    row = 0
    for e, (s, c) in enumerate(entries):
        q = qkv[row:row + c, : nh * hd].cpu().view(c, nh, hd)
        want = plain_attention(q, ks[e], vs[e], s, scale, window, nh // nkv).reshape(c, nh * hd)
        got = out[row:row + c].double().cpu()
        tol = 2e-5 if dtype is torch.float32 else 2e-2
        err = (got - want).abs().max() / want.abs().max()
        assert err < tol, f"entry {e} ({s}, {c}): {err:.3e}"
        row += c


TWO_PIECE_CASES = [c for c in ATTN_CASES if c[2] <= 64] + [
    # groups of 1, 3, 8, 33 and 40 heads (tiles of 256, 255, 256, 264, 240 rows; the last pieces are short or half
    # empty), one token, a window, portions beside decoded tokens
    (5, 5, 64, 16, 0, [(0, 300), (700, 1)]),
    (3, 1, 16, 16, 0, [(0, 100), (50, 86), (3, 1)]),
    (16, 2, 64, 16, 0, [(100, 75), (2100, 33), (0, 7)]),
    (33, 1, 32, 16, 0, [(0, 20), (40, 9)]),
    (40, 1, 64, 16, 70, [(0, 130), (300, 2)]),
]


@pytest.mark.parametrize("nh,nkv,hd,page,window,entries", TWO_PIECE_CASES)
def test_attention_with_two_pieces_of_rows_a_wave(nh, nkv, hd, page, window, entries, monkeypatch):
    """Prompt tiles that walk many keys give every wave two pieces of 32 rows against the same keys.  Here the
    threshold is taken away, so that every step with a prompt tile runs that way."""
    from atoma_infer_amd.kernels import attention_bf16
    monkeypatch.setattr(attention_bf16, "TWO_PIECES_MIN_KEYS", 0)
    starts, counts = [s for s, _ in entries], [c for _, c in entries]
    ks, vs, kc, vc, bt = paged_setup([s + c for s, c in entries], nkv, hd, page, torch.bfloat16, seed=hd + nh)
    t = sum(counts)
    g = torch.Generator().manual_seed(1)
    qkv = (torch.randn(t, (nh + 2 * nkv) * hd, generator=g) * 1.5).bfloat16().to(DEV)
    out = torch.full((t, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ctx, cache = FakeCtx(starts, counts), FakeCache(bt, page)
    scale = 1.0 / math.sqrt(hd)
    assert attention_bf16.try_attention(qkv, kc, vc, out, ctx, cache, scale, window, nh, nkv, hd)
    plan = [v for k, v in ctx.scratch.items() if k[0] == "attention_tasks_adhoc"][0]
    assert plan[1][4] == 2, "the step was meant to run with two pieces a wave"
    row = 0
    for e, (s0, c) in enumerate(entries):
        q = qkv[row:row + c, : nh * hd].cpu().view(c, nh, hd)
        want = plain_attention(q, ks[e], vs[e], s0, scale, window, nh // nkv).reshape(c, nh * hd)
        err = (out[row:row + c].double().cpu() - want).abs().max() / want.abs().max()
        assert err < 2e-2, f"entry {e} ({s0}, {c}): {err:.3e}"
        row += c


HEADS_AND_SIZES = [(6, 2, hd) for hd in range(16, 257, 16)] + [
    # groups of 1, 7, 32, 33 and 40 heads to a KV head (more than 32 take several pieces of rows), many KV heads
    (5, 5, 64), (7, 1, 32), (64, 2, 64), (33, 1, 32), (40, 1, 64), (80, 2, 16), (24, 24, 48), (9, 3, 128)]


@pytest.mark.parametrize("nh,nkv,hd", HEADS_AND_SIZES)
def test_attention_at_every_head_size_and_grouping(nh, nkv, hd):
    """Every multiple of 16 up to 256, and groups of any size: a prompt of several tiles, a portion behind a
    prefix, and decoded tokens whose keys are cut into chunks and merged."""
    from atoma_infer_amd.kernels import attention_bf16
    page = 16
    entries = [(0, 70), (300, 9), (700, 1), (129, 1), (15, 1)]
    starts, counts = [s for s, _ in entries], [c for _, c in entries]
    ks, vs, kc, vc, bt = paged_setup([s + c for s, c in entries], nkv, hd, page, torch.bfloat16, seed=hd)
    t = sum(counts)
    g = torch.Generator().manual_seed(hd)
    qkv = (torch.randn(t, (nh + 2 * nkv) * hd, generator=g) * 1.5).bfloat16().to(DEV)
    out = torch.full((t, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    scale = 1.0 / math.sqrt(hd)
    assert attention_bf16.try_attention(qkv, kc, vc, out, FakeCtx(starts, counts), FakeCache(bt, page), scale, 0,
                                        nh, nkv, hd)
    row = 0
    for e, (s, c) in enumerate(entries):
        q = qkv[row:row + c, : nh * hd].cpu().view(c, nh, hd)
        want = plain_attention(q, ks[e], vs[e], s, scale, 0, nh // nkv).reshape(c, nh * hd)
        got = out[row:row + c].double().cpu()
        err = (got - want).abs().max() / want.abs().max()
        assert err < 2e-2, f"head size {hd}, entry {e} ({s}, {c}): {err:.3e}"
        row += c


STAND_OUT = [
    # (window, [(start, count)], key that gets the large score)
    (0, [(699, 1)], 0), (0, [(699, 1)], 15), (0, [(699, 1)], 16), (0, [(699, 1)], 127), (0, [(699, 1)], 128),
    (0, [(699, 1)], 255), (0, [(699, 1)], 256), (0, [(699, 1)], 511), (0, [(699, 1)], 512), (0, [(699, 1)], 698),
    (0, [(699, 1)], 699),
    (100, [(699, 1)], 599),      # just outside the window: must not be seen
    (100, [(699, 1)], 600),      # the window's first key
    (0, [(480, 40)], 479), (0, [(480, 40)], 500), (0, [(480, 40)], 519),      # a portion: all rows, some rows, one row
    (64, [(480, 40)], 440), (64, [(480, 40)], 456),      # a window's edge that moves through the portion's rows
    (0, [(0, 300)], 0), (0, [(0, 300)], 31), (0, [(0, 300)], 32), (0, [(0, 300)], 287),
]


@pytest.mark.parametrize("window,entries,key", STAND_OUT)
@pytest.mark.parametrize("kind", ["generic_f32", "generic_bf16", "mfma"])
def test_attention_when_one_key_stands_out(window, entries, key, kind):
    """Among hundreds of random keys a wrong one changes the result by less than the tolerance.  Here every query
    points at one key, whose weight is then nearly one wherever the row may see it: a fault at a page's edge, at
    a chunk's border, at the window's edge or in the causal mask shows as a wrong row."""
    from atoma_infer_amd.kernels import attention_bf16, ops
    nh, nkv, hd, page = 4, 2, 64, 16
    dtype = torch.float32 if kind == "generic_f32" else torch.bfloat16
    starts, counts = [s for s, _ in entries], [c for _, c in entries]
    lens = [s + c for s, c in entries]
    ks, vs, kc, vc, bt = paged_setup(lens, nkv, hd, page, dtype, seed=key + 1)
    t = sum(counts)
    # every head's query is three times its KV head's key at `key`: that score is about 24, the others' about 3
    q = (3.0 * ks[0][key].float()).repeat_interleave(nh // nkv, dim=0)        # [nh, hd]
    qkv = torch.zeros(t, (nh + 2 * nkv) * hd)
    qkv[:, : nh * hd] = q.reshape(1, nh * hd)
    qkv = qkv.to(dtype).to(DEV)
    out = torch.empty(t, nh * hd, dtype=dtype, device=DEV)
    ctx, cache = FakeCtx(starts, counts), FakeCache(bt, page)
    scale = 1.0 / math.sqrt(hd)
    if kind == "mfma":
        assert attention_bf16.try_attention(qkv, kc, vc, out, ctx, cache, scale, window, nh, nkv, hd)
        assert attention_bf16.lib(hd, page=page).atoma_attention_mfma_page_size() == page
    else:
        ops.paged_attention_generic(qkv, kc, vc, out, bt, ctx.token_seq, ctx.positions, scale, window, page, nh,
                                    nkv, hd)
    (s0, c0) = entries[0]
    qq = qkv[:, : nh * hd].cpu().view(c0, nh, hd)
    want = plain_attention(qq, ks[0], vs[0], s0, scale, window, nh // nkv).reshape(c0, nh * hd)
    got = out.double().cpu()
    tol = 2e-5 if dtype is torch.float32 else 2e-2
    for r in range(c0):
        err = (got[r] - want[r]).abs().max() / want[r].abs().max()
        assert err < tol, f"row at position {s0 + r}: {err:.3e}"
    # the test means what it says: rows that may see the key return its value, nearly
    p = torch.arange(s0, s0 + c0)
    sees = (key <= p) & ((key > p - window) if window else torch.ones_like(p, dtype=torch.bool))
    vj = vs[0][key].double().repeat_interleave(nh // nkv, dim=0).reshape(nh * hd)
    for r in range(c0):
        close = (want[r] - vj).abs().max() < 0.05
        assert bool(close) == bool(sees[r]), (r, float((want[r] - vj).abs().max()))


def test_attention_reference_vectors():
    """The reference's own golden values: csrc/tests/flash_attn_tests.rs:31-93 (no mask, as a one-token decode of the
    second row is not what they test, the unmasked case is rebuilt as two single-key requests...) and the causal
    ones of models/src/flash_attention.rs:632-705: q = arange(48)/30, k = /40, v = /50 shaped (3 heads, 2 tokens,
    8), scale 0.5; row 0 of every head equals v[0]."""
    from atoma_infer_amd.kernels import ops
    base = torch.arange(48, dtype=torch.float32).reshape(3, 2, 8).half().float()
    q, k, v = (base / 30).half().float(), (base / 40).half().float(), (base / 50).half().float()
    causal = torch.tensor([
        [[0.0, 0.02, 0.04, 0.06, 0.08, 0.1, 0.12, 0.14],
         [0.0922, 0.1122, 0.1322, 0.1522, 0.1721, 0.1921, 0.2122, 0.2322]],
        [[0.3201, 0.3401, 0.3601, 0.3801, 0.4001, 0.4202, 0.4402, 0.4602],
         [0.428, 0.448, 0.468, 0.488, 0.5083, 0.5283, 0.5483, 0.5684]],
        [[0.6401, 0.6602, 0.6802, 0.7002, 0.7202, 0.7402, 0.7603, 0.7803],
         [0.7622, 0.7822, 0.8022, 0.8223, 0.8423, 0.8623, 0.8823, 0.9023]]])
    # head size 8 is below what the kernels take: embed each head into 16 columns, the upper 8 zero
    hd, nh, page = 16, 3, 16
    qq = torch.zeros(2, nh, hd)
    qq[:, :, :8] = q.permute(1, 0, 2)
    kc = torch.zeros(1, nh, page, hd)
    vc = torch.zeros(1, nh, hd, page)
    kc[0, :, :2, :8] = k
    vc[0, :, :8, :2] = v.permute(0, 2, 1)
    from atoma_infer_amd.cache.layout import pack_keys, pack_values
    kc, vc = pack_keys(kc), pack_values(vc)
    out = torch.empty(2, nh * hd, device=DEV)
    bt = torch.zeros(1, 1, dtype=torch.int32, device=DEV)
    ctx = FakeCtx([0], [2])
    ops.paged_attention_generic(qq.reshape(2, nh * hd).to(DEV), kc.to(DEV), vc.to(DEV), out, bt, ctx.token_seq,
                                ctx.positions, 0.5, 0, page, nh, nh, hd)
    got = out.cpu().view(2, nh, hd)[:, :, :8].permute(1, 0, 2)
    # the goldens were computed in float16 and rounded to 4 places
    assert (got - causal).abs().max() < 1.5e-3
    assert torch.allclose(got[:, 0], v[:, 0], atol=1e-6)


@pytest.mark.parametrize("nh,nkv,hd,page", [(5, 2, 48, 4), (8, 2, 64, 16), (3, 1, 40, 16), (2, 2, 128, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t", [9, 45])      # few tokens and many take different kernels in bfloat16
@pytest.mark.parametrize("paired", [False, True])
def test_rope_cache_write(dtype, nh, nkv, hd, page, t, paired):
    """``paired``: the members of pair i arrive as columns 2i and 2i + 1 and the rotated q leaves to a buffer of its
    own: the same rows in pair order must give the plain result, in the plain order."""
    from atoma_infer_amd.kernels import ops
    order = torch.stack([torch.arange(hd // 2), torch.arange(hd // 2) + hd // 2], dim=1).reshape(-1)
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(t, (nh + 2 * nkv) * hd, generator=g).to(dtype)
    pos = torch.tensor(([0, 1, 2, 3, 4, 50, 51, 7, 8] * 5)[:t], dtype=torch.int32)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2).float() / hd))
    ang = torch.arange(64).float()[:, None] * inv[None]
    cos, sin = torch.cos(ang), torch.sin(ang)
    # slots in pages 0, 2 and 7 whatever the page size; pages 3..6 must stay untouched
    slots = torch.tensor([2 * page, 2 * page + 1, 2 * page + 2, 2 * page + 3, 0, 1, -1, 8 * page - 2, 8 * page - 1]
                         + [-1] * (t - 9), dtype=torch.int32)
    kc = torch.zeros(8, nkv, page, hd, dtype=dtype)
    vc = torch.zeros(8, nkv, hd, page, dtype=dtype)
    from atoma_infer_amd.cache.layout import pack_keys, pack_values, unpack_keys, unpack_values
    x_in = qkv.view(t, nh + 2 * nkv, hd).clone()
    if paired:
        x_in[:, :nh + nkv] = x_in[:, :nh + nkv][:, :, order]        # q and k heads in pair order, v as it is
    d_qkv, d_kc, d_vc = x_in.reshape(t, -1).to(DEV), pack_keys(kc).to(DEV), pack_values(vc).to(DEV)
    q_out = torch.empty(t, nh * hd, dtype=dtype, device=DEV) if paired else None
    before = d_qkv.clone()
    ops.rope_cache_write(d_qkv, pos.to(DEV), cos.to(DEV), sin.to(DEV), hd, d_kc, d_vc, slots.to(DEV), page, nh, nkv, hd,
                         q_out)
    d_kc, d_vc = unpack_keys(d_kc, page, hd), unpack_values(d_vc, page, hd)
    if paired:       # the rotated q is in q_out, in its own column order; the input is left alone
        assert torch.equal(d_qkv, before)
        d_qkv = torch.cat([q_out, d_qkv[:, nh * hd:]], dim=1)
    x = qkv.float().view(t, nh + 2 * nkv, hd)
    c, s = cos[pos.long()][:, None, :], sin[pos.long()][:, None, :]
    x1, x2 = x[..., : hd // 2], x[..., hd // 2:]
    rot = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1)
    tol = 1e-6 if dtype is torch.float32 else 1e-2
    got = d_qkv.float().cpu().view(t, nh + 2 * nkv, hd)
    assert torch.allclose(got[:, :nh], rot[:, :nh], atol=tol, rtol=tol)
    assert torch.equal(got[:, nh + nkv:], x[:, nh + nkv:])          # v untouched in place
    for i in range(t):
        sl = int(slots[i])
        if sl < 0:
            continue
        assert torch.allclose(d_kc.float().cpu()[sl // page, :, sl % page, :], rot[i, nh:nh + nkv], atol=tol, rtol=tol)
        assert torch.equal(d_vc.cpu()[sl // page, :, :, sl % page].float(), x[i, nh + nkv:].to(dtype).float())
    # slot -1 wrote nothing: pages 2..6 stay zero
    assert torch.count_nonzero(d_kc[3:7]) == 0 and torch.count_nonzero(d_vc[3:7]) == 0
    # position 0 is the identity
    assert torch.allclose(got[0, :nh], x[0, :nh], atol=tol)


def interleave16(g, u):
    """Rows of gate and up in blocks of 16: 16 gate rows, then the 16 up rows of the same outputs."""
    i, w = g.shape
    return torch.stack([g.view(i // 16, 16, w), u.view(i // 16, 16, w)], dim=1).reshape(2 * i, w).contiguous()


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_swiglu_interleaved_layout(dt):
    from atoma_infer_amd.kernels import ops
    inter = 48
    g, u = rnd(5, inter, dtype=dt, seed=1, scale=2.0), rnd(5, inter, dtype=dt, seed=2, scale=2.0)
    gu = interleave16(g.t().contiguous(), u.t().contiguous()).t().contiguous()      # columns interleaved
    out = ops.swiglu(gu, block=16)
    want = torch.nn.functional.silu(g.float()) * u.float()
    tol = 1e-6 if dt is torch.float32 else 2e-2
    assert torch.allclose(out.float(), want, rtol=tol, atol=tol)


@pytest.mark.parametrize("m", [1, 8, 17, 32, 50, 64])
@pytest.mark.parametrize("inter,k", [(16, 32), (160, 64), (8192, 2048), (1024, 96), (8208, 256)])
def test_gemm_with_swiglu_epilogue(m, inter, k):
    from atoma_infer_amd.kernels import gemm_bf16
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    wg, wu = rnd(inter, k, dtype=torch.bfloat16, seed=2, scale=0.1), rnd(inter, k, dtype=torch.bfloat16, seed=3, scale=0.1)
    out = gemm_bf16.try_linear_swiglu(x, interleave16(wg, wu))
    assert out is not None and tuple(out.shape) == (m, inter)
    g, u = x.double().cpu() @ wg.double().cpu().T, x.double().cpu() @ wu.double().cpu().T
    want = torch.nn.functional.silu(g) * u
    assert (out.double().cpu() - want).abs().max() <= 1e-2 * want.abs().max()
    assert gemm_bf16.try_linear_swiglu(rnd(70, k, dtype=torch.bfloat16), interleave16(wg, wu)) is None   # too many rows


@pytest.mark.parametrize("m", [1, 8, 16, 23, 40, 64])
@pytest.mark.parametrize("nh,nkv,hd,k", [(8, 2, 64, 256), (3, 1, 16, 64), (32, 8, 64, 2048), (5, 5, 48, 96),
                                         (24, 8, 128, 256), (32, 8, 128, 512), (3, 1, 128, 384)])
@pytest.mark.parametrize("planes", [False, True])
def test_gemm_with_rotary_epilogue(m, nh, nkv, hd, k, planes, monkeypatch):
    """The q, k, v projection that rotates and stores in its epilogue (or, with ``planes`` and more than 16 rows, as
    a K-split product whose planes a second kernel sums, rotates and stores, as the planner has it from 41 rows on)
    against product, rotation and store done apart."""
    from atoma_infer_amd.kernels import gemm_bf16, ops
    if planes:
        if m <= 16:
            pytest.skip("one tile of rows: the epilogue always")
        monkeypatch.setattr(gemm_bf16, "ROPE_PLANES_MIN_M", 16)
    else:
        monkeypatch.setattr(gemm_bf16, "ROPE_PLANES_MIN_M", 64)
    from atoma_infer_amd.cache.layout import pack_keys, pack_values
    page, pages = 16, 6
    n = (nh + 2 * nkv) * hd
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)   # (96 slots: enough for 64 rows)
    w = rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.2)
    g = torch.Generator().manual_seed(5)
    pos = torch.randint(0, 90, (m,), generator=g).int().to(DEV)
    slots = torch.randperm(pages * page, generator=g)[:m].int()
    if m > 2:
        slots[2] = -1
    slots = slots.to(DEV)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2).float() / hd))
    ang = torch.arange(96).float()[:, None] * inv[None]
    cos, sin = torch.cos(ang).to(DEV), torch.sin(ang).to(DEV)

    def caches():
        gg = torch.Generator().manual_seed(9)
        return (pack_keys(torch.randn(pages, nkv, page, hd, generator=gg).bfloat16()).to(DEV),
                pack_values(torch.randn(pages, nkv, hd, page, generator=gg).bfloat16()).to(DEV))
    kc1, vc1 = caches()
    q1 = gemm_bf16.try_linear_rope(x, w, pos, cos, sin, kc1, vc1, slots, page, nh, nkv, hd, always=True)
    assert q1 is not None and tuple(q1.shape) == (m, nh * hd)
    # over the copy of the weight in the order the kernel's waves read it: the same bits
    tw = gemm_bf16.tile_copies_rope(w)
    assert (tw is not None and tw.few is not None) == (k % 512 == 0 and n % 16 == 0)
    tiled_runs = tw is not None and ((tw.few is not None and (m <= 8 or (m <= 16 and n < 5120)))
                                     or (tw.many is not None and planes))
    if tiled_runs:
        kc3, vc3 = caches()
        with monkeypatch.context() as mp:
            def row_major(*a):
                raise AssertionError("the row-major kernel ran")
            mp.setattr(gemm_bf16.lib(), "atoma_gemm_bf16_skinny_rope", row_major)
            mp.setattr(gemm_bf16.lib(), "atoma_gemm_bf16_skinny", row_major)
            q3 = gemm_bf16.try_linear_rope(x, w, pos, cos, sin, kc3, vc3, slots, page, nh, nkv, hd, always=True, tiled=tw)
        assert torch.equal(q3, q1) and torch.equal(kc3, kc1) and torch.equal(vc3, vc1)
    # apart, with float32 in between (the fused kernel rotates the float32 sums)
    kc2, vc2 = caches()
    qkv = ops.gemm_generic(x, w, torch.float32)
    kc2f, vc2f = kc2.float(), vc2.float()
    q2 = torch.empty(m, nh * hd, dtype=torch.float32, device=DEV)
    ops.rope_cache_write(qkv, pos, cos, sin, hd, kc2f, vc2f, slots, page, nh, nkv, hd, q2)
    tol = 1e-2
    assert (q1.float() - q2).abs().max() <= tol * q2.abs().max()
    assert (kc1.float() - kc2f).abs().max() <= tol * kc2f.abs().max()
    assert (vc1.float() - vc2f).abs().max() <= tol * vc2f.abs().max()
    # the row without a slot wrote nothing, and untouched slots keep what they held
    kc0, vc0 = caches()
    same = (kc1 == kc0)
    assert int((~same).sum()) <= (m - (1 if m > 2 else 0)) * nkv * hd
    assert gemm_bf16.try_linear_rope(rnd(70, k, dtype=torch.bfloat16), w, pos, cos, sin, kc1, vc1, slots, page, nh, nkv,
                                     hd) is None   # too many rows


def _rms(x, g, eps):
    x = x.double()
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * g.double()


@pytest.mark.parametrize("m", [1, 5, 8, 16])
@pytest.mark.parametrize("n,k", [(2048, 2048), (2048, 8192), (96, 64), (200, 96), (3072, 512), (3072, 1024), (4096, 2048)])
@pytest.mark.parametrize("gdt", [torch.float32, torch.bfloat16])
def test_product_into_the_residual_begins_the_norm(m, n, k, gdt):
    """``resid += x w^T`` with the following RMSNorm begun in the product's epilogue (residual times norm weight and
    the rows' sums of squares in shares), against the product, the sum and the norm done apart in float64; then the
    begun norm finished as a tensor, and finished inside plain, SiLU-multiply and rotary products."""
    from atoma_infer_amd.kernels import gemm_bf16
    eps = 1e-5
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    resid0 = rnd(m, n, dtype=torch.float32, seed=3)
    gamma = (1 + 0.1 * rnd(n, dtype=torch.float32, seed=4)).to(gdt)
    resid = resid0.clone()
    b = gemm_bf16.try_linear_resid(x, w, resid, gamma, eps)
    assert b is not None and b.shares.shape[1] == 16
    want_resid = resid0.double().cpu() + x.double().cpu() @ w.double().cpu().T
    assert (resid.double().cpu() - want_resid).abs().max() <= 1e-5 * want_resid.abs().max()
    want_u = want_resid * gamma.double().cpu()
    assert (b.data.double().cpu() - want_u).abs().max() <= 1e-2 * want_u.abs().max()
    ss = b.shares.double().cpu().sum(0)
    assert torch.allclose(ss[:m], want_resid.pow(2).sum(-1), rtol=1e-5)
    assert float(ss[m:].abs().sum()) == 0.0
    want_normed = _rms(want_resid, gamma.cpu(), eps)
    got = b.tensor()
    assert got.dtype is torch.bfloat16
    assert (got.double().cpu() - want_normed).abs().max() <= 1.2e-2 * want_normed.abs().max()
    # finished inside the products that read it: float32 sums of the normed rows
    w2 = rnd(72, n, dtype=torch.bfloat16, seed=5)
    if n % 32 == 0:
        y = gemm_bf16.try_linear(b, w2, torch.float32)
        exact = b.data.double().cpu() / torch.sqrt(want_resid.pow(2).mean(-1, keepdim=True) + eps)   # same bf16 rows
        want_y = exact @ w2.double().cpu().T
        assert (y.double().cpu() - want_y).abs().max() <= 1e-5 * want_y.abs().max()
        # a second product into the residual whose rows are the begun norm
        resid2 = resid.clone()
        b2 = gemm_bf16.try_linear_resid(b, rnd(n, n, dtype=torch.bfloat16, seed=6, scale=0.05), resid2, gamma, eps)
        want2 = resid.double().cpu() + exact @ rnd(n, n, dtype=torch.bfloat16, seed=6, scale=0.05).double().cpu().T
        assert (resid2.double().cpu() - want2).abs().max() <= 1e-5 * want2.abs().max()
        assert torch.allclose(b2.shares.double().cpu().sum(0)[:m], want2.pow(2).sum(-1), rtol=1e-5)


@pytest.mark.parametrize("m", [1, 8, 13])
def test_begun_norms_are_finished_by_the_fused_products(m):
    from atoma_infer_amd.kernels import gemm_bf16, ops
    from atoma_infer_amd.cache.layout import pack_keys, pack_values
    eps, width = 1e-6, 256
    table = rnd(50, width, dtype=torch.bfloat16, seed=1)
    gamma = (1 + 0.1 * rnd(width, dtype=torch.float32, seed=2)).bfloat16()
    tokens = torch.randint(0, 50, (m,), generator=torch.Generator().manual_seed(3)).int().to(DEV)
    resid, u, ss = ops.embed_begin_norm(tokens, table, gamma)
    rows = table[tokens.long()].double().cpu()
    assert torch.equal(resid.cpu(), rows.float())
    assert torch.allclose(ss.double().cpu()[0, :m], rows.pow(2).sum(-1), rtol=1e-6)
    b = gemm_bf16.Begun(u, ss, eps, width)
    normed = b.tensor()                      # bfloat16 rows of the finished norm
    want = _rms(rows, gamma.cpu(), eps)
    assert (normed.double().cpu() - want).abs().max() <= 1.2e-2 * want.abs().max()
    exact = u.double().cpu() / torch.sqrt(rows.pow(2).mean(-1, keepdim=True) + eps)
    # SiLU-multiply epilogue
    inter = 160
    wg, wu = rnd(inter, width, dtype=torch.bfloat16, seed=4, scale=0.1), rnd(inter, width, dtype=torch.bfloat16, seed=5, scale=0.1)
    out = gemm_bf16.try_linear_swiglu(b, interleave16(wg, wu))
    g, up = exact @ wg.double().cpu().T, exact @ wu.double().cpu().T
    want = torch.nn.functional.silu(g) * up
    assert (out.double().cpu() - want).abs().max() <= 1e-2 * want.abs().max()
    # rotary epilogue with the cache write
    nh, nkv, hd, page, pages = 4, 2, 32, 16, 4
    w = rnd((nh + 2 * nkv) * hd, width, dtype=torch.bfloat16, seed=6, scale=0.2)
    gen = torch.Generator().manual_seed(7)
    pos = torch.randint(0, 60, (m,), generator=gen).int().to(DEV)
    slots = torch.randperm(pages * page, generator=gen)[:m].int().to(DEV)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2).float() / hd))
    ang = torch.arange(64).float()[:, None] * inv[None]
    cos, sin = torch.cos(ang).to(DEV), torch.sin(ang).to(DEV)

    def caches():
        gg = torch.Generator().manual_seed(9)
        return (pack_keys(torch.randn(pages, nkv, page, hd, generator=gg).bfloat16()).to(DEV),
                pack_values(torch.randn(pages, nkv, hd, page, generator=gg).bfloat16()).to(DEV))
    kc1, vc1 = caches()
    q1 = gemm_bf16.try_linear_rope(b, w, pos, cos, sin, kc1, vc1, slots, page, nh, nkv, hd, always=True)
    kc2, vc2 = caches()
    qkv = (exact @ w.double().cpu().T).float().to(DEV)
    kc2f, vc2f = kc2.float(), vc2.float()
    q2 = torch.empty(m, nh * hd, dtype=torch.float32, device=DEV)
    ops.rope_cache_write(qkv, pos, cos, sin, hd, kc2f, vc2f, slots, page, nh, nkv, hd, q2)
    assert (q1.float() - q2).abs().max() <= 1e-2 * q2.abs().max()
    assert (kc1.float() - kc2f).abs().max() <= 1e-2 * kc2f.abs().max()
    assert (vc1.float() - vc2f).abs().max() <= 1e-2 * vc2f.abs().max()


@pytest.mark.parametrize("m,n,k,cdt", [(40, 2048, 8192, torch.bfloat16), (64, 16384, 2048, torch.bfloat16),
                                       (48, 40000, 2048, torch.float32), (64, 3072, 2048, torch.bfloat16)])
def test_products_replay_in_graphs(m, n, k, cdt):
    """Decode steps of large batches are captured in HIP graphs together with the library's products.  A captured
    product must give, on every replay, what an eager call gives for the operand's current content, also with
    eager work and synchronisations between the replays."""
    from atoma_infer_amd.kernels import gemm_bf16
    w = rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    gemm_bf16.try_linear(x, w, cdt)                       # loads every kernel before capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = gemm_bf16.try_linear(x, w, cdt)
    other = rnd(512, 512, dtype=torch.bfloat16, seed=3)
    for i in range(6):
        x.copy_(rnd(m, k, dtype=torch.bfloat16, seed=10 + i))
        graph.replay()
        got = y.clone()
        want = gemm_bf16.try_linear(x, w, cdt)            # eager, between replays
        assert torch.equal(got, want), f"replay {i}"
        (other @ other).sum().item()                      # more eager work and a synchronisation
        if i == 3:
            torch.cuda.synchronize()


@pytest.mark.parametrize("more", [30, 8])      # 320 and 144 workgroups: more and fewer than the GPU has CUs
@pytest.mark.parametrize("window", [0, 200])
def test_attention_whole_ranges_with_eight_waves(window, more):
    """A decode step of many requests: every (request, KV head) pair is one task whose keys eight waves share and
    merge in LDS.  Lengths from one key to a few thousand, so that waves with nothing to do sit beside full ones."""
    from atoma_infer_amd.kernels import attention_bf16 as A
    nh, nkv, hd, page = 32, 8, 64, 16
    g = torch.Generator().manual_seed(7)
    starts = [0, 1, 30, 31, 32, 255, 256, 257, 511, 1000] + torch.randint(0, 2300, (more,), generator=g).tolist()
    counts = [1] * len(starts)
    lens = [s + 1 for s in starts]
    ks, vs, kc, vc, bt = paged_setup(lens, nkv, hd, page, torch.bfloat16, seed=3)
    q = (torch.randn(len(starts), (nh + 2 * nkv) * hd, generator=g) * 1.5).bfloat16().to(DEV)
    out = torch.empty(len(starts), nh * hd, dtype=torch.bfloat16, device=DEV)
    ctx, cache = FakeCtx(starts, counts), FakeCache(bt, page)
    bucket = -(-max(lens) // 256) * 256
    arr, meta = A.build_tasks(ctx.h_starts, ctx.h_counts, nh // nkv, window, bucket, kv_heads=nkv, max_waves=8)
    assert meta[1:] == (0, 0, 8, 1, False)
    ctx.plans = {A.plan_key(nh // nkv, window, nkv, hd): (torch.from_numpy(arr).to(DEV), meta)}
    scale = 1.0 / math.sqrt(hd)
    assert A.try_attention(q, kc, vc, out, ctx, cache, scale, window, nh, nkv, hd)
    for e, s in enumerate(starts):
        qq = q[e:e + 1, : nh * hd].cpu().view(1, nh, hd)
        want = plain_attention(qq, ks[e], vs[e], s, scale, window, nh // nkv).reshape(nh * hd)
        err = (out[e].double().cpu() - want).abs().max() / want.abs().max()
        assert err < 2e-2, f"request {e} of length {s + 1}: {err:.3e}"


def test_tokens_outside_the_table_and_rows_of_nan_do_no_harm():
    """A sampled token reaches the next step without passing the host: the embedding checks it, and the sampler
    names a token of the vocabulary whatever its logits hold."""
    from atoma_infer_amd.kernels import ops
    table = rnd(50, 24, dtype=torch.bfloat16, seed=1)
    toks = torch.tensor([3, 50, -1, 2 ** 31 - 1, 49], dtype=torch.int32, device=DEV)
    out = ops.embed(toks, table)
    assert torch.equal(out[0], table[3].float()) and torch.equal(out[4], table[49].float())
    assert bool(torch.isnan(out[1:4]).all())
    logits = torch.randn(4, 1000, generator=torch.Generator().manual_seed(0)).to(DEV)
    logits[1] = float("nan")
    logits[2, 100:200] = float("nan")
    logits[3] = float("-inf")
    dev = lambda x, dt: torch.tensor(x, dtype=dt, device=DEV)
    for temp, k, p in ((0.0, 0, 1.0), (0.8, 0, 1.0), (0.8, 20, 0.9)):
        tok, _ = ops.sample(logits, dev([temp] * 4, torch.float32), dev([k] * 4, torch.int32),
                            dev([p] * 4, torch.float32), dev([0.3] * 4, torch.float32))
        tok = tok.cpu().tolist()
        assert all(0 <= t < 1000 for t in tok), tok
        if temp == 0.0:
            assert tok[0] == int(torch.argmax(logits[0])) and tok[3] == 0


PLANS = ["chunks", "chunks, second kernel", "whole"]


@pytest.mark.parametrize("plan", PLANS)
@pytest.mark.parametrize("nh,nkv,hd", [(40, 1, 64), (33, 1, 32), (6, 2, 112), (64, 2, 64), (3, 3, 208)])
def test_decode_plans_with_large_groups(nh, nkv, hd, plan, monkeypatch):
    """The task lists of decode steps as the engine builds them (every request owns its bucket's chunk slots), for
    groups of more than 32 heads, which take several pieces of rows: chunks merged by the wave that finishes the last
    one or by the second kernel, and whole key ranges walked by eight waves."""
    import numpy as np
    from atoma_infer_amd.kernels import attention_bf16
    whole = plan == "whole"
    if whole:
        if attention_bf16.max_waves_for(hd) < 8:
            pytest.skip("eight waves a task do not fit this head size")
        monkeypatch.setattr(attention_bf16, "WHOLE_MIN_PAIRS", 2)
    else:
        force_chunked_decode(monkeypatch, second_kernel=plan.endswith("second kernel"))
    group, page = nh // nkv, 16
    starts = [700, 129, 15, 256, 511]
    counts = [1] * len(starts)
    ks, vs, kc, vc, bt = paged_setup([s + 1 for s in starts], nkv, hd, page, torch.bfloat16, seed=hd + nh)
    t = len(starts)
    g = torch.Generator().manual_seed(3)
    qkv = (torch.randn(t, (nh + 2 * nkv) * hd, generator=g) * 1.5).bfloat16().to(DEV)
    out = torch.full((t, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ctx = FakeCtx(starts, counts)
    arr, meta = attention_bf16.build_tasks(np.asarray(starts, dtype=np.int32), np.asarray(counts, dtype=np.int32),
                                           group, 0, 3 * 256, kv_heads=nkv, max_waves=attention_bf16.max_waves_for(hd))
    assert (meta[1] == 0) == whole                       # no merge records with whole ranges
    assert meta[5] == (plan == "chunks")
    ctx.plans = {attention_bf16.plan_key(group, 0, nkv, hd): (torch.from_numpy(arr).to(DEV), meta)}
    scale = 1.0 / math.sqrt(hd)
    # the block tables of a bucket of three cover 768 keys
    wide = torch.zeros((t, 3 * 256 // page), dtype=torch.int32, device=DEV)
    wide[:, : bt.shape[1]] = bt
    assert attention_bf16.try_attention(qkv, kc, vc, out, ctx, FakeCache(wide, page), scale, 0, nh, nkv, hd)
    for e, s in enumerate(starts):
        q = qkv[e:e + 1, : nh * hd].cpu().view(1, nh, hd)
        want = plain_attention(q, ks[e], vs[e], s, scale, 0, group).reshape(1, nh * hd)
        err = (out[e:e + 1].double().cpu() - want).abs().max() / want.abs().max()
        assert err < 2e-2, f"request {e} at {s}: {err:.3e}"


@pytest.mark.parametrize("nh,nkv,hd,starts,chunk,window", [
    (32, 8, 64, [20000], 512, 0),                   # 40 parts for one wave to merge, in rounds
    (32, 8, 64, [5000, 0, 4999, 2303, 17], 1024, 0),
    (8, 2, 128, [9000, 8000, 1], 256, 0),
    (16, 8, 64, [3000] * 7 + [8191], 2048, 0),      # four parts, of which most requests fill two
    (32, 8, 64, [9000, 3100, 2999, 40], 512, 3000), # a window of 3,000 keys wherever it lies: its chunks' slots
    (32, 8, 64, [30000] * 6 + [7], 1024, 5000),
])
def test_decode_chunks_that_grow_with_the_context(nh, nkv, hd, starts, chunk, window):
    """Decode steps beyond the contexts of a few thousand keys: four waves a chunk, chunks the longer the more there
    are, and the wave that finishes a row piece's last chunk merges all of its parts, however many.  One key far
    from the decoded token is made to stand out in the first request, so that a part lost in the merge shows."""
    import numpy as np
    from atoma_infer_amd.kernels import attention_bf16
    group, page = nh // nkv, 16
    counts = [1] * len(starts)
    far = min(37, starts[0]) if not window else starts[0] - window + 2       # (the second key the window shows)

    def edit(ks, vs):
        ks[0][far] *= 3.0
    ks, vs, kc, vc, bt = paged_setup([s + 1 for s in starts], nkv, hd, page, torch.bfloat16, seed=hd + len(starts),
                                     edit=edit)
    t = len(starts)
    g = torch.Generator().manual_seed(5)
    qkv = (torch.randn(t, (nh + 2 * nkv) * hd, generator=g) * 1.5).bfloat16().to(DEV)
    # the first request's queries look for the far key
    qkv[0, : nh * hd] = (ks[0][far].float().repeat_interleave(group, dim=0).reshape(-1) * 0.5).bfloat16().to(DEV)
    out = torch.full((t, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ctx = FakeCtx(starts, counts)
    bucket = -(-(max(starts) + 1) // 256) * 256
    arr, meta = attention_bf16.build_tasks(np.asarray(starts, dtype=np.int32), np.asarray(counts, dtype=np.int32),
                                           group, window, bucket, kv_heads=nkv,
                                           max_waves=attention_bf16.max_waves_for(hd), head_size=hd)
    assert meta[3] == 4 and meta[5] is True
    live = arr[: meta[0]][arr[: meta[0], 0] >= 0]
    assert int((live[:, 5] - live[:, 4]).max()) == chunk
    ctx.plans = {attention_bf16.plan_key(group, window, nkv, hd): (torch.from_numpy(arr).to(DEV), meta)}
    scale = 1.0 / math.sqrt(hd)
    wide = torch.zeros((t, bucket // page), dtype=torch.int32, device=DEV)
    wide[:, : bt.shape[1]] = bt
    for _ in range(2):                                 # the second launch finds the counters as the first left them
        out.fill_(float("nan"))
        assert attention_bf16.try_attention(qkv, kc, vc, out, ctx, FakeCache(wide, page), scale, window, nh, nkv, hd)
        for e, s in enumerate(starts):
            q = qkv[e:e + 1, : nh * hd].cpu().view(1, nh, hd)
            want = plain_attention(q, ks[e], vs[e], s, scale, window, group).reshape(1, nh * hd)
            err = (out[e:e + 1].double().cpu() - want).abs().max() / want.abs().max()
            assert err < 2e-2, f"request {e} at {s}: {err:.3e}"


@pytest.mark.parametrize("plan", PLANS)
@pytest.mark.parametrize("window", [64, 200, 1000])
def test_decode_plans_behind_a_window(window, plan, monkeypatch):
    """Decoded tokens far behind a window, planned as the engine plans them: in chunks, their requests own slots only
    for the chunks a window can touch, the first of which is wherever the window begins; as whole ranges, eight
    waves begin where the window does."""
    import numpy as np
    from atoma_infer_amd.kernels import attention_bf16
    whole = plan == "whole"
    if whole:
        monkeypatch.setattr(attention_bf16, "WHOLE_MIN_PAIRS", 2)
    else:
        force_chunked_decode(monkeypatch, second_kernel=plan.endswith("second kernel"))
    nh, nkv, hd, page = 8, 2, 64, 16
    starts = [1500, 700, 300, 129, 5]
    counts = [1] * len(starts)
    ks, vs, kc, vc, bt = paged_setup([s + 1 for s in starts], nkv, hd, page, torch.bfloat16, seed=window)
    t = len(starts)
    g = torch.Generator().manual_seed(4)
    qkv = (torch.randn(t, (nh + 2 * nkv) * hd, generator=g) * 1.5).bfloat16().to(DEV)
    out = torch.full((t, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ctx = FakeCtx(starts, counts)
    bucket = -(-(max(starts) + 1) // 256) * 256
    arr, meta = attention_bf16.build_tasks(np.asarray(starts, dtype=np.int32), np.asarray(counts, dtype=np.int32),
                                           nh // nkv, window, bucket, kv_heads=nkv,
                                           max_waves=attention_bf16.max_waves_for(hd))
    if whole:
        assert meta[1:4] == (0, 0, 8)
    else:
        assert 0 < meta[2] <= t * (window // 128 + 2)
    ctx.plans = {attention_bf16.plan_key(nh // nkv, window, nkv, hd): (torch.from_numpy(arr).to(DEV), meta)}
    scale = 1.0 / math.sqrt(hd)
    assert attention_bf16.try_attention(qkv, kc, vc, out, ctx, FakeCache(bt, page), scale, window, nh, nkv, hd)
    for e, s0 in enumerate(starts):
        q = qkv[e:e + 1, : nh * hd].cpu().view(1, nh, hd)
        want = plain_attention(q, ks[e], vs[e], s0, scale, window, nh // nkv).reshape(1, nh * hd)
        err = (out[e:e + 1].double().cpu() - want).abs().max() / want.abs().max()
        assert err < 2e-2, f"request {e} at {s0}: {err:.3e}"


def test_the_probes_of_what_the_gpu_delivers():
    """The yardsticks that the bench prints beside its own figures: a read stream faster than any kernel here reads, a
    copy, a loop of MFMAs near the published peak; and the costs of a chain of kernels (an empty kernel, read streams,
    a grid-wide barrier whose waits are bounded and report if they run out)."""
    from atoma_infer_amd.kernels import ops
    peaks = ops.measure_device_peaks(size_bytes=1 << 28)
    assert 3000 < peaks["hbm_read_gbs"] < 8000 and peaks["hbm_read_how"]
    assert 2000 < peaks["hbm_copy_gbs"] < 8000
    assert 1500 < peaks["mfma_bf16_tflops"] < 2600
    floors = ops.measure_chain_floors()
    assert 0.5 < floors["empty_kernel_us"] < 10
    assert floors["empty_kernel_us"] < floors["read_8mb_us"] < floors["read_32mb_us"] < floors["read_64mb_us"] < 40
    assert 0.5 < floors["grid_barrier_us"] < 50


@pytest.mark.parametrize("m", [1, 5, 8, 13, 16])
@pytest.mark.parametrize("n,k,rt,wk", [(128, 512, 2, 8), (4032, 1024, 2, 8), (256, 256, 4, 4), (1000 * 64, 256, 4, 4),
                                       (96, 256, 2, 4), (2048, 2048, 2, 4)])
def test_gemm_over_a_tiled_weight_equals_the_row_major_one(m, n, k, rt, wk):
    """The copy of a weight laid out in the order the streaming kernel's waves read it (batch of steps, workgroup,
    wave, step, tile, lane) gives the very bits of the row-major weight read by the same plan, also with the rows a
    begun norm; and the offsets the library states are where the Python tiling puts every element."""
    from atoma_infer_amd.kernels import gemm_bf16, ops
    x = rnd(m, k, dtype=torch.bfloat16, seed=m)
    w = rnd(n, k, dtype=torch.bfloat16, seed=n + k, scale=0.1)
    tw = gemm_bf16.tile_weight(w, rt, wk)
    assert tw is not None and (tw.n, tw.k, tw.rt, tw.wk) == (n, k, rt, wk) and tw.data.numel() == n * k
    g = torch.Generator().manual_seed(3)
    off = gemm_bf16.lib().atoma_gemm_bf16_tiled_offset
    off.restype = ctypes.c_longlong
    for _ in range(50):
        i, j = int(torch.randint(0, n, (1,), generator=g)), int(torch.randint(0, k, (1,), generator=g))
        at = off(ctypes.c_longlong(i), ctypes.c_longlong(j), ctypes.c_longlong(n), ctypes.c_longlong(k), rt, wk, tw.u)
        assert tw.data[at] == w[i, j], (i, j, at)
    for dtype in (torch.float32, torch.bfloat16):
        if dtype is torch.bfloat16 and (rt, wk) == (4, 4):
            continue                                            # no such instance: the head's plan, float32 out
        want = torch.empty(m, n, dtype=dtype, device=DEV)
        gemm_bf16.skinny(x, w, want, 1, rt, wk)
        got = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
        gemm_bf16.skinny_tiled(x, tw, got)
        assert torch.equal(got, want)
    ref = x.double().cpu() @ w.double().cpu().T
    assert (got.double().cpu() - ref).abs().max() <= 2e-2 * ref.abs().max()
    # a begun norm as the rows
    ss = torch.rand(7, 16, device=DEV) + 0.5
    b = gemm_bf16.Begun(x, ss, 1e-5, k)
    want = torch.empty(m, n, dtype=torch.float32, device=DEV)
    gemm_bf16.skinny(b, w, want, 1, rt, wk)
    got = torch.empty(m, n, dtype=torch.float32, device=DEV)
    gemm_bf16.skinny_tiled(b, tw, got)
    assert torch.equal(got, want)
    assert gemm_bf16.tile_weight(rnd(n + 16, k + 32, dtype=torch.bfloat16), rt, wk) is None      # no whole batches


@pytest.mark.parametrize("m", [1, 8, 16, 23, 48, 64])
@pytest.mark.parametrize("inter,k,rt", [(64, 256, 2), (8192, 2048, 2), (1024, 512, 4)])
def test_swiglu_gemm_over_a_tiled_weight_equals_the_row_major_one(m, inter, k, rt, monkeypatch):
    from atoma_infer_amd.kernels import gemm_bf16
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    wg, wu = rnd(inter, k, dtype=torch.bfloat16, seed=2, scale=0.1), rnd(inter, k, dtype=torch.bfloat16, seed=3, scale=0.1)
    w = interleave16(wg, wu)
    # the plan that the fused product would choose must be the tiled copy's: force it for the small shapes
    monkeypatch.setattr(gemm_bf16, "_plan", lambda *a, **kw: (rt, 4, 1))
    tw = gemm_bf16.tile_weight(w, rt, 4)
    assert tw is not None
    want = gemm_bf16.try_linear_swiglu(x, w)
    got = gemm_bf16.try_linear_swiglu(x, w, tw)
    assert want is not None and got is not None and torch.equal(got, want)
    g, u = x.double().cpu() @ wg.double().cpu().T, x.double().cpu() @ wu.double().cpu().T
    ref = torch.nn.functional.silu(g) * u
    assert (got.double().cpu() - ref).abs().max() <= 1e-2 * ref.abs().max()


@pytest.mark.parametrize("m", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("n,k", [(2048, 2048), (2048, 8192), (72, 4096), (1000, 2048), (4096, 2048), (3072, 8192),
                                 (3072, 3072), (4096, 14336)])
def test_residual_product_over_a_tiled_weight_equals_the_row_major_one(m, n, k):
    """The product that adds into the residual rows and begins the next norm, over the copy of its weight laid out in
    the order its waves read it (half tiles): the very bits of the row-major product, and the library's offsets are
    where the Python tiling puts every element."""
    from atoma_infer_amd.kernels import gemm_bf16
    x = rnd(m, k, dtype=torch.bfloat16, seed=m)
    w = rnd(n, k, dtype=torch.bfloat16, seed=n + k, scale=0.05)
    gamma = (1 + 0.1 * rnd(n, dtype=torch.float32, seed=2)).bfloat16()
    tw = gemm_bf16.tile_weight_resid(w)
    assert tw is not None and tw.data.numel() == n * k
    half = gemm_bf16.resid_plan(m, n, k)[3]
    assert (tw.rt == 0) == bool(half) == (n <= 2048)
    off = gemm_bf16.lib().atoma_gemm_bf16_tiled_offset_half if half else gemm_bf16.lib().atoma_gemm_bf16_tiled_offset
    off.restype = ctypes.c_longlong
    g = torch.Generator().manual_seed(4)
    ll = ctypes.c_longlong
    for _ in range(50):
        i, j = int(torch.randint(0, n, (1,), generator=g)), int(torch.randint(0, k, (1,), generator=g))
        at = off(ll(i), ll(j), ll(n), ll(k), tw.wk, tw.u) if half else off(ll(i), ll(j), ll(n), ll(k), 1, tw.wk, tw.u)
        assert tw.data[at] == w[i, j], (i, j, at)
    r0 = rnd(m, n, dtype=torch.float32, seed=9)
    want_r, got_r = r0.clone(), r0.clone()
    want = gemm_bf16.try_linear_resid(x, w, want_r, gamma, 1e-5)
    got = gemm_bf16.try_linear_resid(x, w, got_r, gamma, 1e-5, tw)
    assert want is not None and got is not None
    assert torch.equal(got_r, want_r) and torch.equal(got.data, want.data) and torch.equal(got.shares, want.shares)
    ref = r0.double().cpu() + x.double().cpu() @ w.double().cpu().T
    assert (got_r.double().cpu() - ref).abs().max() <= 1e-2 * ref.abs().max()
    # shapes that do not divide into whole batches of the plan's tiles have no such copy
    assert gemm_bf16.tile_weight_resid(rnd(2048, 1024 + 512, dtype=torch.bfloat16)) is None
    assert gemm_bf16.tile_weight_resid(rnd(4096 + 8, 2048, dtype=torch.bfloat16)) is None


@pytest.mark.parametrize("n,k", [(2048, 2048), (2048, 8192), (3072, 2048), (4096, 4096), (4096, 14336), (96, 1024)])
def test_planes_of_a_split_product_over_a_tiled_weight_equal_the_row_major_ones(n, k):
    """17 to 64 rows: the float32 planes of the K-split product over the copy of the weight in the order its waves read
    it (every slice of K, over workgroup and grid, a wave of the layout) are the very bits of the row-major planes."""
    from atoma_infer_amd.kernels import gemm_bf16
    w = rnd(n, k, dtype=torch.bfloat16, seed=n + k, scale=0.05)
    tw = gemm_bf16.tile_weight_planes(w)
    rt, wk, slices = gemm_bf16._plan(64, n, k, True)
    assert tw is not None and (tw.rt, tw.wk, tw.u) == (rt, wk * slices, 2) and slices > 1
    for m in (17, 32, 33, 48, 64):
        x = rnd(m, k, dtype=torch.bfloat16, seed=m)
        want = gemm_bf16.linear_planes(x, w)
        got = gemm_bf16.linear_planes(x, w, tw)
        assert want.shape == (slices, m, n) and torch.equal(got, want)
        ref = x.double().cpu() @ w.double().cpu().T
        assert (got.double().sum(0).cpu() - ref).abs().max() <= 1e-2 * ref.abs().max()
    x = rnd(16, k, dtype=torch.bfloat16)
    assert torch.equal(gemm_bf16.linear_planes(x, w, tw), gemm_bf16.linear_planes(x, w))     # (few rows: row-major)
