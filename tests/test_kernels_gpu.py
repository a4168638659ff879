"""Each kernel alone against a plain float32 formula in PyTorch, at sizes other than the engine's."""
import math

import pytest
import torch

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
@pytest.mark.parametrize("inter", [10, 250, 1024])
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
    c = gemm_bf16.try_linear(a, w, cdt)
    assert c is not None and c.dtype is cdt
    want = a.double().cpu() @ w.double().cpu().T
    tol = 1e-5 if cdt is torch.float32 else 1e-2
    assert (c.double().cpu() - want).abs().max() <= tol * want.abs().max()
    planes = gemm_bf16.linear_planes(a, w)
    assert planes is not None and planes.dim() == 3
    assert (planes.sum(0).double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()


def test_gemm_bf16_rows_do_not_depend_on_the_batch():
    from atoma_infer_amd.kernels import gemm_bf16
    a, w = rnd(64, 512, dtype=torch.bfloat16, seed=1), rnd(300, 512, dtype=torch.bfloat16, seed=2)
    full = gemm_bf16.try_linear(a, w, torch.float32)
    for lo, hi in [(0, 1), (5, 6), (10, 33), (63, 64)]:
        part = gemm_bf16.try_linear(a[lo:hi], w, torch.float32)
        assert torch.equal(part, full[lo:hi])


def test_gemm_bf16_float32_out_for_many_rows():
    from atoma_infer_amd.kernels import gemm_bf16
    a, w = rnd(150, 64, dtype=torch.bfloat16, seed=1), rnd(333, 64, dtype=torch.bfloat16, seed=2)
    c = gemm_bf16.try_linear(a, w, torch.float32)
    want = a.double().cpu() @ w.double().cpu().T
    assert (c.double().cpu() - want).abs().max() <= 1e-5 * want.abs().max()
    cb = gemm_bf16.try_linear(a, w, torch.bfloat16)   # the library product
    assert (cb.double().cpu() - want).abs().max() <= 1e-2 * want.abs().max()
    assert gemm_bf16.try_linear(a[:, :40], w[:, :40], torch.float32) is None   # K no multiple of 32: refused
