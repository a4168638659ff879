"""bfloat16 x bfloat16 products on the matrix cores.

``try_linear`` picks, for x [M, K] and w [N, K]:

* the hand-written weight-streaming MFMA kernel when M is small (decode steps, short portions) or when float32
  output is wanted (logits), running it over blocks of 64 rows of x;
* the library product (hipBLASLt through ``torch.mm``) for products with many rows of x (more than 64; more
  than 32 on large weights; more than 16 for float32 output), as the reference uses a library for its linears;
* nothing (None) when the shape fits neither: the caller then runs the float32 FMA kernel.
"""
from __future__ import annotations

import ctypes
import dataclasses
from typing import Optional

import torch

from ..parts.base import Begun        # (a norm begun by the product before it: the parts' type, finished here)
from .library import load_hip_module
from .ops import BF16, F32, _check, _p, _stream

SKINNY_MAX_M = 64
BEGUN_MAX_M = 16              # rows of a step whose norms are begun and finished by the products around them


def _begun_args(x):
    """The four trailing arguments of a product whose rows may be a begun norm."""
    if isinstance(x, Begun):
        return _p(x.shares), x.shares.shape[0], ctypes.c_float(x.eps), x.width
    return _p(None), 0, ctypes.c_float(0.0), 0

LIBRARY_MIN_M_WIDE = 32       # beyond this many rows the library takes products whose weight has 2^24 elements or more
# weights up to this size keep the fused SiLU-multiply up to 64 rows (the gate-up product of the Llama 1B and 3B widths:
# at 3B, 8 layers, 33 / 48 / 64 rows 1,364 / 1,454 / 1,724 us a step against 1,405 / 1,489 / 1,735 with the library's
# product and the activation kernel; at the 8B width the library's is quicker)
SWIGLU_WIDE = 1 << 26
_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = load_hip_module("gemm_bf16")
    return _lib


def _aligned(t: torch.Tensor) -> bool:
    return t.data_ptr() % 16 == 0 and (t.shape[0] == 1 or t.stride(0) % 8 == 0) and t.stride(1) == 1


def _plan(m: int, n: int, k: int, allow_slices: bool):
    """(rows-of-16 per wave, waves splitting K, K slices over the grid) for x [m, k] @ w [n, k]^T.

    Chosen from measurements on MI355X at the sizes of Llama-3.2-1B.  Up to 16 rows of x want many waves that split
    K (every wave's loads are in flight at once).  With more rows the fragments of x weigh as much as the weight,
    so a wave owns 32 or 64 rows of W for each fragment of x it fetches; where N is small that leaves too few
    workgroups, and K is split over the grid into float32 planes, about 256 workgroups in all, if the caller takes
    planes.
    """
    tiles = -(-n // 16)
    if m <= 16:
        if tiles >= 4096:
            rt, wk = (2, 8) if m <= 8 else (4, 4)      # (the head at 16 rows: 106 against 115 us)
        elif tiles >= 512:
            rt, wk = 2, 4
        else:
            rt, wk = 1, 4
        max_slices = 2        # two planes already put enough workgroups in flight (more measured no faster)
    elif tiles >= 4096:
        rt, wk, max_slices = 4, 1, 1
    elif allow_slices and tiles < 640:
        # 64 rows of W per wave where K is long enough for the four waves of each of about 256 workgroups, else 32
        rt, wk, max_slices = 4, 4, 8
        if k // (4 * _slices_for(tiles, 4, 8)) < 128:
            rt = 2
    else:
        # as many rows of W per wave as still leave 160 workgroups
        rt, wk, max_slices = (4 if tiles >= 640 else 2 if tiles >= 320 else 1), 4, 1
    while wk > 1 and k % (32 * wk):
        wk //= 2
    if wk == 2:
        wk = 1
    slices = 1
    if allow_slices and max_slices > 1:
        per_group = (4 if wk == 1 else 1) * rt
        slices = 2 if m <= 16 and -(-tiles // per_group) <= 512 else _slices_for(tiles, per_group, max_slices)
        while slices > 1 and (k % (32 * wk * slices) or k // (wk * slices) < 128):
            slices //= 2
    return rt, wk, slices


def _slices_for(tiles: int, tiles_per_group: int, most: int) -> int:
    """The power of two, at most ``most``, of K slices that brings the grid to about 256 workgroups."""
    groups = -(-tiles // tiles_per_group)
    slices = 1
    while slices < most and groups * slices * 2 <= 256:
        slices *= 2
    return slices


@dataclasses.dataclass
class TiledWeight:
    """A weight [n, k] laid out in the order in which the streaming kernel's waves read it, for steps of at most 16
    rows (``csrc/kernels/gemm_bf16.hip``, TILED): tiles of 16 rows x 32 values of K in the lanes' order, ordered by
    batch of ``u`` steps, workgroup, wave, step, tile, for waves of ``rt`` tiles and ``wk`` waves a workgroup.  The
    loads of a whole launch then sweep memory front to back as a plain read stream does (the gate-up matrix of Llama
    1B: 11.5 us for the loads alone against 13.3 row-major).  A second copy of the weight: the row-major one serves
    the products of more rows."""
    data: torch.Tensor
    n: int
    k: int
    rt: int
    wk: int
    u: int


@dataclasses.dataclass
class TiledCopies:
    """The tiled copies of one weight: for steps of at most 16 rows, and for the K-split product of 17 to 64."""
    few: Optional[TiledWeight] = None
    many: Optional[TiledWeight] = None


TILED_COPIES = True               # False: no part gets a tiled copy of a weight (half the memory, slower decode steps)
TILED_MAX_M = 16
TILED_FOUR_TILES_MIN_M = 32
TILED_SWIGLU_MAX_M = 64          # the fused SiLU-multiply reads the tiled copy with more rows too, in the copy's tiles
TILED_MIN_ELEMENTS = 1 << 24      # smaller weights stream at the same pace row-major (measured: 8 and 34 MB)


def tile_weight(w: torch.Tensor, rt: int, wk: int, u: int = 0) -> Optional[TiledWeight]:
    """The tiled copy of ``w`` [n, k] (bfloat16, row-major) for waves of ``rt`` tiles and ``wk`` waves a workgroup, or
    None where the shape does not divide into whole batches of tiles.  ``u``: steps a batch, for a kernel that does
    not take the depth that goes with (rt, wk)."""
    n, k = w.shape
    u = u or int(lib().atoma_gemm_bf16_batch_depth(1, rt, wk))
    if (not TILED_COPIES or w.dtype is not torch.bfloat16 or n % (16 * rt) or k % (32 * wk * u)
            or not w.is_contiguous()):
        return None
    groups, batches = n // (16 * rt), k // (32 * wk * u)
    t = w.view(groups, rt, 16, wk, batches, u, 4, 8)             # group, tile, row, wave, batch, step, piece, value
    t = t.permute(4, 0, 3, 5, 1, 6, 2, 7).contiguous()            # batch, group, wave, step, tile, piece, row, value
    return TiledWeight(t.view(-1), n, k, rt, wk, u)


def tile_weight_resid(w: torch.Tensor) -> Optional[TiledWeight]:
    """The tiled copy of ``w`` [n, k] for the product that adds into the residual stream, in the plan that
    ``resid_plan`` gives it: eight waves a workgroup and batches of 4 or 8 steps, of whole tiles or (``rt`` 0 in the
    result) of half tiles, 8 rows of the weight and 64 values of K a wave and step.  None where the plan is another
    or the shape does not divide."""
    n, k = w.shape
    rt, wk, u, half = resid_plan(1, n, k)
    if w.dtype is not torch.bfloat16 or not w.is_contiguous() or (rt, wk) != (1, 8) or u not in (4, 8):
        return None
    if not half:
        return tile_weight(w, 1, wk, u)
    if not TILED_COPIES or n % 8 or k % (64 * wk * u):
        return None
    t = w.view(n // 8, 8, wk, k // (64 * wk * u), u, 2, 4, 8)     # group, row, wave, batch, step, half, piece, value
    t = t.permute(3, 0, 2, 4, 6, 5, 1, 7).contiguous()            # batch, group, wave, step, piece, half, row, value
    return TiledWeight(t.view(-1), n, k, 0, wk, u)


def tile_weight_rope(w: torch.Tensor) -> Optional[TiledWeight]:
    """The tiled copy of a fused q, k, v weight for the product with the rotary epilogue at up to 8 rows, or None
    where that product's plan has no tiled kernel."""
    n, k = w.shape
    rt, wk, _ = _plan(8, n, k, False)
    if wk != 4 or rt > 2:
        return None
    return tile_weight(w, rt, wk)


def tile_copies_resid(w: torch.Tensor) -> Optional[TiledCopies]:
    """The tiled copies of a weight whose product is added to the residual stream; None if there is none."""
    c = TiledCopies(tile_weight_resid(w), tile_weight_planes(w))
    return c if c.few is not None or c.many is not None else None


def tile_copies_rope(w: torch.Tensor) -> Optional[TiledCopies]:
    """The tiled copies of a fused q, k, v weight; None if there is none."""
    c = TiledCopies(tile_weight_rope(w), tile_weight_planes(w))
    return c if c.few is not None or c.many is not None else None


def tiled_plan(n: int, k: int, swiglu: bool):
    """(rt, wk) of the tiled layout for a weight [n, k]: what ``_plan`` gives steps of at most 8 rows (the fused
    SiLU-multiply's own choice for the gate-up matrix), so that the tiled kernel is the planned one; None for
    weights that gain nothing."""
    if n * k < TILED_MIN_ELEMENTS:
        return None
    rt, wk, _ = _plan(8, n, k, False)
    if swiglu:
        if rt % 2:
            rt = 2
        if wk == 4 and -(-n // 16) >= 1536:
            rt = 4
        if wk != 4 or rt not in (2, 4):
            return None
    elif (rt, wk) not in ((2, 8), (4, 4), (2, 4)):
        return None
    return rt, wk


def skinny_tiled(x, tw: TiledWeight, out: torch.Tensor) -> None:
    """out [M <= 16, n] = x @ w^T over the tiled copy of w; x may be a ``Begun`` norm."""
    begun = _begun_args(x)
    if isinstance(x, Begun):
        x = x.data
    m, k = x.shape
    code = {torch.float32: F32, torch.bfloat16: BF16}[out.dtype]
    _check(lib().atoma_gemm_bf16_skinny_tiled(_p(x), _p(tw.data), _p(out), code, m, tw.n, k, x.stride(0) if m > 1 else k,
                                              out.stride(-2) if m > 1 else tw.n, tw.rt, tw.wk, *begun, _stream()),
           "gemm_bf16_skinny_tiled")


def skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype is torch.bfloat16 and w.dtype is torch.bfloat16 and x.dim() == 2 and w.dim() == 2
            and x.shape[1] == w.shape[1] and x.shape[1] % 32 == 0 and _aligned(x) and _aligned(w))


def skinny(x, w: torch.Tensor, out: torch.Tensor, slices: int = 1, rt: int = 0, wk: int = 0) -> None:
    """out [M, N] (or [slices, M, N] float32 planes) = x [M <= 64, K] @ w [N, K]^T; x may be a ``Begun`` norm."""
    begun = _begun_args(x)
    if isinstance(x, Begun):
        x = x.data
    m, k = x.shape
    n = w.shape[0]
    if not rt:
        rt, wk, _ = _plan(m, n, k, False)
        if k % (32 * wk * slices):
            wk = 1
    ldc = out.stride(-2) if m > 1 else n
    code = {torch.float32: F32, torch.bfloat16: BF16}[out.dtype]
    _check(lib().atoma_gemm_bf16_skinny(_p(x), _p(w), _p(out), code, m, n, k, x.stride(0) if m > 1 else k,
                                        w.stride(0) if n > 1 else k, ldc, rt, wk, slices, *begun, _stream()),
           "gemm_bf16_skinny")


def _library_wins(m: int, n: int, k: int, out_dtype: torch.dtype) -> bool:
    """Measured on MI355X at the layer shapes of Llama 1B, 3B and 8B: where the library's tiles beat the streaming
    kernel for a product with output in ``out_dtype``.

    The streaming kernel fetches the activations anew for every 16 to 64 rows of the weight, which costs little up
    to 16 rows of activations and as much as the weight itself beyond 32."""
    if out_dtype is torch.float32:
        return m > 16 and _MM_OUT_DTYPE
    if m > SKINNY_MAX_M:
        return True
    return m > LIBRARY_MIN_M_WIDE and n * k >= (1 << 24)


def _probe_mm_out_dtype() -> bool:
    """Whether this torch has ``mm(..., out_dtype=float32)`` for bfloat16 operands (float32 accumulation either way)."""
    doc = getattr(torch.mm, "__doc__", "") or ""
    return "out_dtype" in doc


_MM_OUT_DTYPE = _probe_mm_out_dtype()


def try_linear(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, out: Optional[torch.Tensor] = None,
               library_only: bool = False, tiled: Optional[TiledWeight] = None) -> Optional[torch.Tensor]:
    """x [M, K] @ w [N, K]^T if a fast kernel takes the shape, else None (the caller falls back to float32 FMAs).
    ``library_only``: None also where the library would not be the choice.  ``tiled``: the tiled copy of ``w``, read
    in its place by steps of at most 16 rows, in the copy's own plan (the head of Llama 1B, 525 MB, tiled for two
    tiles and eight waves: 88, 90 and 99 us at 1, 8 and 16 rows against 88, 95 and 103 for the best row-major plan of
    each)."""
    if tiled is not None and not library_only and x.shape[0] <= TILED_MAX_M and x.shape[1] == tiled.k:
        xd = x.data if isinstance(x, Begun) else x
        dtype = out_dtype if out is None else out.dtype
        if (xd.dtype is torch.bfloat16 and _aligned(xd)
                and (dtype is torch.float32 or (dtype is torch.bfloat16 and (tiled.rt, tiled.wk) != (4, 4)))):
            if out is None:
                out = torch.empty((xd.shape[0], tiled.n), dtype=out_dtype, device=xd.device)
            skinny_tiled(x, tiled, out)
            return out
    if isinstance(x, Begun):
        if not skinny_ok(x.data, w):
            return None
        if out is None:
            out = torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=w.device)
        skinny(x, w, out)
        return out
    m, n = x.shape[0], w.shape[0]
    k = x.shape[1]
    ok = skinny_ok(x, w)
    if library_only:
        if not (_MM_OUT_DTYPE and out_dtype is torch.float32 and m > LIBRARY_MIN_M_WIDE):
            return None
    elif not (ok and _library_wins(m, n, k, out_dtype)) and ok and (m <= SKINNY_MAX_M or out_dtype is torch.float32):
        if out is None:
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        for lo in range(0, m, SKINNY_MAX_M):
            hi = min(lo + SKINNY_MAX_M, m)
            skinny(x[lo:hi], w, out[lo:hi])
        return out
    if out_dtype is torch.float32 and _MM_OUT_DTYPE and m > 16:
        y = torch.mm(x, w.t(), out_dtype=torch.float32)
        if out is None:
            return y
        out.copy_(y)
        return out
    if out_dtype is torch.bfloat16 and m > LIBRARY_MIN_M_WIDE:
        if out is None:
            return torch.mm(x, w.t())
        return torch.mm(x, w.t(), out=out)
    return None


def _probe_addmm_out_dtype() -> bool:
    doc = getattr(torch.addmm, "__doc__", "") or ""
    return "out_dtype" in doc


_ADDMM_OUT_DTYPE = _probe_addmm_out_dtype()


def try_addmm_resid(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor) -> bool:
    """``resid += x @ w^T`` by the library (hipBLASLt with beta = 1: the float32 sums of the product are added to the
    float32 rows in place, so the product's own result is never written or read again), for products of more rows
    than the streaming kernels take; False, nothing done, where that is not the choice."""
    m = x.shape[0]
    if not (_ADDMM_OUT_DTYPE and m > SKINNY_MAX_M and x.dtype is torch.bfloat16 and w.dtype is torch.bfloat16
            and resid.dtype is torch.float32 and resid.is_contiguous() and tuple(resid.shape) == (m, w.shape[0])):
        return False
    torch.addmm(resid, x, w.t(), out_dtype=torch.float32, out=resid)
    return True


def tile_weight_planes(w: torch.Tensor) -> Optional[TiledWeight]:
    """The tiled copy of ``w`` [n, k] for the K-split product of 17 to 64 rows (``linear_planes``; the plan is the same
    for all of them): ``wk`` in the result counts the slices of K over workgroup and grid.  None where that plan has
    no tiled kernel or the shape does not divide."""
    n, k = w.shape
    rt, wk, slices = _plan(SKINNY_MAX_M, n, k, True)
    if wk != 4 or rt not in (2, 4) or slices < 2:
        return None
    return tile_weight(w, rt, wk * slices, 2)


def linear_planes(x: torch.Tensor, w: torch.Tensor, tiled: Optional[TiledWeight] = None) -> Optional[torch.Tensor]:
    """For M <= 64: float32 planes [slices, M, N] whose sum is x @ w^T (K split over the grid), else None.
    ``tiled``: the copy of ``w`` that ``tile_weight_planes`` made, read in its place by 17 rows and more."""
    m, k = x.shape
    n = w.shape[0]
    if m > SKINNY_MAX_M or not skinny_ok(x, w):
        return None
    rt, wk, slices = _plan(m, n, k, True)
    out = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
    if tiled is not None and m > 16 and (tiled.n, tiled.k, tiled.rt, tiled.wk, tiled.u) == (n, k, rt, wk * slices, 2):
        _check(lib().atoma_gemm_bf16_skinny_tiled_planes(_p(x), _p(tiled.data), _p(out), m, n, k, x.stride(0), n, rt,
                                                         slices, _stream()), "gemm_bf16_skinny_tiled_planes")
        return out
    skinny(x, w, out, slices, rt, wk)
    return out


def try_linear_swiglu(x: torch.Tensor, w: torch.Tensor, tiled: Optional[TiledWeight] = None) -> Optional[torch.Tensor]:
    """silu(gate) * up of x @ w^T in one kernel, for few rows of x; w [2 I, K] is interleaved in blocks of 16.

    None when the shape is not taken (the caller then runs the product and the activation separately).
    """
    begun = _begun_args(x)
    if isinstance(x, Begun):
        x = x.data
    m, k = x.shape
    n = w.shape[0]
    if m > SKINNY_MAX_M or (m > LIBRARY_MIN_M_WIDE and n * k > SWIGLU_WIDE) or n % 32 or not skinny_ok(x, w):
        return None
    rt, wk, _ = _plan(m, n, k, False)
    if rt % 2:
        rt = 2
    # few rows against very many columns: 64 rows of the weight a wave (the gate-up product of Llama 8B with 8 rows:
    # 43.7 us against 46.9 with 32, and 1.4 % of a decode step; at the 16,384 columns of Llama 1B and 3B it measures
    # quicker alone, 15.3 and 20.8 us against 15.9 and 21.6, and 1 % slower within a step)
    if m <= 16 and wk == 4 and -(-n // 16) >= 1536:
        rt = 4
    if (rt, wk) not in ((2, 1), (4, 1), (2, 4), (2, 8), (4, 4)):
        return None
    out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    if tiled is not None and (tiled.n, tiled.k) == (n, k) and tiled.wk == wk and m <= TILED_SWIGLU_MAX_M:
        # waves of four tiles read a copy made for two as well, and gain on it from 32 rows on (measured over the
        # 16 layers of Llama 1B: 1,346 against 1,362 us a step at 32 rows, 1,929 against 1,970 at 64; 1,235 against
        # 1,231 at 24)
        rt = 4 if tiled.rt == 4 or (m >= TILED_FOUR_TILES_MIN_M and n % 64 == 0) else 2
        _check(lib().atoma_gemm_bf16_skinny_swiglu_tiled(_p(x), _p(tiled.data), _p(out), m, n, k,
                                                         x.stride(0) if m > 1 else k, n // 2, rt, tiled.rt, wk, *begun,
                                                         _stream()),
               "gemm_bf16_skinny_swiglu_tiled")
        return out
    _check(lib().atoma_gemm_bf16_skinny_swiglu(_p(x), _p(w), _p(out), m, n, k, x.stride(0) if m > 1 else k,
                                               w.stride(0), n // 2, rt, wk, *begun, _stream()),
           "gemm_bf16_skinny_swiglu")
    return out


ROPE_MAX_M = SKINNY_MAX_M
# Rows beyond which the q, k, v product is split along K into planes and a second kernel sums, rotates and stores
# (measured on MI355X over the 16 layers of a Llama 1B decode step: 1 to 2 % slower steps at 17 to 32 rows, 1 % quicker
# at 48, 2 % at 64: 16.3 us become 8 + 6)
ROPE_PLANES_MIN_M = 40


def try_linear_rope(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                    kcache: torch.Tensor, vcache: torch.Tensor, slot_mapping: torch.Tensor, page_size: int, nh: int,
                    nkv: int, hd: int, always: bool = False, tiled: Optional[TiledCopies] = None,
                    ) -> Optional[torch.Tensor]:
    """The fused q, k, v projection with rotary encoding and the cache write in its epilogue, for few rows of x.

    ``w`` has the rows of its q and k heads in pair order (see ``parts/attention.py``).  Returns the rotated q
    [M, nh * hd]; k (rotated) and v are in the cache.  None when the shape is not taken, or when the library's
    product followed by the rotary kernel is the quicker way (unless ``always``).
    """
    begun = _begun_args(x)
    if isinstance(x, Begun):
        x = x.data
    m, k = x.shape
    n = w.shape[0]
    if (m > ROPE_MAX_M or (not always and _library_wins(m, n, k, torch.bfloat16)) or n != (nh + 2 * nkv) * hd or hd % 4 or not skinny_ok(x, w)
            or kcache.dtype is not torch.bfloat16 or vcache.dtype is not torch.bfloat16
            or cos.dtype is not torch.float32 or cos.shape[1] != hd // 2 or not cos.is_contiguous()
            or not sin.is_contiguous() or not kcache.is_contiguous() or not vcache.is_contiguous()):
        return None
    out = torch.empty((m, nh * hd), dtype=torch.bfloat16, device=x.device)
    if m > ROPE_PLANES_MIN_M and begun[1] == 0:
        # more rows than one tile: K split over the grid into float32 planes (every workgroup then fetches a slice of
        # the activations, not all of them), summed, rotated and stored by a second kernel
        rt, wk, slices = _plan(m, n, k, True)
        if slices > 1:
            planes = linear_planes(x, w, tiled.many if tiled is not None else None)
            _check(lib().atoma_rope_from_planes(_p(planes), slices, m, _p(out), nh * hd, _p(positions), _p(cos), _p(sin),
                                                _p(kcache), _p(vcache), _p(slot_mapping), int(page_size), nh, nkv, hd,
                                                _stream()), "rope_from_planes")
            return out
    rt, wk, _ = _plan(m, n, k, False)
    if rt > 2:
        rt = 2
    if 8 < m <= 16 and rt == 1 and wk == 4 and n >= 5120:
        rt = 2          # (9 to 16 rows at Llama 3B's and 8B's sizes: 14.1 and 17.1 us against 15.3 and 18.9)
    few = tiled.few if tiled is not None else None
    if few is not None and m <= TILED_MAX_M and (few.n, few.k, few.rt, few.wk) == (n, k, rt, wk):
        _check(lib().atoma_gemm_bf16_skinny_rope_tiled(_p(x), _p(few.data), _p(out), m, k, x.stride(0) if m > 1 else k,
                                                       nh * hd, rt, wk, _p(positions), _p(cos), _p(sin), _p(kcache),
                                                       _p(vcache), _p(slot_mapping), int(page_size), nh, nkv, hd, *begun,
                                                       _stream()), "gemm_bf16_skinny_rope_tiled")
        return out
    _check(lib().atoma_gemm_bf16_skinny_rope(_p(x), _p(w), _p(out), m, k, x.stride(0) if m > 1 else k, w.stride(0),
                                             nh * hd, rt, wk, _p(positions), _p(cos), _p(sin), _p(kcache), _p(vcache),
                                             _p(slot_mapping), int(page_size), nh, nkv, hd, *begun, _stream()),
           "gemm_bf16_skinny_rope")
    return out


def resid_plan(m: int, n: int, k: int):
    """(tiles of 16 rows of the weight per wave, waves splitting K, steps of K per batch of loads, half tiles) of the
    product that adds into the residual stream: K is split over the waves of a workgroup only (every sum has one
    owner, which also begins the norm), as many ways as K allows.  With N up to 2,048 a wave owns 8 rows of the
    weight, not 16, so that 256 workgroups share the product; the lanes of the other 8 rows fetch the same rows
    further along K (measured at Llama 1B's o and down products with 8 rows of activations: 5.3 and 11.7 us against
    5.9 and 15.0 with 16 rows a wave, and 12.7 when those lanes fetched nothing); wider outputs fill the GPU with
    whole tiles, and half tiles cost them a third more (Llama 3B: 7.8 and 15.0 us against 10.5 and 21.4; 8B: 9.6 and
    27.0 against 12.9 and 35.9)."""
    wk = 8
    while wk > 1 and k % (32 * wk):
        wk //= 2
    if wk == 2:
        wk = 1
    half = 1 if n <= 2048 and k % (64 * wk) == 0 else 0        # (a step of half tiles covers 64 values of K)
    depths = {(8, 1): (4, 2, 8), (8, 0): (8, 4, 2), (4, 1): (4, 8), (4, 0): (4,), (1, 1): (4,), (1, 0): (4,)}[(wk, half)]
    depth = next((d for d in depths if k % ((64 if half else 32) * wk * d) == 0), 4)
    return 1, wk, depth, half


def try_linear_resid(x, w: torch.Tensor, resid: torch.Tensor, gamma: torch.Tensor, eps: float,
                     tiled: Optional[TiledWeight] = None) -> Optional[Begun]:
    """resid [M <= 16, N] float32 += x @ w^T in place, with the norm (gamma, eps) of the new rows begun: returns
    it as ``Begun``, or None (and nothing done) when the shape is not taken.  x may itself be ``Begun``.  ``tiled``:
    the copy of ``w`` that ``tile_weight_resid`` made, read in its place."""
    begun = _begun_args(x)
    xd = x.data if isinstance(x, Begun) else x
    m, k = xd.shape
    n = w.shape[0]
    if (m > BEGUN_MAX_M or not skinny_ok(xd, w) or n % 4 or resid.dtype is not torch.float32
            or tuple(resid.shape) != (m, n) or not resid.is_contiguous() or not gamma.is_contiguous()
            or gamma.numel() != n or gamma.dtype not in (torch.float32, torch.bfloat16)):
        return None
    rt, wk, depth, half = resid_plan(m, n, k)
    parts = lib().atoma_gemm_bf16_resid_parts(n, rt, wk, half)
    u = torch.empty((m, n), dtype=torch.bfloat16, device=w.device)
    shares = torch.empty((parts, 16), dtype=torch.float32, device=w.device)
    code = F32 if gamma.dtype is torch.float32 else BF16
    if tiled is not None and (tiled.n, tiled.k, tiled.rt, tiled.wk, tiled.u) == (n, k, 0 if half else rt, wk, depth):
        _check(lib().atoma_gemm_bf16_skinny_resid_tiled(_p(xd), _p(tiled.data), m, n, k, xd.stride(0) if m > 1 else k,
                                                        depth, half, *begun, _p(resid), _p(gamma), code, _p(u),
                                                        _p(shares), _stream()), "gemm_bf16_skinny_resid_tiled")
        return Begun(u, shares, float(eps), n)
    _check(lib().atoma_gemm_bf16_skinny_resid(_p(xd), _p(w), m, n, k, xd.stride(0) if m > 1 else k, w.stride(0), rt, wk,
                                              depth, half, *begun, _p(resid), _p(gamma), code, _p(u), _p(shares), _stream()),
           "gemm_bf16_skinny_resid")
    return Begun(u, shares, float(eps), n)
