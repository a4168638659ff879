"""Python face of the HIP kernels: argument checks on the host, then one C call per op on the current stream.

Every function takes device tensors and writes into tensors the caller passes or that it allocates with torch
(torch is the allocator and the stream owner; it computes nothing here).  Shapes, strides and dtypes are checked
before a launch, because a kernel that reads outside a tensor can take the GPU down.  A missing or unbuildable
library raises ``KernelBuildError``; there is no other code path.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .library import load_hip_module

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream of the current device as the kernels' launch argument.  Asked for at every launch (a
    graph capture changes it); the raw accessor costs a fraction of a microsecond, the public one several."""
    if _raw_stream is not None and _raw_device is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int, op: str):
    if rc == 0:
        return
    if rc == -2:
        raise KernelError(f"{op}: unsupported combination of element types")
    if rc == -3:
        raise KernelError(f"{op}: the kernel refuses these sizes")
    raise KernelError(f"{op}: HIP error {rc}")


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*ts):
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "kernels run on device tensors only; got a CPU tensor")


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None):
    _need(t.dtype is torch.int32 and t.is_contiguous(), f"{what} must be a contiguous int32 tensor")
    if n is not None:
        _need(t.numel() >= n, f"{what} has {t.numel()} entries, {n} are needed")


_core = None


def core():
    global _core
    if _core is None:
        _core = load_hip_module("core")
    return _core


# ------------------------------------------------------------------------------------------------------------

def embed(tokens: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = table[tokens[t]] as float32; a token outside the table gives a row of NaN."""
    _dev(tokens, table)
    _i32(tokens, "tokens")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [vocab, width]")
    n, width = tokens.numel(), table.shape[1]
    if out is None:
        out = torch.empty((n, width), dtype=torch.float32, device=table.device)
    _need(out.dtype is torch.float32 and out.is_contiguous() and tuple(out.shape) == (n, width), "embed: bad out")
    _check(core().atoma_embed(_p(tokens), _p(table), _code(table, "embedding table"), _p(out), n, width,
                              table.shape[0], _stream()), "embed")
    return out


def embed_begin_norm(tokens: torch.Tensor, table: torch.Tensor, gamma: torch.Tensor):
    """The embedding gather with a norm begun, for at most 16 tokens: (resid float32 [T, W], u bfloat16 [T, W] =
    resid * gamma, ss float32 [1, 16] the rows' sums of squares).  A product finishes the norm (gemm_bf16)."""
    _dev(tokens, table, gamma)
    _i32(tokens, "tokens")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [vocab, width]")
    n, width = tokens.numel(), table.shape[1]
    _need(0 < n <= 16, "embed_begin_norm takes at most 16 tokens")
    _need(gamma.is_contiguous() and gamma.numel() == width, "norm weight must have one entry per column")
    resid = torch.empty((n, width), dtype=torch.float32, device=table.device)
    u = torch.empty((n, width), dtype=torch.bfloat16, device=table.device)
    ss = torch.empty((1, 16), dtype=torch.float32, device=table.device)
    _check(core().atoma_embed_begin_norm(_p(tokens), _p(table), _code(table, "embedding table"), _p(resid), _p(gamma),
                                         _code(gamma, "norm weight"), _p(u), _p(ss), n, width, table.shape[0],
                                         _stream()), "embed_begin_norm")
    return resid, u, ss


def finish_norm(u: torch.Tensor, ss: torch.Tensor, eps: float, width: int) -> torch.Tensor:
    """u [T <= 16, W] bfloat16 divided by sqrt(sum_p ss[p, row] / width + eps), row by row, as bfloat16."""
    _dev(u, ss)
    _need(u.dtype is torch.bfloat16 and u.dim() == 2 and u.is_contiguous() and u.shape[0] <= 16, "finish_norm: bad u")
    _need(ss.dtype is torch.float32 and ss.dim() == 2 and ss.shape[1] == 16 and ss.is_contiguous(),
          "finish_norm: shares must be float32 [parts, 16]")
    out = torch.empty_like(u)
    _check(core().atoma_finish_norm(_p(u), _p(ss), ss.shape[0], ctypes.c_float(eps), _p(out), u.shape[0], u.shape[1],
                                    _stream()), "finish_norm")
    return out


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """resid += delta (in place, float32); return rmsnorm(resid) * weight in ``out_dtype``.

    With ``rows`` (int32 row numbers) only those rows are summed and normed, into a result of len(rows) rows,
    and resid is left as it is.
    """
    _dev(resid, delta, weight, rows)
    _need(resid.dtype is torch.float32 and resid.dim() == 2 and resid.is_contiguous(), "resid must be float32 [T, W]")
    t, width = resid.shape
    _need(weight.is_contiguous() and weight.numel() == width, "norm weight must have one entry per column")
    planes, plane_stride = 1, 0
    if delta is not None:
        if delta.dim() == 3:  # planes of a K-split product, summed here
            planes, plane_stride = delta.shape[0], t * width
            _need(delta.is_contiguous() and tuple(delta.shape[1:]) == (t, width), "delta planes must match resid")
        else:
            _need(delta.is_contiguous() and tuple(delta.shape) == (t, width), "delta must match resid")
    n = t
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    if out is None:
        out = torch.empty((n, width), dtype=out_dtype, device=resid.device)
    _need(out.is_contiguous() and tuple(out.shape) == (n, width) and out.dtype is out_dtype, "add_rmsnorm: bad out")
    _check(core().atoma_add_rmsnorm(_p(resid), _p(delta), _code(delta, "delta") if delta is not None else F32,
                                    _p(weight), _code(weight, "norm weight"), _p(out), _code(out, "out"), _p(rows),
                                    n, width, ctypes.c_float(eps), planes, ctypes.c_size_t(plane_stride),
                                    _stream()), "add_rmsnorm")
    return out


def rope_cache_write(qkv: torch.Tensor, positions: torch.Tensor, cos: Optional[torch.Tensor],
                     sin: Optional[torch.Tensor], rotary_dim: int, kcache: Optional[torch.Tensor],
                     vcache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], page_size: int, nh: int,
                     nkv: int, hd: int, q_out: Optional[torch.Tensor] = None) -> None:
    """Rotate q and k of ``qkv`` [T, (nh + 2 nkv) hd] (q in place), store rotated k and v at ``slot_mapping``.

    kcache and vcache are [pages, nkv, page_size * hd] tiles (order: cache/layout.py).  Null caches: rotate q only.
    With ``q_out`` [T, nh hd] the members of pair i arrive as columns 2i and 2i + 1 of a q or k head (rows of the
    projection reordered at load time); the rotated q is written to ``q_out`` and k to the cache in their own
    column order, and ``qkv`` is left as it is.
    """
    _dev(qkv, positions, cos, sin, kcache, vcache, slot_mapping)
    t = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= (nh + 2 * nkv) * hd, "qkv: bad shape")
    _i32(positions, "positions", t)
    if cos is not None:
        _need(sin is not None and cos.dtype is torch.float32 and sin.dtype is torch.float32 and cos.is_contiguous()
              and sin.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == rotary_dim // 2,
              "rotary tables must be float32 [positions, rotary_dim/2]")
    cache_code = _code(qkv, "qkv")
    if q_out is not None:
        _dev(q_out)
        _need(q_out.dtype is qkv.dtype and q_out.dim() == 2 and q_out.stride(1) == 1 and q_out.shape[0] == t
              and q_out.shape[1] >= nh * hd and cos is not None and rotary_dim == hd,
              "q_out must be [T, nh hd] of qkv's dtype, with the whole head rotated")
    if kcache is not None:
        _need(vcache is not None and slot_mapping is not None, "cache write needs k, v and slots")
        _i32(slot_mapping, "slot_mapping", t)
        pages = kcache.shape[0]
        _need(kcache.is_contiguous() and vcache.is_contiguous() and tuple(kcache.shape) == (pages, nkv, page_size * hd)
              and tuple(vcache.shape) == (pages, nkv, page_size * hd) and kcache.dtype is vcache.dtype,
              "cache tensors must be [pages, nkv, page_size * hd] tiles")
        cache_code = _code(kcache, "cache")
    _check(core().atoma_rope_cache_write(_p(qkv), _code(qkv, "qkv"), qkv.stride(0), _p(positions), _p(cos), _p(sin),
                                         rotary_dim, _p(kcache), _p(vcache), cache_code, _p(slot_mapping), page_size,
                                         t, nh, nkv, hd, _p(q_out), q_out.stride(0) if q_out is not None else 0,
                                         _stream()), "rope_cache_write")


def paged_attention_generic(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, out: torch.Tensor,
                            block_tables: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor,
                            scale: float, window: int, page_size: int, nh: int, nkv: int, hd: int,
                            slopes: Optional[torch.Tensor] = None) -> None:
    """Attention of every token of ``q`` [T, >= nh hd] (row stride free) over its request's cached keys.

    Token t belongs to row ``token_seq[t]`` of ``block_tables`` and sits at absolute position ``positions[t]``;
    it sees keys max(0, p - window + 1) .. p (window 0: all).  ``out`` is [T, nh hd].  ``slopes`` (float32 [nh]):
    head h's score of key j gains ``slopes[h] * (j - p)``.
    """
    _dev(q, kcache, vcache, out, block_tables, token_seq, positions)
    t = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd, "q: bad shape")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == t and out.shape[1] >= nh * hd
          and out.dtype is q.dtype, "out: bad shape")
    pages = kcache.shape[0]
    _need(kcache.is_contiguous() and vcache.is_contiguous() and tuple(kcache.shape) == (pages, nkv, page_size * hd)
          and tuple(vcache.shape) == (pages, nkv, page_size * hd) and kcache.dtype is vcache.dtype,
          "cache tensors must be [pages, nkv, page_size * hd] tiles")
    _need(block_tables.dim() == 2 and block_tables.dtype is torch.int32 and block_tables.is_contiguous(),
          "block_tables must be contiguous int32 [requests, blocks]")
    _i32(token_seq, "token_seq", t)
    _i32(positions, "positions", t)
    if slopes is not None:
        _dev(slopes)
        _need(slopes.dtype is torch.float32 and slopes.is_contiguous() and slopes.numel() == nh,
              "slopes must be contiguous float32, one per query head")
    _check(core().atoma_paged_attention_generic(
        _p(q), q.stride(0), _p(kcache), _p(vcache), _p(out), out.stride(0), _code(q, "q"), _code(kcache, "cache"),
        _p(block_tables), block_tables.shape[1], _p(token_seq), _p(positions), ctypes.c_float(scale), int(window),
        page_size, t, nh, nkv, hd, _p(slopes), _stream()), "paged_attention_generic")


def swiglu(gu: torch.Tensor, out: Optional[torch.Tensor] = None, block: int = 0) -> torch.Tensor:
    """out[t, i] = silu(gate[t, i]) * up[t, i] for gu [T, 2 I].

    ``block`` 0: gate is the first half of a row and up the second; 16: blocks of 16 gate values followed by
    their 16 up values (the order of the fused gate-up product's weight rows).
    """
    _dev(gu)
    _need(gu.dim() == 2 and gu.is_contiguous() and gu.shape[1] % 2 == 0, "swiglu input must be contiguous [T, 2 I]")
    t, inter = gu.shape[0], gu.shape[1] // 2
    if out is None:
        out = torch.empty((t, inter), dtype=gu.dtype, device=gu.device)
    _need(out.is_contiguous() and tuple(out.shape) == (t, inter) and out.dtype is gu.dtype, "swiglu: bad out")
    _check(core().atoma_swiglu(_p(gu), _p(out), _code(gu, "swiglu input"), t, inter, int(block), _stream()), "swiglu")
    return out


def gemm_generic(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, out: Optional[torch.Tensor] = None,
                 ) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed, in true float32 arithmetic; any sizes."""
    _dev(a, w)
    _need(a.dim() == 2 and w.dim() == 2 and a.stride(1) == 1 and w.stride(1) == 1 and a.shape[1] == w.shape[1],
          f"gemm: a {tuple(a.shape)} and w {tuple(w.shape)} do not fit")
    m, k = a.shape
    n = w.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    _need(out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (m, n) and out.dtype is out_dtype,
          "gemm: bad out")
    _check(core().atoma_gemm_generic(_p(a), _code(a, "a"), _p(w), _code(w, "w"), _p(out), _code(out, "out"), m, n, k,
                                     a.stride(0) if m > 1 else k, w.stride(0) if n > 1 else k,
                                     out.stride(0) if m > 1 else n, _stream()), "gemm_generic")
    return out


SPLIT_MAX_VOCAB = 262144       # the largest vocabulary whose rows ``sample_packed(split=True)`` cuts into parts


def sample_packed(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                  uniform: torch.Tensor, workspace: Optional[torch.Tensor] = None, split: bool = False,
                  cuts: bool = True) -> torch.Tensor:
    """Per row of float32 ``logits`` [S, V]: argmax where temperature <= 0, else a draw (see sampling.hip).

    Returns one float32 tensor [2, S]: row 0 holds the tokens (int32 bits), row 1 the logits of the chosen tokens,
    so that one copy brings both to the host.  ``split``: every row is shared by several blocks over six short
    launches instead of one long one (the same tokens; quicker when rows draw from a large vocabulary: one block
    walks a row with top-k and top-p in over 100 us); vocabularies beyond ``SPLIT_MAX_VOCAB`` keep the one launch.
    ``cuts=False`` (with ``split``): the caller knows that no row has a top-k or top-p cut, and the three launches
    that search for them are left out (``top_k`` and ``top_p`` are then not read).
    """
    _dev(logits, temperature, top_k, top_p, uniform)
    _need(logits.dim() == 2 and logits.dtype is torch.float32 and logits.stride(1) == 1, "logits must be float32 [S, V]")
    s, v = logits.shape
    for name, x, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("uniform", uniform, torch.float32)):
        _need(x.dtype is dt and x.is_contiguous() and x.numel() == s, f"{name} must be {dt} [S]")
    if workspace is None:
        workspace = torch.empty((s, v), dtype=torch.float32, device=logits.device)
    _need(workspace.dtype is torch.float32 and workspace.is_contiguous() and workspace.numel() >= s * v,
          "sample: workspace too small")
    out = torch.empty((2, s), dtype=torch.float32, device=logits.device)
    ld = logits.stride(0) if s > 1 else v
    if split and v <= SPLIT_MAX_VOCAB:
        lib = core()
        lib.atoma_sample_split_scratch_bytes.restype = ctypes.c_size_t
        scratch = torch.empty((int(lib.atoma_sample_split_scratch_bytes(s)) + 3) // 4, dtype=torch.int32,
                              device=logits.device)
        _check(lib.atoma_sample_split(_p(logits), ld, s, v, _p(temperature), _p(top_k), _p(top_p), _p(uniform),
                                      _p(workspace), _p(scratch), 1 if cuts else 0, _p(out[0]), _p(out[1]), _stream()),
               "sample (split)")
        return out
    _check(core().atoma_sample(_p(logits), ld, s, v, _p(temperature), _p(top_k),
                               _p(top_p), _p(uniform), _p(workspace), _p(out[0]), _p(out[1]), _stream()), "sample")
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, workspace: Optional[torch.Tensor] = None, split: bool = False, cuts: bool = True):
    """``sample_packed`` as (tokens int32 [S], logits of the chosen tokens float32 [S])."""
    out = sample_packed(logits, temperature, top_k, top_p, uniform, workspace, split, cuts)
    return out[0].view(torch.int32), out[1]


def repeat_penalty(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, penalty: torch.Tensor) -> None:
    """In place: for each pair (rows[i], tokens[i]) the logit is divided (if >= 0) or multiplied by penalty[row]."""
    _dev(logits, rows, tokens, penalty)
    _need(logits.dim() == 2 and logits.dtype is torch.float32 and logits.stride(1) == 1, "logits must be float32 [S, V]")
    n = rows.numel()
    _i32(rows, "rows")
    _i32(tokens, "tokens", n)
    _need(penalty.dtype is torch.float32 and penalty.numel() == logits.shape[0], "penalty must be float32 [S]")
    _check(core().atoma_repeat_penalty(_p(logits), logits.stride(0), _p(rows), _p(tokens), _p(penalty), n, _stream()),
           "repeat_penalty")


def feed_tokens(dst: torch.Tensor, src: torch.Tensor, pairs: torch.Tensor) -> None:
    """dst[pairs[i, 0]] = src[pairs[i, 1]] for int32 device tensors; the caller guarantees the indices' ranges."""
    _dev(dst, src, pairs)
    _i32(dst, "dst")
    _i32(src, "src")
    _need(pairs.dtype is torch.int32 and pairs.is_contiguous() and pairs.dim() == 2 and pairs.shape[1] == 2,
          "pairs must be contiguous int32 [n, 2]")
    _check(core().atoma_feed_tokens(_p(dst), _p(src), _p(pairs), pairs.shape[0], _stream()), "feed_tokens")


def measure_device_peaks(device: Optional[torch.device] = None, size_bytes: int = 1 << 30) -> dict:
    """What the GPU delivers, measured with the probes of ``microbench.hip``: GB/s of a read stream and of a copy
    (bytes read plus bytes written) over device memory, and TFLOP/s of a loop of bfloat16 MFMAs.

    The read stream is the yardstick that no kernel of this repository may beat, so it is the best of a sweep: 4, 8
    and 16 loads of 16 bytes in flight a thread, 4 to 32 workgroups a CU, over ``size_bytes`` and over four times as
    much (``hbm_read_how`` says which won)."""
    lib = load_hip_module("microbench")
    dev = device or torch.device("cuda:0")
    big = 4 * size_bytes
    src = torch.empty(big, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty(size_bytes, dtype=torch.uint8, device=dev)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count

    def best(launch, reps=5):
        launch()
        torch.cuda.synchronize(dev)
        times = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            launch()
            b.record()
            torch.cuda.synchronize(dev)
            times.append(a.elapsed_time(b) * 1e-3)
        return min(times)

    out = {}
    with torch.cuda.device(dev):
        reads = []
        for nbytes in (size_bytes, big):
            for per_cu in (4, 8, 16, 32):
                for u in (4, 8, 16):
                    t = best(lambda: _check(lib.atoma_probe_read(_p(src), ctypes.c_size_t(nbytes), cus * per_cu, u,
                                                                 _p(sink), _stream()), "probe_read"), reps=3)
                    reads.append((nbytes / t / 1e9, f"{nbytes >> 20} MiB, {per_cu} workgroups a CU, {u} loads in flight"))
        copy = min(best(lambda g=g: _check(lib.atoma_probe_copy(_p(src), _p(dst), ctypes.c_size_t(size_bytes), g,
                                                                 _stream()), "probe_copy")) for g in (cus * 8, cus * 16))
        iters, grid = 20000, cus * 8
        mfma = best(lambda: _check(lib.atoma_probe_mfma(iters, grid, _p(sink), _stream()), "probe_mfma"), reps=3)
    rate, how = max(reads)
    out["hbm_read_gbs"] = round(rate, 1)
    out["hbm_read_how"] = how
    out["hbm_copy_gbs"] = round(2 * size_bytes / copy / 1e9, 1)
    out["mfma_bf16_tflops"] = round(grid * 4 * iters * 4 * 2 * 32 * 32 * 16 / mfma / 1e12, 1)
    return out


def measure_chain_floors(device: Optional[torch.device] = None) -> dict:
    """What a chain of dependent kernels costs on this GPU beyond its bytes, in microseconds a kernel (the probes of
    ``microbench.hip``, each launched 32 times in a row inside one graph, every launch over other memory, so that
    nothing comes from a cache): an empty kernel behind another; a read stream of 8, 16, 32 and 64 MB (the sizes of a
    decode step's weight matrices); and a barrier over a grid of one workgroup a CU inside one kernel, which is what
    a persistent kernel would pay where the chain pays a launch."""
    lib = load_hip_module("microbench")
    dev = device or torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    n = 32
    out = {}
    with torch.cuda.device(dev):
        src = torch.empty(n * (64 << 20), dtype=torch.uint8, device=dev).random_(0, 255)
        sink = torch.zeros(4, dtype=torch.float32, device=dev)
        base = src.data_ptr()

        def chain(nbytes: int) -> float:
            def launches():
                for i in range(n):
                    _check(lib.atoma_probe_read(ctypes.c_void_p(base + i * (64 << 20)), ctypes.c_size_t(nbytes), cus * 2,
                                                4, _p(sink), _stream()), "probe_read")
            launches()
            torch.cuda.synchronize(dev)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                launches()
            graph.replay()
            torch.cuda.synchronize(dev)
            best = float("inf")
            for _ in range(4):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                graph.replay()
                b.record()
                torch.cuda.synchronize(dev)
                best = min(best, a.elapsed_time(b) * 1e3 / n)
            return round(best, 2)

        out["empty_kernel_us"] = chain(0)
        for mb in (8, 16, 32, 64):
            out[f"read_{mb}mb_us"] = chain(mb << 20)
        nb = 2000
        best = float("inf")
        for _ in range(3):
            ctrl = torch.zeros(128, dtype=torch.int32, device=dev)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            _check(lib.atoma_probe_barrier(_p(ctrl), cus, nb, _stream()), "probe_barrier")
            b.record()
            torch.cuda.synchronize(dev)
            if int(ctrl[64]) != 0:
                raise KernelError("probe_barrier: a wait ran out (the grid was not resident at once)")
            best = min(best, a.elapsed_time(b) * 1e3 / nb)
        out["grid_barrier_us"] = round(best, 2)
    return out
