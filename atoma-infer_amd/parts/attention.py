"""Causal self-attention over the paged cache, with grouped KV heads and an optional window.

Projections without bias (models/src/llama.rs:269-271, 311, 322-325), head split by columns (:273-296), rotation
of q and k (:298-299), keys and values written to the cache before attention (models/src/flash_attention.rs:
360-361), softmax scale 1/sqrt(head size) (models/src/llama.rs:342), query head h on KV head h // (nh/nkv)
(csrc/kernels/flash_fwd_kernel.h:593).  Where the reference runs separate kernels for prompt rows and decode rows
(models/src/flash_attention.rs:380-466), one rule serves here: a token at position p sees keys 0..p (or the
last ``window`` of them) of its own request through the block table.

The three projection matrices are fused into one [(nh + 2 nkv) hd, width] matrix at load time; results equal
the separate products.  When the position encoding rotates whole heads in half-split pairs (i, i + hd/2), the rows
of every q and k head are reordered at load time so that a pair's members leave the projection as neighbours
(2i, 2i + 1): then the projection's own epilogue can rotate q and k and write k and v into the cache, and decode
steps need no kernel between the projection and attention.  Rotated q and cached k are always in their own column
order, whoever rotated them, so any call may read any call's cache.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import CacheSpec, Mixer, PositionEncoding, WeightSpec, register_mixer
from .linear import as_tensor, linear, linear_delta


class PagedAttention(Mixer):
    def __init__(self, width: int, num_heads: int, num_kv_heads: int, head_size: int,
                 position: Optional[PositionEncoding] = None, window: Optional[int] = None,
                 scale: Optional[float] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot be grouped over {num_kv_heads} KV heads")
        # every multiple of 8 up to 256, as the reference's kernels take (csrc/src/lib.rs:136-143, 790)
        if head_size % 8 or not 8 <= head_size <= 256:
            raise ValueError(f"head size {head_size} is not supported: the attention kernels take multiples of 8 "
                             f"from 8 to 256")
        if window is not None and window <= 0:
            raise ValueError("window must be positive")
        self.width, self.nh, self.nkv, self.hd = int(width), int(num_heads), int(num_kv_heads), int(head_size)
        self.position = position
        self.window = window
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.hd)
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.w_qkv_tiled = self.w_o_tiled = None
        self.act_dtype = torch.float32
        self.paired = False      # q and k columns in pair order (set at load time)
        self.slopes: Optional[torch.Tensor] = None      # per-head bias of the scores by distance, if the encoding has one

    # -- declaration ----------------------------------------------------------------------------------
    def graph_safe(self) -> bool:
        # the kernels take the step from device tensors and from the plan made before the step is recorded
        return self.position is None or self.position.graph_safe()

    def weight_specs(self) -> Dict[str, WeightSpec]:
        q, kv = self.nh * self.hd, self.nkv * self.hd
        return {"q_proj.weight": WeightSpec((q, self.width)), "k_proj.weight": WeightSpec((kv, self.width)),
                "v_proj.weight": WeightSpec((kv, self.width)), "o_proj.weight": WeightSpec((self.width, q))}

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.nkv, self.hd, self.window)

    def load(self, get, device, act_dtype) -> None:
        ws = [get("q_proj.weight"), get("k_proj.weight"), get("v_proj.weight")]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        if self.position is not None:
            self.position.load(get, device, act_dtype)
        tables = self.position.rotary_tables() if self.position is not None else None
        self.slopes = self.position.score_slopes(self.nh) if self.position is not None else None
        if self.slopes is not None:
            self.slopes = self.slopes.to(device=device, dtype=torch.float32).contiguous()
            if self.slopes.numel() != self.nh:
                raise ValueError(f"score_slopes gave {self.slopes.numel()} slopes for {self.nh} heads")
        self.paired = tables is not None and tables[2] == self.hd
        if self.paired:
            half = self.hd // 2
            order = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1)   # 0, half, 1, ...
            ws[0] = ws[0].reshape(self.nh, self.hd, self.width)[:, order].reshape(self.nh * self.hd, self.width)
            ws[1] = ws[1].reshape(self.nkv, self.hd, self.width)[:, order].reshape(self.nkv * self.hd, self.width)
        self.w_qkv = torch.cat([w.to(device=device, dtype=dt) for w in ws], dim=0).contiguous()
        self.w_o = get("o_proj.weight").to(device).contiguous()
        self.act_dtype = act_dtype
        # second copies in the order in which the kernels of steps of few rows read them
        self.w_qkv_tiled = self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_qkv.dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            if self.paired:
                self.w_qkv_tiled = gemm_bf16.tile_copies_rope(self.w_qkv)
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_qkv, self.w_o))

    def step_planner(self, page_size: int, cache_dtype: torch.dtype):
        """(key, fn(starts, counts, bucket_tokens) -> (int32 array, meta)): the task list of the MFMA attention
        kernels, built once per step on the host and shipped with the step's metadata.  ``bucket_tokens`` is None, or
        for a step that only decodes the context length its plan must serve (a multiple of the runner's bucket)."""
        from ..kernels import attention_bf16
        if self.slopes is not None:
            return None          # scores with a bias take the general kernel, which needs no plan
        if cache_dtype is torch.bfloat16 and self.hd % 16:
            import warnings
            warnings.warn(f"bfloat16 attention with heads of {self.hd} columns runs the general kernel (one wave per "
                          f"token and head), many times slower than the matrix-core kernel, which takes head sizes "
                          f"that are multiples of 16", stacklevel=2)
            return None
        if cache_dtype is torch.bfloat16 and not attention_bf16.page_ok(page_size):
            import warnings
            warnings.warn(f"bfloat16 attention with pages of {page_size} tokens runs the general kernel (one wave per "
                          f"token and head), many times slower than the matrix-core kernel, which needs pages of a "
                          f"multiple of 16 tokens ([cache] block_size = 16, 32, 64, ...)", stacklevel=2)
        if cache_dtype is not torch.bfloat16 or not attention_bf16.page_ok(page_size):
            return None
        group, window, nkv = self.nh // self.nkv, self.window or 0, self.nkv
        cus = torch.cuda.get_device_properties(self.w_qkv.device).multi_processor_count
        return (attention_bf16.plan_key(group, window, nkv, self.hd),
                lambda starts, counts, bucket: attention_bf16.build_tasks(
                    starts, counts, group, window, bucket, kv_heads=nkv,
                    max_waves=attention_bf16.max_waves_for(self.hd),
                    row_tiles=attention_bf16.max_row_tiles_for(self.hd), head_size=self.hd, compute_units=cus))

    # -- execution ------------------------------------------------------------------------------------
    accepts_begun = True
    takes_sink = True

    def forward(self, x, ctx, cache, sink=None):
        nh, nkv, hd = self.nh, self.nkv, self.hd
        t = x.shape[0]
        writes = cache.writable
        # a call that reads another call's cache needs its queries only
        w = self.w_qkv if writes else self.w_qkv[: nh * hd]
        k_cache, v_cache = cache.k, cache.v
        tables = self.position.rotary_tables() if self.position is not None else None
        qkv = None
        if self.paired and writes and x.dtype is torch.bfloat16 and w.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            qkv = gemm_bf16.try_linear_rope(x, w, ctx.positions, tables[0], tables[1], k_cache, v_cache,
                                            cache.slot_mapping, cache.page_size, nh, nkv, hd,
                                            tiled=self.w_qkv_tiled)
        if qkv is None:
            x = as_tensor(x)
        if qkv is not None:
            pass        # rotated and stored by the product's epilogue
        elif tables is not None or self.position is None:
            raw = linear(x, w)
            cos, sin, rd = tables if tables is not None else (None, None, 0)
            # pair order in, own order out: q cannot be rotated in place then
            qkv = torch.empty((t, nh * hd), dtype=raw.dtype, device=raw.device) if self.paired else raw
            q_out = qkv if self.paired else None
            if writes:
                ops.rope_cache_write(raw, ctx.positions, cos, sin, rd, k_cache, v_cache, cache.slot_mapping,
                                     cache.page_size, nh, nkv, hd, q_out)
            else:
                ops.rope_cache_write(raw, ctx.positions, cos, sin, rd, None, None, None, 1, nh, 0, hd, q_out)
        else:
            qkv = linear(x, w)
            q = qkv[:, : nh * hd].view(t, nh, hd)
            if writes:
                k = qkv[:, nh * hd: (nh + nkv) * hd].view(t, nkv, hd)
                self.position.apply(q, k, ctx.positions)
                ops.rope_cache_write(qkv, ctx.positions, None, None, 0, k_cache, v_cache, cache.slot_mapping,
                                     cache.page_size, nh, nkv, hd)
            else:
                self.position.apply(q, q[:, :0], ctx.positions)
        out = torch.empty((t, nh * hd), dtype=qkv.dtype, device=qkv.device)
        self.attend(qkv, k_cache, v_cache, out, ctx, cache)
        return linear_delta(out, self.w_o, sink, self.w_o_tiled)

    def attend(self, q, k_cache, v_cache, out, ctx, cache) -> None:
        if self.slopes is None and q.dtype is torch.bfloat16 and k_cache.dtype is torch.bfloat16:
            from ..kernels import attention_bf16
            if attention_bf16.try_attention(q, k_cache, v_cache, out, ctx, cache, self.scale, self.window or 0,
                                            self.nh, self.nkv, self.hd):
                return
        ops.paged_attention_generic(q, k_cache, v_cache, out, cache.block_tables, ctx.token_seq, ctx.positions,
                                    self.scale, self.window or 0, cache.page_size, self.nh, self.nkv, self.hd,
                                    self.slopes)


register_mixer("attention", PagedAttention)
