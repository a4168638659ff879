// Row-wise kernels: embedding gather, fused residual-add + RMSNorm, rotary encoding fused with the
// write of keys and values into the paged cache, SiLU(gate)*up.  All arithmetic is float32; element
// types only decide how values are read and stored.
#include "common.h"

using namespace atoma;

// ---------------------------------------------------------------------------------------------
// Embedding gather into the float32 residual stream: out[t, :] = table[token[t], :].
// Reference: models/src/llama.rs:470 (candle Embedding).
template <typename TW>
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const TW* __restrict__ table,
                             float* __restrict__ out, int width) {
  const int t = blockIdx.x;
  const size_t src = (size_t)tokens[t] * width, dst = (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[dst + i] = to_f32(table[src + i]);
}

extern "C" int atoma_embed(const int32_t* tokens, const void* table, int table_dtype, float* out, int n_tokens,
                           int width, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  dim3 grid(n_tokens), block(256);
  if (table_dtype == kF32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, tokens, (const float*)table, out, width);
  else if (table_dtype == kBF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, tokens, (const bf16_t*)table, out, width);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// resid += delta; out = resid * rsqrt(mean(resid^2) + eps) * w.
// delta may come as several planes [planes][rows][width] (the slices of a K-split product); they are added in
// order of their index.  One block per row.  With `rows`, block r reads row rows[r], leaves resid untouched and writes out row r.
// The sum of squares is reduced in an order fixed by (width, block size) alone.
// Reference: models/src/llama.rs:401-408 (norm placement and residual sums), :416-421 (eps).
template <typename TD, typename TW, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                   const TW* __restrict__ w, TO* __restrict__ out,
                                   const int32_t* __restrict__ rows, int width, float eps, int planes,
                                   size_t plane_stride) {
  __shared__ float scratch[4];
  const int r = blockIdx.x;
  const size_t src = (size_t)(rows ? rows[r] : r) * width, dst = (size_t)r * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    float v = resid[src + i];
    if (delta) {
      for (int p = 0; p < planes; ++p) v += to_f32(delta[p * plane_stride + src + i]);
      if (!rows) resid[src + i] = v;
    }
    ss += v * v;
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += 256) {
    float v = resid[src + i];
    if (delta && rows)
      for (int p = 0; p < planes; ++p) v += to_f32(delta[p * plane_stride + src + i]);
    out[dst + i] = from_f32<TO>(v * inv * to_f32(w[i]));
  }
}

template <typename TD, typename TW>
static int add_rmsnorm_out(float* resid, const TD* delta, const TW* w, void* out, int out_dtype, const int32_t* rows,
                           int n_rows, int width, float eps, int planes, size_t plane_stride,
                           hipStream_t stream) {
  dim3 grid(n_rows), block(256);
  if (out_dtype == kF32)
    hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TW, float>), grid, block, 0, stream, resid, delta, w, (float*)out,
                       rows, width, eps, planes, plane_stride);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TW, bf16_t>), grid, block, 0, stream, resid, delta, w,
                       (bf16_t*)out, rows, width, eps, planes, plane_stride);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <typename TD>
static int add_rmsnorm_w(float* resid, const TD* delta, const void* w, int w_dtype, void* out, int out_dtype,
                         const int32_t* rows, int n_rows, int width, float eps, int planes, size_t plane_stride,
                           hipStream_t stream) {
  if (w_dtype == kF32)
    return add_rmsnorm_out<TD, float>(resid, delta, (const float*)w, out, out_dtype, rows, n_rows, width, eps, planes, plane_stride, stream);
  if (w_dtype == kBF16)
    return add_rmsnorm_out<TD, bf16_t>(resid, delta, (const bf16_t*)w, out, out_dtype, rows, n_rows, width, eps,
                                       planes, plane_stride, stream);
  return ATOMA_ERR_DTYPE;
}

extern "C" int atoma_add_rmsnorm(float* resid, const void* delta, int delta_dtype, const void* w, int w_dtype,
                                 void* out, int out_dtype, const int32_t* rows, int n_rows, int width, float eps,
                                 int planes, size_t plane_stride, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (delta_dtype == kF32)
    return add_rmsnorm_w<float>(resid, (const float*)delta, w, w_dtype, out, out_dtype, rows, n_rows, width, eps,
                                planes, plane_stride, stream);
  if (delta_dtype == kBF16)
    return add_rmsnorm_w<bf16_t>(resid, (const bf16_t*)delta, w, w_dtype, out, out_dtype, rows, n_rows, width, eps,
                                 planes, plane_stride, stream);
  return ATOMA_ERR_DTYPE;
}

// ---------------------------------------------------------------------------------------------
// Rotary encoding of q and k in half-split pairs (i, i + rd/2), and the write of k (rotated) and v into the
// paged cache.  qkv is [T, row_stride]: q heads, then k heads, then v heads, each head hd wide.
// q is rotated in place.  K pages are [page][kv_head][slot][hd]; V pages are [page][kv_head][hd][slot], so that
// the attention kernels read keys along hd and values along the slot axis contiguously.
// A negative slot, or null caches, skip the cache write (the reference skips negative slots:
// csrc/kernels/cache_manager.cu:151-155).  cos/sin may be null: then nothing is rotated.
// Pairing and signs: csrc/kernels/rotary.h:116-131; rotation applies to q and k only: models/src/llama.rs:298-299.
template <typename TA, typename TC>
__global__ void rope_cache_write_kernel(TA* __restrict__ qkv, int row_stride, const int32_t* __restrict__ positions,
                                        const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                        int rotary_dim, TC* __restrict__ kcache, TC* __restrict__ vcache,
                                        const int32_t* __restrict__ slot_mapping, int page_size, int nh, int nkv,
                                        int hd) {
  const int t = blockIdx.x;
  TA* row = qkv + (size_t)t * row_stride;
  const int half = rotary_dim / 2;
  const int slot = (kcache && slot_mapping) ? slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const float* cs = cos_t ? cos_t + (size_t)positions[t] * half : nullptr;
  const float* sn = sin_t ? sin_t + (size_t)positions[t] * half : nullptr;

  // rotated pairs of q and k
  const int n_rot = cs ? (nh + nkv) * half : 0;
  for (int it = threadIdx.x; it < n_rot; it += blockDim.x) {
    const int head = it / half, i = it % half;
    TA* x = row + (size_t)head * hd;
    const float x1 = to_f32(x[i]), x2 = to_f32(x[i + half]);
    const float c = cs[i], s = sn[i];
    const float o1 = x1 * c - x2 * s, o2 = x2 * c + x1 * s;
    if (head < nh) {
      x[i] = from_f32<TA>(o1);
      x[i + half] = from_f32<TA>(o2);
    } else if (slot >= 0) {
      const int kvh = head - nh;
      TC* dst = kcache + (((size_t)page * nkv + kvh) * page_size + off) * hd;
      dst[i] = from_f32<TC>(o1);
      dst[i + half] = from_f32<TC>(o2);
    }
  }
  if (slot < 0) return;
  // the part of k that is not rotated (all of it without tables)
  const int rd = cs ? rotary_dim : 0;
  const int tail = hd - rd;
  for (int it = threadIdx.x; it < nkv * tail; it += blockDim.x) {
    const int kvh = it / tail, i = rd + it % tail;
    kcache[(((size_t)page * nkv + kvh) * page_size + off) * hd + i] =
        from_f32<TC>(to_f32(row[(size_t)(nh + kvh) * hd + i]));
  }
  // v, transposed inside the page
  for (int it = threadIdx.x; it < nkv * hd; it += blockDim.x) {
    const int kvh = it / hd, i = it % hd;
    vcache[(((size_t)page * nkv + kvh) * hd + i) * page_size + off] =
        from_f32<TC>(to_f32(row[(size_t)(nh + nkv + kvh) * hd + i]));
  }
}

extern "C" int atoma_rope_cache_write(void* qkv, int act_dtype, int row_stride, const int32_t* positions,
                                      const float* cos_t, const float* sin_t, int rotary_dim, void* kcache,
                                      void* vcache, int cache_dtype, const int32_t* slot_mapping, int page_size,
                                      int n_tokens, int nh, int nkv, int hd, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (rotary_dim < 0 || rotary_dim > hd || (rotary_dim & 1) || row_stride < (nh + 2 * nkv) * hd || page_size <= 0)
    return ATOMA_ERR_SHAPE;
  dim3 grid(n_tokens), block(256);
#define ATOMA_ROPE(TA, TC)                                                                                        \
  hipLaunchKernelGGL((rope_cache_write_kernel<TA, TC>), grid, block, 0, stream, (TA*)qkv, row_stride, positions, \
                     cos_t, sin_t, rotary_dim, (TC*)kcache, (TC*)vcache, slot_mapping, page_size, nh, nkv, hd)
  if (act_dtype == kF32 && cache_dtype == kF32) ATOMA_ROPE(float, float);
  else if (act_dtype == kBF16 && cache_dtype == kBF16) ATOMA_ROPE(bf16_t, bf16_t);
  else if (act_dtype == kF32 && cache_dtype == kBF16) ATOMA_ROPE(float, bf16_t);
  else if (act_dtype == kBF16 && cache_dtype == kF32) ATOMA_ROPE(bf16_t, float);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_ROPE
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i], silu(z) = z * sigmoid(z).
// Reference: models/src/llama.rs:364.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inter;
    const int i = (int)(idx % inter);
    const float g = to_f32(gu[t * 2 * inter + i]), u = to_f32(gu[t * 2 * inter + inter + i]);
    out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
  }
}

extern "C" int atoma_swiglu(const void* gu, void* out, int dtype, int n_tokens, int inter, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  const size_t total = (size_t)n_tokens * inter;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 65536) blocks = 65536;
  if (dtype == kF32)
    hipLaunchKernelGGL(swiglu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gu, (float*)out, inter,
                       total);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)gu, (bf16_t*)out,
                       inter, total);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}
