// Row-wise kernels: embedding gather, fused residual-add + RMSNorm, rotary encoding fused with the
// write of keys and values into the paged cache, SiLU(gate)*up.  All arithmetic is float32; element
// types only decide how values are read and stored.
#include "common.h"
#include "cache_layout.h"

using namespace atoma;

// four neighbouring values at a time
struct f4 { float v[4]; };
__device__ __forceinline__ f4 load4(const float* p) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  return f4{{t.x, t.y, t.z, t.w}};
}
__device__ __forceinline__ f4 load4(const bf16_t* p) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  return f4{{bf16_bits_to_f32((uint16_t)(t.x & 0xffff)), bf16_bits_to_f32((uint16_t)(t.x >> 16)),
             bf16_bits_to_f32((uint16_t)(t.y & 0xffff)), bf16_bits_to_f32((uint16_t)(t.y >> 16))}};
}
__device__ __forceinline__ void store4(float* p, const f4& a) {
  *reinterpret_cast<float4*>(p) = make_float4(a.v[0], a.v[1], a.v[2], a.v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const f4& a) {
  uint2 t;
  t.x = (uint32_t)f32_to_bf16_bits(a.v[0]) | ((uint32_t)f32_to_bf16_bits(a.v[1]) << 16);
  t.y = (uint32_t)f32_to_bf16_bits(a.v[2]) | ((uint32_t)f32_to_bf16_bits(a.v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = t;
}

// ---------------------------------------------------------------------------------------------
// Embedding gather into the float32 residual stream: out[t, :] = table[token[t], :].
// Tokens that the host has not seen (fed from the sampler on the device) are checked here: an id outside the table
// reads nothing and leaves a row of NaN, which shows in that request's logits and in nobody else's.
// Reference: models/src/llama.rs:470 (candle Embedding).
template <typename TW>
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const TW* __restrict__ table,
                             float* __restrict__ out, int width, int vocab) {
  const int t = blockIdx.x;
  const int token = tokens[t];
  const size_t dst = (size_t)t * width;
  if (token < 0 || token >= vocab) {
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[dst + i] = __int_as_float(0x7fc00000);
    return;
  }
  const size_t src = (size_t)token * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[dst + i] = to_f32(table[src + i]);
}

extern "C" int atoma_embed(const int32_t* tokens, const void* table, int table_dtype, float* out, int n_tokens,
                           int width, int vocab, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  dim3 grid(n_tokens), block(256);
  if (table_dtype == kF32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, tokens, (const float*)table, out, width, vocab);
  else if (table_dtype == kBF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, tokens, (const bf16_t*)table, out, width,
                       vocab);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// A norm begun by the kernel that makes the residual row and finished by the product that reads it (decode steps of
// at most 16 rows; the products are in gemm_bf16.hip).  "Begun" is: u = residual * norm weight, as bfloat16, and the
// row's sum of squares in shares ss [parts][16]; "finished" is the division by sqrt(sum / width + eps).

// Embedding gather with the first norm begun: resid [T][width] float32, u [T][width] bfloat16, ss [1][16].
// One block of 256 threads per row, 16 blocks: those beyond T only clear their share.  Four columns a thread at a
// time where the row allows 8- and 16-byte accesses (VEC), one otherwise.
template <typename TW, typename TG, bool VEC>
__global__ void __launch_bounds__(256)
embed_begin_norm_kernel(const int32_t* __restrict__ tokens, const TW* __restrict__ table, float* __restrict__ resid,
                        const TG* __restrict__ gamma, bf16_t* __restrict__ u, float* __restrict__ ss, int n_tokens,
                        int width, int vocab) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  if (t >= n_tokens) {
    if (threadIdx.x == 0) ss[t] = 0.f;
    return;
  }
  const int token = tokens[t];
  const bool ok = token >= 0 && token < vocab;
  const size_t dst = (size_t)t * width, src = (size_t)(ok ? token : 0) * width;
  const float nan = __int_as_float(0x7fc00000);
  float sq = 0.f;
  if (VEC) {
    for (int i = 4 * threadIdx.x; i < width; i += 1024) {
      f4 v = load4(table + src + i);
      const f4 g = load4(gamma + i);
      f4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (!ok) v.v[j] = nan;
        o.v[j] = v.v[j] * g.v[j];
        sq += v.v[j] * v.v[j];
      }
      store4(resid + dst + i, v);
      store4(u + dst + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < width; i += 256) {
      const float v = ok ? to_f32(table[src + i]) : nan;
      resid[dst + i] = v;
      u[dst + i] = from_f32<bf16_t>(v * to_f32(gamma[i]));
      sq += v * v;
    }
  }
  sq = block_sum<4>(sq, scratch);
  if (threadIdx.x == 0) ss[t] = sq;
}

extern "C" int atoma_embed_begin_norm(const int32_t* tokens, const void* table, int table_dtype, float* resid,
                                      const void* gamma, int gamma_dtype, void* u, float* ss, int n_tokens, int width,
                                      int vocab, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (n_tokens > 16) return ATOMA_ERR_SHAPE;
  const bool vec = width % 4 == 0 && (((uintptr_t)table | (uintptr_t)gamma | (uintptr_t)resid | (uintptr_t)u) & 15) == 0;
#define ATOMA_EBN(TW, TG)                                                                                           \
  do {                                                                                                              \
    if (vec)                                                                                                        \
      hipLaunchKernelGGL((embed_begin_norm_kernel<TW, TG, true>), dim3(16), dim3(256), 0, stream, tokens,           \
                         (const TW*)table, resid, (const TG*)gamma, (bf16_t*)u, ss, n_tokens, width, vocab);        \
    else                                                                                                            \
      hipLaunchKernelGGL((embed_begin_norm_kernel<TW, TG, false>), dim3(16), dim3(256), 0, stream, tokens,          \
                         (const TW*)table, resid, (const TG*)gamma, (bf16_t*)u, ss, n_tokens, width, vocab);        \
  } while (0)
  if (table_dtype == kF32 && gamma_dtype == kF32) ATOMA_EBN(float, float);
  else if (table_dtype == kF32 && gamma_dtype == kBF16) ATOMA_EBN(float, bf16_t);
  else if (table_dtype == kBF16 && gamma_dtype == kF32) ATOMA_EBN(bf16_t, float);
  else if (table_dtype == kBF16 && gamma_dtype == kBF16) ATOMA_EBN(bf16_t, bf16_t);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_EBN
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// out [T][width] = u [T][width] / sqrt(sum_p ss[p][row] / width + eps), both bfloat16: the finished norm as a tensor,
// for a reader that cannot finish it itself.
__global__ void __launch_bounds__(256)
finish_norm_kernel(const uint16_t* __restrict__ u, const float* __restrict__ ss, int parts, float eps,
                   uint16_t* __restrict__ out, int width) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  float s = 0.f;
  for (int p = threadIdx.x; p < parts; p += 256) s += ss[(size_t)p * 16 + t];
  s = block_sum<4>(s, scratch);
  const float scale = 1.0f / sqrtf(s / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += 256)
    out[(size_t)t * width + i] = f32_to_bf16_bits(bf16_bits_to_f32(u[(size_t)t * width + i]) * scale);
}

extern "C" int atoma_finish_norm(const void* u, const float* ss, int parts, float eps, void* out, int n_rows,
                                 int width, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (n_rows > 16 || parts <= 0 || width <= 0) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(finish_norm_kernel, dim3(n_rows), dim3(256), 0, stream, (const uint16_t*)u, ss, parts, eps,
                     (uint16_t*)out, width);
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

// The same for rows of at most 4096 columns, a multiple of 4, with 16-byte aligned rows: every thread keeps its
// values in registers between the two passes and all loads of a pass are issued together.
// MAXJ: pieces of four columns a thread (1, 2 or 4: rows of up to 1024, 2048, 4096 columns).
template <typename TD, typename TW, typename TO, int MAXJ>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(float* __restrict__ resid, const TD* __restrict__ delta, const TW* __restrict__ w,
                       TO* __restrict__ out, const int32_t* __restrict__ rows, int width, float eps, int planes,
                       size_t plane_stride) {
  __shared__ float scratch[4];
  const int r = blockIdx.x;
  const size_t src = (size_t)(rows ? rows[r] : r) * width, dst = (size_t)r * width;
  const int n4 = width >> 2;
  f4 v[MAXJ];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    const int c = threadIdx.x + j * 256;
    if (c < n4) v[j] = load4(resid + src + 4 * c);
  }
  if (delta) {
    // the planes of a K-split product: the loads of up to eight planes are issued together (each is a trip to memory,
    // and a plane at a time would make as many trips as there are planes); they are added in the order of their index
    constexpr int PB = MAXJ <= 2 ? 8 : 4;
    for (int p0 = 0; p0 < planes; p0 += PB) {
      f4 d[PB][MAXJ];
#pragma unroll
      for (int q = 0; q < PB; ++q) {
        const int p = p0 + q < planes ? p0 + q : planes - 1;
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
          const int c = threadIdx.x + j * 256;
          if (c < n4) d[q][j] = load4(delta + p * plane_stride + src + 4 * c);
        }
      }
#pragma unroll
      for (int q = 0; q < PB; ++q) {
        if (p0 + q < planes) {
#pragma unroll
          for (int j = 0; j < MAXJ; ++j) {
            const int c = threadIdx.x + j * 256;
            if (c < n4)
#pragma unroll
              for (int i = 0; i < 4; ++i) v[j].v[i] += d[q][j].v[i];
          }
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    const int c = threadIdx.x + j * 256;
    if (c < n4) {
      if (delta && !rows) store4(resid + src + 4 * c, v[j]);
#pragma unroll
      for (int i = 0; i < 4; ++i) ss += v[j].v[i] * v[j].v[i];
    }
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int j = 0; j < MAXJ; ++j) {
    const int c = threadIdx.x + j * 256;
    if (c < n4) {
      const f4 wv = load4(w + 4 * c);
      f4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o.v[i] = v[j].v[i] * inv * wv.v[i];
      store4(out + dst + 4 * c, o);
    }
  }
}

template <typename TD, typename TW>
static int add_rmsnorm_out(float* resid, const TD* delta, const TW* w, void* out, int out_dtype, const int32_t* rows,
                           int n_rows, int width, float eps, int planes, size_t plane_stride,
                           hipStream_t stream) {
  dim3 grid(n_rows), block(256);
  const bool vec = width % 4 == 0 && width <= 4096 && ((uintptr_t)resid & 15) == 0 && ((uintptr_t)delta & 15) == 0 &&
                   ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0 && plane_stride % 4 == 0;
#define ATOMA_NORM_VEC(TO_)                                                                                         \
  do {                                                                                                             \
    if (width <= 1024)                                                                                             \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TW, TO_, 1>), grid, block, 0, stream, resid, delta, w,        \
                         (TO_*)out, rows, width, eps, planes, plane_stride);                                       \
    else if (width <= 2048)                                                                                        \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TW, TO_, 2>), grid, block, 0, stream, resid, delta, w,        \
                         (TO_*)out, rows, width, eps, planes, plane_stride);                                       \
    else                                                                                                           \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TW, TO_, 4>), grid, block, 0, stream, resid, delta, w,        \
                         (TO_*)out, rows, width, eps, planes, plane_stride);                                       \
  } while (0)
  if (out_dtype == kF32) {
    if (vec)
      ATOMA_NORM_VEC(float);
    else
      hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TW, float>), grid, block, 0, stream, resid, delta, w, (float*)out,
                         rows, width, eps, planes, plane_stride);
  } else if (out_dtype == kBF16) {
    if (vec)
      ATOMA_NORM_VEC(bf16_t);
    else
      hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TW, bf16_t>), grid, block, 0, stream, resid, delta, w,
                         (bf16_t*)out, rows, width, eps, planes, plane_stride);
  } else {
    return ATOMA_ERR_DTYPE;
  }
#undef ATOMA_NORM_VEC
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
// q is rotated in place.  Keys and values go into (page, kv_head) tiles of page_size * hd elements whose inner
// order is that of cache_layout.h (the order in which the MFMA attention kernel reads them).
// A negative slot, or null caches, skip the cache write (the reference skips negative slots:
// csrc/kernels/cache_manager.cu:151-155).  cos/sin may be null: then nothing is rotated.
// Pairing and signs: csrc/kernels/rotary.h:116-131; rotation applies to q and k only: models/src/llama.rs:298-299.
// With `q_out` ([T, q_stride], the whole head rotated): the rows of the q and k projections were reordered at load
// time so that the members of pair i arrive as columns 2i and 2i + 1 of the head (which lets the projection's own
// epilogue rotate, for few rows); the rotated q then goes to q_out and k to the cache in their own column order.
template <typename TA, typename TC>
__global__ void __launch_bounds__(256)
rope_cache_write_kernel(TA* __restrict__ qkv, int row_stride, const int32_t* __restrict__ positions,
                        const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rotary_dim,
                        TC* __restrict__ kcache, TC* __restrict__ vcache, const int32_t* __restrict__ slot_mapping,
                        int page_size, int nh, int nkv, int hd, int heads, TA* __restrict__ q_out, int q_stride) {
  // One thread per item of a token: a rotated pair (or, beyond the rotary dimension, a pair of plain columns)
  // of a q or k head, or two columns of a v head.  `heads` is how many heads of the row are touched.
  const int t = blockIdx.x;
  const int hp = hd >> 1;                       // items per head
  const int item = blockIdx.y * 256 + threadIdx.x;
  if (item >= heads * hp) return;
  const int head = item / hp, i = item % hp;
  TA* x = qkv + (size_t)t * row_stride + (size_t)head * hd;
  const int slot = (kcache && slot_mapping) ? slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  if (head >= nh + nkv) {
    // v: stored transposed inside the page
    if (slot < 0) return;
    TC* tile = vcache + ((size_t)page * nkv + (head - nh - nkv)) * hd * page_size;
    tile[value_offset(2 * i, off, hd, page_size)] = from_f32<TC>(to_f32(x[2 * i]));
    tile[value_offset(2 * i + 1, off, hd, page_size)] = from_f32<TC>(to_f32(x[2 * i + 1]));
    return;
  }
  const bool is_k = head >= nh;
  if (is_k && slot < 0) return;
  TC* ktile = is_k ? kcache + ((size_t)page * nkv + (head - nh)) * page_size * hd : nullptr;
  const int half = cos_t ? rotary_dim / 2 : 0;
  if (i < half) {
    // with q_out, the members of pair i come in as neighbours (2i, 2i + 1) and leave to their own columns
    const int a = q_out ? 2 * i : i, b = q_out ? 2 * i + 1 : i + half;
    const float c = cos_t[(size_t)positions[t] * half + i], sv = sin_t[(size_t)positions[t] * half + i];
    const float x1 = to_f32(x[a]), x2 = to_f32(x[b]);
    const float o1 = x1 * c - x2 * sv, o2 = x2 * c + x1 * sv;
    if (is_k) {
      ktile[key_offset(off, i, page_size)] = from_f32<TC>(o1);
      ktile[key_offset(off, i + half, page_size)] = from_f32<TC>(o2);
    } else {
      TA* y = q_out ? q_out + (size_t)t * q_stride + (size_t)head * hd : x;
      y[i] = from_f32<TA>(o1);
      y[i + half] = from_f32<TA>(o2);
    }
  } else if (is_k) {
    // columns beyond the rotary dimension are copied as they are (all of them without tables)
    const int a = 2 * half + 2 * (i - half);
    ktile[key_offset(off, a, page_size)] = from_f32<TC>(to_f32(x[a]));
    ktile[key_offset(off, a + 1, page_size)] = from_f32<TC>(to_f32(x[a + 1]));
  }
}

// The same for bfloat16 rows and caches with hd % 16 == 0, the whole head rotated and 16-byte aligned rows: a
// thread takes eight neighbouring pairs of a q or k head (two 16-byte loads, and since eight columns of a key are
// one piece of its cache tile, two 16-byte stores).  One block per four tokens: a value tile keeps four
// neighbouring tokens of a column side by side, so when the block's tokens fill four neighbouring slots of a
// page (as a prompt's do), a thread turns four columns of the four tokens into four 8-byte stores.
constexpr int kRopeTokens = 4;

__global__ void __launch_bounds__(256)
rope_cache_write_vec_kernel(uint16_t* __restrict__ qkv, int row_stride, const int32_t* __restrict__ positions,
                            const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                            uint16_t* __restrict__ kcache, uint16_t* __restrict__ vcache,
                            const int32_t* __restrict__ slot_mapping, int page_size, int nh, int nkv, int hd,
                            uint16_t* __restrict__ q_out, int q_stride, int n_tokens) {
  const int t0 = blockIdx.x * kRopeTokens;
  const int nt = n_tokens - t0 < kRopeTokens ? n_tokens - t0 : kRopeTokens;
  const int half = hd >> 1;
  const int per_qk = hd >> 4;                              // items per head
  const int n_qk = (nh + nkv) * per_qk;
  const bool paired = q_out != nullptr;
  // the block's items are dealt over gridDim.y blocks, which keeps the GPU busy when the tokens are few
  const int first = blockIdx.y * 256 + threadIdx.x, stride = gridDim.y * 256;
  for (int item = first; item < nt * n_qk; item += stride) {
    const int t = t0 + item / n_qk, it = item % n_qk;
    const int head = it / per_qk, i0 = (it % per_qk) * 8;
    const bool is_k = head >= nh;
    const int slot = (kcache && slot_mapping) ? slot_mapping[t] : -1;
    if (is_k && slot < 0) continue;
    uint16_t* x = qkv + (size_t)t * row_stride + (size_t)head * hd;
    const size_t pos = (size_t)positions[t];
    // where the eight pairs' members come from: columns i0.. and i0 + half.. (one member in each 16-byte piece), or,
    // with q_out, neighbours 2 i0 .. 2 i0 + 15 (four pairs in each piece); they leave to columns i0.. and i0 + half..
    const uint4 r1 = *reinterpret_cast<const uint4*>(x + (paired ? 2 * i0 : i0));
    const uint4 r2 = *reinterpret_cast<const uint4*>(x + (paired ? 2 * i0 + 8 : i0 + half));
    const f4 c0 = load4(cos_t + pos * half + i0), c1 = load4(cos_t + pos * half + i0 + 4);
    const f4 s0 = load4(sin_t + pos * half + i0), s1 = load4(sin_t + pos * half + i0 + 4);
    const uint16_t* a = reinterpret_cast<const uint16_t*>(&r1);
    const uint16_t* b = reinterpret_cast<const uint16_t*>(&r2);
    uint4 w1, w2;
    uint16_t* o1 = reinterpret_cast<uint16_t*>(&w1);
    uint16_t* o2 = reinterpret_cast<uint16_t*>(&w2);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float c = e < 4 ? c0.v[e] : c1.v[e - 4], sn = e < 4 ? s0.v[e] : s1.v[e - 4];
      const uint16_t m1 = paired ? (e < 4 ? a[2 * e] : b[2 * (e - 4)]) : a[e];
      const uint16_t m2 = paired ? (e < 4 ? a[2 * e + 1] : b[2 * (e - 4) + 1]) : b[e];
      const float x1 = bf16_bits_to_f32(m1), x2 = bf16_bits_to_f32(m2);
      o1[e] = f32_to_bf16_bits(x1 * c - x2 * sn);
      o2[e] = f32_to_bf16_bits(x2 * c + x1 * sn);
    }
    if (is_k) {
      const int page = slot / page_size, off = slot % page_size;
      uint16_t* ktile = kcache + ((size_t)page * nkv + (head - nh)) * page_size * hd;
      *reinterpret_cast<uint4*>(ktile + key_offset(off, i0, page_size)) = w1;
      *reinterpret_cast<uint4*>(ktile + key_offset(off, i0 + half, page_size)) = w2;
    } else {
      uint16_t* y = paired ? q_out + (size_t)t * q_stride + (size_t)head * hd : x;
      *reinterpret_cast<uint4*>(y + i0) = w1;
      *reinterpret_cast<uint4*>(y + i0 + half) = w2;
    }
  }
  if (!kcache || !slot_mapping) return;

  // values: four columns of the block's tokens per thread
  int slots[kRopeTokens];
#pragma unroll
  for (int j = 0; j < kRopeTokens; ++j) slots[j] = j < nt ? slot_mapping[t0 + j] : -1;
  const int off0 = slots[0] >= 0 ? slots[0] % page_size : 0;
  const bool together = nt == kRopeTokens && slots[0] >= 0 && (off0 & 3) == 0 && (page_size & 3) == 0 &&
                        slots[1] == slots[0] + 1 &&
                        slots[2] == slots[0] + 2 && slots[3] == slots[0] + 3;    // (then all in one page)
  const int quads = hd >> 2;
  for (int item = first; item < nkv * quads; item += stride) {
    const int head = item / quads, d0 = (item % quads) * 4;
    uint2 raw[kRopeTokens];
#pragma unroll
    for (int j = 0; j < kRopeTokens; ++j)
      if (j < nt)
        raw[j] = *reinterpret_cast<const uint2*>(qkv + (size_t)(t0 + j) * row_stride + (size_t)(nh + nkv + head) * hd + d0);
    if (together) {
      uint16_t* tile = vcache + ((size_t)(slots[0] / page_size) * nkv + head) * hd * page_size;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // column d0 + e of the four tokens: 16 bits out of each token's 8 bytes
        uint2 col;
        const uint32_t v0 = ((e < 2 ? raw[0].x : raw[0].y) >> ((e & 1) * 16)) & 0xffffu;
        const uint32_t v1 = ((e < 2 ? raw[1].x : raw[1].y) >> ((e & 1) * 16)) & 0xffffu;
        const uint32_t v2 = ((e < 2 ? raw[2].x : raw[2].y) >> ((e & 1) * 16)) & 0xffffu;
        const uint32_t v3 = ((e < 2 ? raw[3].x : raw[3].y) >> ((e & 1) * 16)) & 0xffffu;
        col.x = v0 | (v1 << 16);
        col.y = v2 | (v3 << 16);
        *reinterpret_cast<uint2*>(tile + value_offset(d0 + e, off0, hd, page_size)) = col;
      }
    } else {
#pragma unroll
      for (int j = 0; j < kRopeTokens; ++j) {
        if (j >= nt || slots[j] < 0) continue;
        uint16_t* tile = vcache + ((size_t)(slots[j] / page_size) * nkv + head) * hd * page_size;
        const uint16_t* v = reinterpret_cast<const uint16_t*>(&raw[j]);
#pragma unroll
        for (int e = 0; e < 4; ++e) tile[value_offset(d0 + e, slots[j] % page_size, hd, page_size)] = v[e];
      }
    }
  }
}

extern "C" int atoma_rope_cache_write(void* qkv, int act_dtype, int row_stride, const int32_t* positions,
                                      const float* cos_t, const float* sin_t, int rotary_dim, void* kcache,
                                      void* vcache, int cache_dtype, const int32_t* slot_mapping, int page_size,
                                      int n_tokens, int nh, int nkv, int hd, void* q_out, int q_stride,
                                      hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (q_out && (cos_t == nullptr || rotary_dim != hd || q_stride < nh * hd)) return ATOMA_ERR_SHAPE;
  if (rotary_dim < 0 || rotary_dim > hd || (rotary_dim & 1) || row_stride < (nh + 2 * nkv) * hd || page_size <= 0)
    return ATOMA_ERR_SHAPE;
  if (nh + 2 * nkv > 65535) return ATOMA_ERR_SHAPE;
  // without caches only q (and, for a caller that rotates k in place of q, all nh heads) is touched
  const int heads = kcache ? nh + 2 * nkv : nh;
  const int items = heads * (hd / 2);
  if (hd & 1) return ATOMA_ERR_SHAPE;
  // few tokens (decode steps) are quicker with many small blocks; measured on MI355X
  if (n_tokens >= 32 && act_dtype == kBF16 && cache_dtype == kBF16 && cos_t && sin_t && rotary_dim == hd && hd % 16 == 0 &&
      row_stride % 8 == 0 && ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)kcache & 15) == 0 && ((uintptr_t)vcache & 7) == 0 &&
      q_stride % 8 == 0 &&
      ((uintptr_t)q_out & 15) == 0 &&
      ((uintptr_t)cos_t & 15) == 0 && ((uintptr_t)sin_t & 15) == 0) {
    const int groups = (n_tokens + kRopeTokens - 1) / kRopeTokens;
    const int passes = (kRopeTokens * (nh + nkv) * (hd >> 4) + 255) / 256;      // of 256 threads over a block's items
    int split = (2048 + groups - 1) / groups;                                  // aim at 2048 blocks: eight a CU
    split = split > passes ? passes : split;
    hipLaunchKernelGGL(rope_cache_write_vec_kernel, dim3(groups, split), dim3(256), 0,
                       stream, (uint16_t*)qkv, row_stride, positions, cos_t, sin_t, (uint16_t*)kcache,
                       (uint16_t*)vcache, slot_mapping, page_size, nh, nkv, hd, (uint16_t*)q_out, q_stride, n_tokens);
    ATOMA_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid(n_tokens, (items + 255) / 256), block(256);
#define ATOMA_ROPE(TA, TC)                                                                                        \
  hipLaunchKernelGGL((rope_cache_write_kernel<TA, TC>), grid, block, 0, stream, (TA*)qkv, row_stride, positions, \
                     cos_t, sin_t, rotary_dim, (TC*)kcache, (TC*)vcache, slot_mapping, page_size, nh, nkv, hd, heads, \
                     (TA*)q_out, q_stride)
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
// out[t, i] = silu(gate[t, i]) * up[t, i], silu(z) = z * sigmoid(z); gate and up come in one row of 2 * inter.
// Reference: models/src/llama.rs:364.
// Where gate and up of output i lie in a row of 2 * inter values: in two halves (block == 0), or interleaved in
// blocks of 16 gate values followed by their 16 up values (block == 16), the layout of the fused gate-up product.
__device__ __forceinline__ int gate_index(int i, int block) { return block ? ((i >> 4) << 5) + (i & 15) : i; }
__device__ __forceinline__ int up_index(int i, int inter, int block) {
  return block ? ((i >> 4) << 5) + 16 + (i & 15) : inter + i;
}

template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, size_t total, int block) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inter;
    const int i = (int)(idx % inter);
    const float g = to_f32(gu[t * 2 * inter + gate_index(i, block)]);
    const float u = to_f32(gu[t * 2 * inter + up_index(i, inter, block)]);
    out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
  }
}

// four values per thread; needs inter % 4 == 0 and 16-byte aligned rows
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int n_tokens, int block) {
  const int quads = inter >> 2;
  const size_t total = (size_t)n_tokens * quads;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
    const size_t t = idx / quads;
    const int i = (int)(idx % quads) * 4;
    const f4 g = load4(gu + t * 2 * inter + gate_index(i, block));
    const f4 u = load4(gu + t * 2 * inter + up_index(i, inter, block));
    f4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o.v[e] = g.v[e] / (1.0f + expf(-g.v[e])) * u.v[e];
    store4(out + t * inter + i, o);
  }
}

// eight bfloat16 values per thread (16-byte loads and stores); needs inter % 8 == 0 and 16-byte aligned rows
__global__ void __launch_bounds__(256)
swiglu_vec8_kernel(const uint16_t* __restrict__ gu, uint16_t* __restrict__ out, int inter, int n_tokens, int block) {
  const int octs = inter >> 3;
  const size_t total = (size_t)n_tokens * octs;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
    const size_t t = idx / octs;
    const int i = (int)(idx % octs) * 8;
    const uint4 graw = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + gate_index(i, block));
    const uint4 uraw = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + up_index(i, inter, block));
    const uint16_t* g = reinterpret_cast<const uint16_t*>(&graw);
    const uint16_t* u = reinterpret_cast<const uint16_t*>(&uraw);
    uint4 oraw;
    uint16_t* o = reinterpret_cast<uint16_t*>(&oraw);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gv = bf16_bits_to_f32(g[e]);
      o[e] = f32_to_bf16_bits(gv / (1.0f + expf(-gv)) * bf16_bits_to_f32(u[e]));
    }
    *reinterpret_cast<uint4*>(out + t * inter + i) = oraw;
  }
}

extern "C" int atoma_swiglu(const void* gu, void* out, int dtype, int n_tokens, int inter, int block,
                            hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (block != 0 && (block != 16 || inter % 16)) return ATOMA_ERR_SHAPE;
  const size_t total = (size_t)n_tokens * inter;
  if (dtype == kBF16 && inter % 8 == 0 && ((uintptr_t)gu & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    size_t octs = total / 8;
    int vb = (int)((octs + 255) / 256);
    if (vb > 16384) vb = 16384;
    hipLaunchKernelGGL(swiglu_vec8_kernel, dim3(vb), dim3(256), 0, stream, (const uint16_t*)gu, (uint16_t*)out, inter,
                       n_tokens, block);
    ATOMA_LAUNCH_CHECK();
    return 0;
  }
  if (inter % 4 == 0 && ((uintptr_t)gu & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    size_t quads = total / 4;
    int vb = (int)((quads + 255) / 256);
    if (vb > 16384) vb = 16384;
    if (dtype == kF32)
      hipLaunchKernelGGL(swiglu_vec_kernel<float>, dim3(vb), dim3(256), 0, stream, (const float*)gu, (float*)out, inter,
                         n_tokens, block);
    else if (dtype == kBF16)
      hipLaunchKernelGGL(swiglu_vec_kernel<bf16_t>, dim3(vb), dim3(256), 0, stream, (const bf16_t*)gu, (bf16_t*)out,
                         inter, n_tokens, block);
    else
      return ATOMA_ERR_DTYPE;
    ATOMA_LAUNCH_CHECK();
    return 0;
  }
  int blocks = (int)((total + 255) / 256);
  if (blocks > 65536) blocks = 65536;
  if (dtype == kF32)
    hipLaunchKernelGGL(swiglu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gu, (float*)out, inter,
                       total, block);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)gu, (bf16_t*)out,
                       inter, total, block);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// dst[dst_idx[i]] = src[src_idx[i]]: puts tokens sampled by the previous step, which the host has not seen yet,
// into the next step's token list on the device.  pairs = [n][2] (dst index, src index).
__global__ void feed_tokens_kernel(int32_t* __restrict__ dst, const int32_t* __restrict__ src,
                                   const int32_t* __restrict__ pairs, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[pairs[2 * i]] = src[pairs[2 * i + 1]];
}

extern "C" int atoma_feed_tokens(int32_t* dst, const int32_t* src, const int32_t* pairs, int n, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(feed_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, dst, src, pairs, n);
  ATOMA_LAUNCH_CHECK();
  return 0;
}
