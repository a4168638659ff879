// Paged attention for any head size up to 256, any page size, float32 or bfloat16: the slow, general kernel.
// It serves the true 32-bit path and every shape that the MFMA kernels refuse.
//
// One wave per (query token, query head).  The token at absolute position p of request s attends keys
// [max(0, p - window + 1), p] of that request, read through its block table, after this step's keys and values
// have been written.  That one rule covers whole prompts, portions of prompts and single decoded tokens
// (bottom-right aligned causal mask, csrc/kernels/mask.h:171-172 of the reference).
// Keys are visited in chunks of 64 starting at the first visible key, so the order of every reduction depends
// only on (p, window): the result for a token does not depend on how the step was cut or batched.
// Online softmax in float32 (csrc/kernels/softmax.h:128-186 of the reference); query head h reads KV head
// h / (nh / nkv) (csrc/kernels/flash_fwd_kernel.h:593).  With slopes (one per query head) the score of key j for the
// token at p gains slopes[h] * (j - p), a bias that is linear in the distance (the reference's kernels take such
// slopes too: csrc/kernels/mask.h:155-157, 179-186; its Llama passes none).
#include "common.h"
#include "cache_layout.h"

using namespace atoma;

constexpr int kMaxHead = 256;

template <typename TQ, typename TC>
__global__ void __launch_bounds__(64)
paged_attention_generic_kernel(const TQ* __restrict__ q, int q_stride, const TC* __restrict__ kcache,
                               const TC* __restrict__ vcache, TQ* __restrict__ out, int out_stride,
                               const int32_t* __restrict__ block_tables, int max_blocks,
                               const int32_t* __restrict__ token_seq, const int32_t* __restrict__ positions,
                               float scale, int window, int page_size, int nh, int nkv, int hd,
                               const float* __restrict__ slopes) {
  __shared__ float qs[kMaxHead];
  __shared__ float ps[kWave];
  __shared__ int32_t pg[kWave];
  __shared__ int32_t of[kWave];

  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = token_seq[t], p = positions[t];
  const int kvh = h / (nh / nkv);
  const int32_t* table = block_tables + (size_t)s * max_blocks;
  const int first = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const float slope = slopes ? slopes[h] : 0.f;

  for (int d = lane; d < hd; d += kWave) qs[d] = to_f32(q[(size_t)t * q_stride + (size_t)h * hd + d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[kMaxHead / kWave] = {0.f, 0.f, 0.f, 0.f};

  for (int base = first; base <= p; base += kWave) {
    const int j = base + lane;
    const bool valid = j <= p;
    float sc = -INFINITY;
    int page = 0, off = 0;
    if (valid) {
      page = table[j / page_size];
      off = j % page_size;
      // the token's columns lie in runs of 8 inside the tile (cache_layout.h)
      const TC* kt = kcache + ((size_t)page * nkv + kvh) * page_size * hd;
      float dot = 0.f;
      for (int d0 = 0; d0 < hd; d0 += 8) {
        const TC* kr = kt + key_offset(off, d0, page_size);
#pragma unroll
        for (int e = 0; e < 8; ++e) dot += qs[d0 + e] * to_f32(kr[e]);
      }
      sc = dot * scale + slope * (float)(j - p);
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float corr = expf(m - m_new);  // exp(-inf) = 0 on the first chunk
    const float pj = valid ? expf(sc - m_new) : 0.f;
    l = l * corr + wave_sum(pj);
    m = m_new;
    __syncthreads();
    ps[lane] = pj;
    pg[lane] = page;
    of[lane] = off;
    __syncthreads();
    const int n = (p - base + 1 < kWave) ? p - base + 1 : kWave;
#pragma unroll
    for (int i = 0; i < kMaxHead / kWave; ++i) {
      const int d = lane + i * kWave;
      if (d < hd) {
        float a = acc[i] * corr;
        for (int jj = 0; jj < n; ++jj)
          a += ps[jj] * to_f32(vcache[((size_t)pg[jj] * nkv + kvh) * hd * page_size +
                                      value_offset(d, of[jj], hd, page_size)]);
        acc[i] = a;
      }
    }
  }
  const float inv = 1.0f / l;  // at least the token's own key is visible, so l > 0
#pragma unroll
  for (int i = 0; i < kMaxHead / kWave; ++i) {
    const int d = lane + i * kWave;
    if (d < hd) out[(size_t)t * out_stride + (size_t)h * hd + d] = from_f32<TQ>(acc[i] * inv);
  }
}

extern "C" int atoma_paged_attention_generic(const void* q, int q_stride, const void* kcache, const void* vcache,
                                             void* out, int out_stride, int act_dtype, int cache_dtype,
                                             const int32_t* block_tables, int max_blocks, const int32_t* token_seq,
                                             const int32_t* positions, float scale, int window, int page_size,
                                             int n_tokens, int nh, int nkv, int hd, const float* slopes,
                                             hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (hd <= 0 || hd > kMaxHead || nkv <= 0 || nh % nkv || page_size <= 0 || max_blocks <= 0 || nh > 65535)
    return ATOMA_ERR_SHAPE;
  dim3 grid(n_tokens, nh), block(kWave);
#define ATOMA_ATTN(TQ, TC)                                                                                       \
  hipLaunchKernelGGL((paged_attention_generic_kernel<TQ, TC>), grid, block, 0, stream, (const TQ*)q, q_stride, \
                     (const TC*)kcache, (const TC*)vcache, (TQ*)out, out_stride, block_tables, max_blocks,      \
                     token_seq, positions, scale, window, page_size, nh, nkv, hd, slopes)
  if (act_dtype == kF32 && cache_dtype == kF32) ATOMA_ATTN(float, float);
  else if (act_dtype == kBF16 && cache_dtype == kBF16) ATOMA_ATTN(bf16_t, bf16_t);
  else if (act_dtype == kF32 && cache_dtype == kBF16) ATOMA_ATTN(float, bf16_t);
  else if (act_dtype == kBF16 && cache_dtype == kF32) ATOMA_ATTN(bf16_t, float);
  else return ATOMA_ERR_DTYPE;
#undef ATOMA_ATTN
  ATOMA_LAUNCH_CHECK();
  return 0;
}
