// Sampling from float32 logits, one block of 1024 threads per row:
//   greedy (temperature <= 0): argmax, lowest index on ties;
//   else weights w_i = exp((l_i - max) / T), optionally cut to the k largest and then to the smallest set of
//   largest weights whose mass reaches top_p of the whole, ties towards the lower index; the token is the first
//   index (in vocabulary order) whose running sum of kept weights exceeds u * (kept mass), u in [0, 1) given
//   by the caller per row.
// The reference samples on the host with candle's LogitsProcessor in the modes All / TopK / TopP / TopKThenTopP
// (backends/vllm/src/llm_service.rs:346-372, model_executor.rs:231-235) and applies a repeat penalty to the
// last repeat_last_n tokens first (model_executor.rs:211-225).
// All reductions run in an order fixed by the vocabulary size alone, so a row's draw does not depend on the batch.
#include "common.h"

using namespace atoma;

constexpr int kSampThreads = 1024;
constexpr int kSampWaves = kSampThreads / kWave;

struct ArgMax {
  float v;
  int i;
};

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__device__ ArgMax block_argmax(ArgMax a, ArgMax* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax b;
    b.v = __shfl_xor(a.v, o, 64);
    b.i = __shfl_xor(a.i, o, 64);
    a = better(a, b);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = a;
  __syncthreads();
  ArgMax r = scratch[0];
  for (int i = 1; i < kSampWaves; ++i) r = better(r, scratch[i]);
  return r;
}

// sum of a float and of an int over the block, both in one pass
__device__ void block_sum2(float& f, int& n, float* fs, int* ns) {
  f = wave_sum(f);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) n += __shfl_xor(n, o, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) {
    fs[wave] = f;
    ns[wave] = n;
  }
  __syncthreads();
  float ft = 0.f;
  int nt = 0;
  for (int i = 0; i < kSampWaves; ++i) {
    ft += fs[i];
    nt += ns[i];
  }
  f = ft;
  n = nt;
}

__global__ void __launch_bounds__(kSampThreads)
sample_kernel(const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
              const int32_t* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
              float* __restrict__ weights, int32_t* __restrict__ out_token, float* __restrict__ out_logit) {
  __shared__ ArgMax am[kSampWaves];
  __shared__ float fs[kSampWaves];
  __shared__ int ns[kSampWaves];
  __shared__ float scan_f[kSampThreads];
  __shared__ int scan_n[kSampThreads];
  __shared__ int chosen;

  const int row = blockIdx.x, tid = threadIdx.x;
  const float* lr = logits + (size_t)row * ld;
  float* w = weights + (size_t)row * vocab;

  ArgMax a = {-INFINITY, 0x7fffffff};
  if ((vocab & 3) == 0 && (((uintptr_t)lr) & 15) == 0) {
    // four values per load, several loads in flight
    const float4* l4 = reinterpret_cast<const float4*>(lr);
    const int n4 = vocab >> 2;
#pragma unroll 4
    for (int i = tid; i < n4; i += kSampThreads) {
      const float4 v = l4[i];
      a = better(a, ArgMax{v.x, 4 * i});
      a = better(a, ArgMax{v.y, 4 * i + 1});
      a = better(a, ArgMax{v.z, 4 * i + 2});
      a = better(a, ArgMax{v.w, 4 * i + 3});
    }
  } else {
    for (int i = tid; i < vocab; i += kSampThreads) a = better(a, ArgMax{lr[i], i});
  }
  a = block_argmax(a, am);
  const float temp = temperature[row];
  if (!(temp > 0.f)) {
    if (tid == 0) {
      out_token[row] = a.i;
      out_logit[row] = a.v;
    }
    return;
  }

  // weights and their total
  const float inv_t = 1.0f / temp;
  float total = 0.f;
  int dummy = 0;
  for (int i = tid; i < vocab; i += kSampThreads) {
    const float wi = expf((lr[i] - a.v) * inv_t);
    w[i] = wi;
    total += wi;
  }
  block_sum2(total, dummy, fs, ns);
  __syncthreads();  // w written by other threads is read below

  // Threshold tau (as float bits; weights are non-negative so bit order is value order) and the number of
  // weights equal to tau that are kept (those of lowest index).  Everything above tau is kept.
  uint32_t tau = 0;            // keep all: w >= 0
  int ties_kept = 0x7fffffff;  // all ties
  const int k = top_k[row];
  const float p = top_p[row];
  if (k > 0 && k < vocab) {
    uint32_t prefix = 0;
    for (int bit = 30; bit >= 0; --bit) {
      const uint32_t cand = prefix | (1u << bit);
      int cnt = 0;
      float f0 = 0.f;
      for (int i = tid; i < vocab; i += kSampThreads) cnt += (__float_as_uint(w[i]) >= cand);
      block_sum2(f0, cnt, fs, ns);
      if (cnt >= k) prefix = cand;
    }
    int gt = 0;
    float f0 = 0.f;
    for (int i = tid; i < vocab; i += kSampThreads) gt += (__float_as_uint(w[i]) > prefix);
    block_sum2(f0, gt, fs, ns);
    tau = prefix;
    ties_kept = k - gt;
  }
  if (p < 1.0f) {
    const float need = p * total;
    uint32_t prefix = 0;
    for (int bit = 30; bit >= 0; --bit) {
      const uint32_t cand = prefix | (1u << bit);
      float mass = 0.f;
      int n0 = 0;
      for (int i = tid; i < vocab; i += kSampThreads) mass += (__float_as_uint(w[i]) >= cand) ? w[i] : 0.f;
      block_sum2(mass, n0, fs, ns);
      if (mass >= need) prefix = cand;
    }
    float mass_gt = 0.f;
    int n_eq = 0;
    for (int i = tid; i < vocab; i += kSampThreads) {
      const uint32_t b = __float_as_uint(w[i]);
      mass_gt += (b > prefix) ? w[i] : 0.f;
      n_eq += (b == prefix);
    }
    block_sum2(mass_gt, n_eq, fs, ns);
    const float tv = __uint_as_float(prefix);
    int ties = n_eq;
    if (tv > 0.f) {
      ties = (int)ceilf((need - mass_gt) / tv);
      if (ties < 1) ties = 1;
      if (ties > n_eq) ties = n_eq;
    }
    // the tighter of the two cuts wins
    if (prefix > tau || (prefix == tau && ties < ties_kept)) {
      tau = prefix;
      ties_kept = ties;
    }
  }

  // Each thread owns a contiguous span of the vocabulary; scan kept mass and tie counts over spans.
  const int span = (vocab + kSampThreads - 1) / kSampThreads;
  const int lo = tid * span, hi = (lo + span < vocab) ? lo + span : vocab;
  int my_ties = 0;
  for (int i = lo; i < hi; ++i) my_ties += (__float_as_uint(w[i]) == tau);
  scan_n[tid] = my_ties;
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int i = 0; i < kSampThreads; ++i) {
      const int c = scan_n[i];
      scan_n[i] = run;
      run += c;
    }
  }
  __syncthreads();
  int rank = scan_n[tid];
  float my_mass = 0.f;
  for (int i = lo; i < hi; ++i) {
    const uint32_t b = __float_as_uint(w[i]);
    const bool keep = b > tau || (b == tau && rank < ties_kept);
    rank += (b == tau);
    my_mass += keep ? w[i] : 0.f;
  }
  scan_f[tid] = my_mass;
  if (tid == 0) chosen = -1;
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    for (int i = 0; i < kSampThreads; ++i) {
      const float c = scan_f[i];
      scan_f[i] = run;
      run += c;
    }
    fs[0] = run;  // kept mass
  }
  __syncthreads();
  const float target = uniform[row] * fs[0];
  const float before = scan_f[tid];
  // the span that contains the target walks it; the last kept token catches a target at the very end
  if (my_mass > 0.f && before <= target && (target < before + my_mass)) {
    float run = before;
    int r = scan_n[tid], pick = -1, last_kept = -1;
    for (int i = lo; i < hi; ++i) {
      const uint32_t b = __float_as_uint(w[i]);
      const bool keep = b > tau || (b == tau && r < ties_kept);
      r += (b == tau);
      if (!keep) continue;
      last_kept = i;
      run += w[i];
      if (run > target) {
        pick = i;
        break;
      }
    }
    if (pick < 0) pick = last_kept;
    atomicMax(&chosen, pick);
  }
  __syncthreads();
  if (tid == 0) {
    int c = chosen;
    if (c < 0) c = a.i;  // rounding left the target beyond every span: fall back to the most likely token
    out_token[row] = c;
    out_logit[row] = lr[c];
  }
}

extern "C" int atoma_sample(const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                            const int32_t* top_k, const float* top_p, const float* uniform, float* weights,
                            int32_t* out_token, float* out_logit, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(kSampThreads), 0, stream, logits, ld, vocab, temperature, top_k,
                     top_p, uniform, weights, out_token, out_logit);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// Repeat penalty: for each listed (row, token), logit >= 0 ? logit / penalty : logit * penalty.
// The caller lists each token of a row's context once.
__global__ void repeat_penalty_kernel(float* __restrict__ logits, int ld, const int32_t* __restrict__ rows,
                                      const int32_t* __restrict__ tokens, const float* __restrict__ penalty, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int r = rows[i];
  float* x = logits + (size_t)r * ld + tokens[i];
  const float v = *x, pen = penalty[r];
  *x = v >= 0.f ? v / pen : v * pen;
}

extern "C" int atoma_repeat_penalty(float* logits, int ld, const int32_t* rows, const int32_t* tokens,
                                    const float* penalty, int n, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(repeat_penalty_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, logits, ld, rows, tokens,
                     penalty, n);
  ATOMA_LAUNCH_CHECK();
  return 0;
}
