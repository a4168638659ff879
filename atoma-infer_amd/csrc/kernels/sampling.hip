// Sampling from float32 logits, one block of 1024 threads per row that draws (two walks over the row without a cut,
// five or six with top-k or top-p), up to eight per greedy row:
//   greedy (temperature <= 0): argmax, lowest index on ties;
//   else weights w_i = exp((l_i - max) / T), optionally cut to the k largest and then to the smallest set of
//   largest weights whose mass reaches top_p of the whole, ties towards the lower index; the token is the first
//   index (in vocabulary order) whose running sum of kept weights exceeds u * (kept mass), u in [0, 1) given
//   by the caller per row.
// The reference samples on the host with candle's LogitsProcessor in the modes All / TopK / TopP / TopKThenTopP
// (backends/vllm/src/llm_service.rs:346-372, model_executor.rs:231-235) and applies a repeat penalty to the
// last repeat_last_n tokens first (model_executor.rs:211-225).
// Masses are summed as integers (see fixed_of), so a row's draw depends on nothing but the row.
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

// Kept weights are summed as integers, in units of 2^-40 of the largest weight (which is 1): integer sums do not
// depend on their order, so thresholds, kept mass and the draw are exact functions of the row, whatever the
// number of threads or the order in which they add.
typedef unsigned long long u64;
// w * 2^40 cut to an integer, as hi * 2^20 + lo, in two exact steps of 20 bits (there is no single
// float-to-64-bit instruction; sums of a few thousand hi or lo parts fit 32 bits)
__device__ __forceinline__ void fixed_parts(float w, uint32_t& hi, uint32_t& lo) {
  const float a = w * 1048576.0f;
  hi = (uint32_t)a;
  lo = (uint32_t)((a - (float)hi) * 1048576.0f);
}
__device__ __forceinline__ u64 fixed_of(float w) {
  uint32_t hi, lo;
  fixed_parts(w, hi, lo);
  return ((u64)hi << 20) + lo;
}

constexpr int kBins = kSampThreads;             // one histogram bin per thread
constexpr int kSlices = 8;                      // per wave, for the draw

template <typename T> __device__ __forceinline__ T wave_total(T v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// inclusive prefix sums over the lanes of a wave
template <typename T> __device__ __forceinline__ T wave_prefix(T v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const T up = __shfl_up(v, o, 64);
    if (lane >= o) v += up;
  }
  return v;
}

// f(value, index) for every element of x[0, n): groups of four neighbours per thread where the row allows
// 16-byte loads
template <typename F> __device__ __forceinline__ void sweep(const float* __restrict__ x, int n, F f) {
  const int tid = threadIdx.x;
  if ((((uintptr_t)x) & 15) == 0) {
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const int n4 = n >> 2;
    // eight loads a thread are issued together: every batch is a trip to memory, and a row of a large vocabulary
    // should take few of them
    constexpr int U = 8;
    for (int i0 = tid; i0 < n4; i0 += U * kSampThreads) {
      float4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + u * kSampThreads;
        v[u] = x4[i < n4 ? i : n4 - 1];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + u * kSampThreads;
        if (i < n4) {
          f(v[u].x, 4 * i);
          f(v[u].y, 4 * i + 1);
          f(v[u].z, 4 * i + 2);
          f(v[u].w, 4 * i + 3);
        }
      }
    }
    for (int i = (n4 << 2) + tid; i < n; i += kSampThreads) f(x[i], i);
  } else {
    for (int i = tid; i < n; i += kSampThreads) f(x[i], i);
  }
}

// The highest bin b whose suffix sum hist[b] + hist[b + 1] + ... reaches target (0 < target <= sum of all bins),
// and what of target is left for bin b itself.  Thread t looks at bin t.  sel < 0 if no bin does.
template <typename T>
__device__ void select_bin(const T* hist, T target, int& sel, T& rest, T* wave_sums, int* sel_s, T* rest_s) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T mine = hist[tid];
  T suffix = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const T down = __shfl_down(suffix, o, 64);
    if (lane + o < 64) suffix += down;
  }
  if (lane == 0) wave_sums[wave] = suffix;
  if (tid == 0) *sel_s = -1;
  __syncthreads();
  for (int w2 = wave + 1; w2 < kSampWaves; ++w2) suffix += wave_sums[w2];
  if (suffix >= target && suffix - mine < target) {      // suffix sums fall with t: one bin at most
    *sel_s = tid;
    *rest_s = target - (suffix - mine);
  }
  __syncthreads();
  sel = *sel_s;
  rest = sel >= 0 ? *rest_s : target;
  __syncthreads();
}

// What the blocks of a greedy row leave for the one that finishes last (see the kernel): a row's bests and how many
// have arrived.  Arrays of the code object, zero when it is loaded and left at zero by every launch; all launches on
// a device share them, so two that overlap in time (two streams, two threads) race, as they would on one workspace.
constexpr int kMaxSplits = 8;
constexpr int kSplitRows = 1024;        // launches of more rows give every row one block
static __device__ float split_val[kSplitRows * kMaxSplits];
static __device__ int split_idx[kSplitRows * kMaxSplits];
static __device__ int split_count[kSplitRows];

// blocks a row: enough that a few rows of a large vocabulary keep many CUs reading
static int sample_splits(int n_rows, int vocab) {
  if (n_rows > kSplitRows || vocab < 16384) return 1;
  int s = 256 / n_rows;
  return s < 1 ? 1 : s > kMaxSplits ? kMaxSplits : s;
}

__global__ void __launch_bounds__(kSampThreads)
sample_kernel(const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
              const int32_t* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
              float* __restrict__ weights, int32_t* __restrict__ out_token, float* __restrict__ out_logit) {
  __shared__ ArgMax am[kSampWaves];
  __shared__ uint32_t hist_k[kBins];       // top-k search: how many weights fall into each bin
  __shared__ uint32_t hist_pn[kBins];      // top-p search: how many, and their mass
  __shared__ u64 hist_pm[kBins];
  __shared__ u64 wave_u64[kSampWaves];
  __shared__ uint32_t wave_u32[kSampWaves];
  __shared__ u64 slice_mass[kSampWaves * kSlices];
  __shared__ uint32_t slice_rank[kSampWaves * kSlices];
  __shared__ int sel_s;
  __shared__ u64 rest_u64;
  __shared__ uint32_t rest_u32;

  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* lr = logits + (size_t)row * ld;
  float* w = weights + (size_t)row * vocab;
  const float temp = temperature[row];

  // A greedy row is shared by the gridDim.y blocks of its row: one block reads a large vocabulary no faster than one
  // CU can load (a row of 128k logits: 10 us).  Each takes a stretch of the row and leaves its best; the block that
  // finishes last picks among them (stores and loads that go through to memory, a device-wide counter that it leaves
  // at zero: no fence that would flush a cache).  Rows that draw keep one block: its walks share what they find.
  const int parts = gridDim.y, part = blockIdx.y;
  if (parts > 1) {
    if (temp > 0.f) {
      if (part > 0) return;
    } else {
      const int len = ((vocab + parts * 4 - 1) / (parts * 4)) * 4;
      const int lo = part * len, hi = lo + len < vocab ? lo + len : vocab;
      ArgMax a = {-INFINITY, 0x7fffffff};
      if (lo < hi) sweep(lr + lo, hi - lo, [&](float v, int i) { a = better(a, ArgMax{v, i + lo}); });
      a = block_argmax(a, am);
      if (tid == 0) {
        __hip_atomic_store(&split_val[row * kMaxSplits + part], a.v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&split_idx[row * kMaxSplits + part], a.i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
        const int before = __hip_atomic_fetch_add(&split_count[row], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (before + 1 == parts) {
          __hip_atomic_store(&split_count[row], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ArgMax r = {-INFINITY, 0x7fffffff};
          for (int p = 0; p < parts; ++p) {
            ArgMax b;
            b.v = __hip_atomic_load(&split_val[row * kMaxSplits + p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            b.i = __hip_atomic_load(&split_idx[row * kMaxSplits + p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            r = better(r, b);
          }
          if ((unsigned)r.i >= (unsigned)vocab) r.i = 0;   // a row of NaN has no largest value: still name a token
          out_token[row] = r.i;
          out_logit[row] = lr[r.i];
        }
      }
      return;
    }
  }

  ArgMax a = {-INFINITY, 0x7fffffff};
  sweep(lr, vocab, [&](float v, int i) { a = better(a, ArgMax{v, i}); });
  a = block_argmax(a, am);
  if ((unsigned)a.i >= (unsigned)vocab) a.i = 0;       // a row of NaN has no largest value: still name a token
  if (tid == 0) {          // the answer of a greedy row, and of a row whose weights are no numbers
    out_token[row] = a.i;
    out_logit[row] = lr[a.i];
  }
  if (!(temp > 0.f)) return;

  const int k = top_k[row];
  const float p = top_p[row];
  const bool cut_k = k > 0 && k < vocab, cut_p = p < 1.0f, cut = cut_k || cut_p;

  // Each wave owns a contiguous stretch of the vocabulary, cut into kSlices slices of whole pieces of 256 values
  // (four neighbours a lane, fetched four pieces at a time: a wave walks at the pace of its loads).
  const int stretch = ((vocab + kSampWaves * 256 - 1) / (kSampWaves * 256)) * 256;
  const int slice_len = ((stretch / 256 + kSlices - 1) / kSlices) * 256;
  const int begin = wave * stretch, end = begin + stretch < vocab ? begin + stretch : vocab;
  const bool vec_l = (((uintptr_t)lr) & 15) == 0, vec_w = (((uintptr_t)w) & 15) == 0;
  // the lane's four values of the piece of x at `at`, up to `stop`; how many exist
  auto piece = [&](const float* x, bool vec, int at, int stop, float* v) -> int {
    const int i = at + lane * 4;
    const int n = stop - i < 0 ? 0 : stop - i > 4 ? 4 : stop - i;
    if (n == 4 && vec) {
      const float4 q = *reinterpret_cast<const float4*>(x + i);
      v[0] = q.x, v[1] = q.y, v[2] = q.z, v[3] = q.w;
    } else {
      for (int e = 0; e < 4; ++e) v[e] = e < n ? x[i + e] : 0.f;
    }
    return n;
  };
  auto slice_range = [&](int sl, int& s_begin, int& s_end) {
    s_begin = begin + sl * slice_len;
    s_end = s_begin + slice_len < end ? s_begin + slice_len : end;
  };

  // Weights w = exp((l - max) / T) = 2^((l - max) * log2(e) / T), largest = 1: one multiply and the hardware's
  // exp2.  The same walk fills what the next step needs: with a cut, the histograms of the first ten bits and the
  // total; without, the kept mass of every slice (everything is kept).
  hist_k[tid] = 0;
  hist_pn[tid] = 0;
  hist_pm[tid] = 0;
  __syncthreads();
  const float inv_t = 1.4426950408889634f / temp;
  uint32_t total_hi = 0, total_lo = 0;
  for (int sl = 0; sl < kSlices; ++sl) {
    int s_begin, s_end;
    slice_range(sl, s_begin, s_end);
    uint32_t hi_sum = 0, lo_sum = 0;
    for (int at0 = s_begin; at0 < s_end; at0 += 4 * 256) {
      float vs[4][4];
      int ns[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) ns[j] = piece(lr, vec_l, at0 + j * 256, s_end, vs[j]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = at0 + j * 256 + lane * 4, n = ns[j];
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o[e] = __builtin_amdgcn_exp2f((vs[j][e] - a.v) * inv_t);
          if (e >= n) continue;
          uint32_t hi, lo;
          fixed_parts(o[e], hi, lo);
          hi_sum += hi;
          lo_sum += lo;
          if (cut) {
            const uint32_t bin = (__float_as_uint(o[e]) >> 20) & (kBins - 1);
            if (cut_k) atomicAdd(&hist_k[bin], 1u);
            if (cut_p) {
              atomicAdd(&hist_pn[bin], 1u);
              atomicAdd(&hist_pm[bin], ((u64)hi << 20) + lo);
            }
          }
        }
        if (n == 4 && vec_w) {
          *reinterpret_cast<float4*>(w + i) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
          for (int e = 0; e < n; ++e) w[i + e] = o[e];
        }
      }
    }
    if (!cut) {
      const u64 mass = wave_total(((u64)hi_sum << 20) + lo_sum);
      if (lane == 0) slice_mass[wave * kSlices + sl] = mass;
    }
    total_hi += hi_sum;
    total_lo += lo_sum;
  }
  u64 total = 0;
  if (cut_p) {
    total = wave_total(((u64)total_hi << 20) + total_lo);
    if (lane == 0) wave_u64[wave] = total;
  }
  __syncthreads();          // w and the histograms written by other threads are read below
  if (cut_p) {
    total = 0;
    for (int i = 0; i < kSampWaves; ++i) total += wave_u64[i];
    __syncthreads();
  }

  // The cut: a threshold tau (as float bits; weights are non-negative, so bit order is value order) above which
  // everything is kept, and the number of weights equal to tau that are kept (those of lowest index).  Both
  // searches walk down the bits of tau ten at a time: a histogram over the next ten bits of the weights that
  // share the bits found so far, then the highest bin whose suffix reaches what is still wanted.  A weight is at
  // most 1 = 0x3f800000, so 30 bits suffice.
  uint32_t bits_k = 0, bits_p = 0;       // the bits of the two thresholds found so far
  uint32_t want_k = cut_k ? (uint32_t)k : 0u, equal_k = 0, equal_p = 0;
  u64 want_p = 0;
  if (cut_p) {
    const double need = ceil((double)p * (double)total);
    want_p = need < 1.0 ? 1ull : (u64)need;
    if (want_p > total) want_p = total;
  }
  if (cut) {
#pragma unroll 1
    for (int level = 0; level < 3; ++level) {
      const int shift = 20 - 10 * level;
      if (level > 0) {                     // (the first histograms were filled with the weights)
        hist_k[tid] = 0;
        hist_pn[tid] = 0;
        hist_pm[tid] = 0;
        __syncthreads();
        sweep(w, vocab, [&](float v, int) {
          const uint32_t b = __float_as_uint(v);
          const uint32_t high = b >> (shift + 10), bin = (b >> shift) & (kBins - 1);
          if (cut_k && high == bits_k) atomicAdd(&hist_k[bin], 1u);
          if (cut_p && high == bits_p) {
            atomicAdd(&hist_pn[bin], 1u);
            atomicAdd(&hist_pm[bin], fixed_of(v));
          }
        });
        __syncthreads();
      }
      int sel;
      if (cut_k) {
        select_bin<uint32_t>(hist_k, want_k, sel, want_k, wave_u32, &sel_s, &rest_u32);
        if (sel < 0) sel = 0, want_k = 0x7fffffff;          // cannot happen: k < vocab weights exist
        bits_k = (bits_k << 10) | (uint32_t)sel;
        equal_k = hist_k[sel];
      }
      if (cut_p) {
        select_bin<u64>(hist_pm, want_p, sel, want_p, wave_u64, &sel_s, &rest_u64);
        if (sel < 0) sel = 0;                               // cannot happen: want_p <= total
        bits_p = (bits_p << 10) | (uint32_t)sel;
        equal_p = hist_pn[sel];
      }
      __syncthreads();
    }
  }
  uint32_t tau = 0, n_equal = 0xffffffffu;
  u64 ties_kept = ~0ull;                 // all of them
  if (cut_k) {
    tau = bits_k;
    ties_kept = want_k;                  // what the weights above tau leave of k
    n_equal = equal_k;
  }
  if (cut_p) {
    // as many ties as it takes to reach the mass still wanted
    const u64 each = fixed_of(__uint_as_float(bits_p));
    u64 ties = each ? (want_p + each - 1) / each : (u64)equal_p;
    if (ties < 1) ties = 1;
    if (ties > equal_p) ties = equal_p;
    if (!cut_k || bits_p > tau || (bits_p == tau && ties < ties_kept)) {     // the tighter of the two cuts wins
      tau = bits_p;
      ties_kept = ties;
      n_equal = equal_p;
    }
  }
  const bool all_ties = ties_kept >= (u64)n_equal;

  // The draw: the first index, in vocabulary order, at which the running sum of kept weights exceeds
  // u * (kept mass).  A tie's rank is the number of ties before it.  A walk over the weights leaves every slice's
  // kept mass (and the rank at its start) in LDS; the slice that holds the target is then walked again with
  // running sums over its lanes.
  // the kept mass of the lane's values of one piece, in two parts; rank: ties before the lane's first value
  auto lane_mass = [&](const float* v, int n, uint32_t rank, bool* keep, uint32_t& hi_sum, uint32_t& lo_sum) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t b = __float_as_uint(v[e]);
      keep[e] = e < n && (b > tau || (b == tau && (all_ties || (u64)rank < ties_kept)));
      if (e < n && b == tau) ++rank;
      if (keep[e]) {
        uint32_t hi, lo;
        fixed_parts(v[e], hi, lo);
        hi_sum += hi;
        lo_sum += lo;
      }
    }
  };
  auto lane_ties = [&](const float* v, int n) -> uint32_t {
    uint32_t ties = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) ties += e < n && __float_as_uint(v[e]) == tau;
    return ties;
  };

  if (cut) {
    uint32_t rank_run = 0;               // ties before the piece at hand
    if (!all_ties) {
      uint32_t mine = 0;
      for (int at0 = begin; at0 < end; at0 += 4 * 256) {
        float vs[4][4];
        int ns[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) ns[j] = piece(w, vec_w, at0 + j * 256, end, vs[j]);
#pragma unroll
        for (int j = 0; j < 4; ++j) mine += lane_ties(vs[j], ns[j]);
      }
      mine = wave_total(mine);
      if (lane == 0) wave_u32[wave] = mine;
      __syncthreads();
      for (int i = 0; i < wave; ++i) rank_run += wave_u32[i];
      __syncthreads();
    }
    for (int sl = 0; sl < kSlices; ++sl) {
      int s_begin, s_end;
      slice_range(sl, s_begin, s_end);
      if (lane == 0) slice_rank[wave * kSlices + sl] = rank_run;
      uint32_t hi_sum = 0, lo_sum = 0;
      for (int at0 = s_begin; at0 < s_end; at0 += 4 * 256) {
        float vs[4][4];
        int ns[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) ns[j] = piece(w, vec_w, at0 + j * 256, s_end, vs[j]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t rank = 0;
          if (!all_ties) {
            const uint32_t ties = lane_ties(vs[j], ns[j]);
            const uint32_t incl = wave_prefix(ties);
            rank = rank_run + incl - ties;
            rank_run += __shfl(incl, 63, 64);
          }
          bool keep[4];
          lane_mass(vs[j], ns[j], rank, keep, hi_sum, lo_sum);
        }
      }
      const u64 mass = wave_total(((u64)hi_sum << 20) + lo_sum);
      if (lane == 0) slice_mass[wave * kSlices + sl] = mass;
    }
  } else if (lane == 0) {
    for (int sl = 0; sl < kSlices; ++sl) slice_rank[wave * kSlices + sl] = 0;
  }
  __syncthreads();

  // which slice holds the target: running sums over the slices, one slice a thread
  constexpr int kAllSlices = kSampWaves * kSlices;
  static_assert(kAllSlices <= kSampThreads && kAllSlices % 64 == 0, "one slice a thread");
  const u64 mine = tid < kAllSlices ? slice_mass[tid] : 0;
  const u64 incl = wave_prefix(mine);
  if (lane == 63) wave_u64[wave] = incl;
  if (tid == 0) sel_s = -1;
  __syncthreads();
  u64 before = incl - mine, kept = 0;
  for (int i = 0; i < kAllSlices / 64; ++i) {
    if (i < wave) before += wave_u64[i];
    kept += wave_u64[i];
  }
  if (kept == 0) return;                           // weights that are no numbers: the default answer stands
  u64 target = (u64)((double)uniform[row] * (double)kept);
  if (target >= kept) target = kept - 1;           // (kept >= 2^40: the largest weight is always kept)
  if (tid < kAllSlices && before <= target && target < before + mine) {
    sel_s = tid;
    rest_u64 = before;
  }
  __syncthreads();
  const int slice = sel_s;
  if (slice < 0 || slice / kSlices != wave) return;         // (one slice does: kept > target)
  u64 run = rest_u64;
  uint32_t rank_at = slice_rank[slice];
  int s_begin, s_end;
  slice_range(slice % kSlices, s_begin, s_end);
  int pick = -1;
  for (int at = s_begin; at < s_end; at += 256) {
    float v[4];
    const int n = piece(w, vec_w, at, s_end, v);
    uint32_t rank = 0;
    if (!all_ties) {
      const uint32_t ties = lane_ties(v, n);
      const uint32_t ti = wave_prefix(ties);
      rank = rank_at + ti - ties;
      rank_at += __shfl(ti, 63, 64);
    }
    bool keep[4];
    uint32_t hi_sum = 0, lo_sum = 0;
    lane_mass(v, n, rank, keep, hi_sum, lo_sum);
    const u64 lm = ((u64)hi_sum << 20) + lo_sum;
    const u64 li = wave_prefix(lm);
    const u64 whole = __shfl(li, 63, 64);
    if (run + whole > target) {
      const u64 ahead = __ballot(run + li > target);
      const int first = __ffsll((long long)ahead) - 1;
      int found = -1;
      if (lane == first) {
        u64 r = run + li - lm;
        for (int e = 0; e < 4; ++e) {
          if (!keep[e]) continue;
          r += fixed_of(v[e]);
          if (r > target) {
            found = at + lane * 4 + e;
            break;
          }
        }
      }
      pick = __shfl(found, first, 64);
      break;
    }
    run += whole;
  }
  if (lane == 0) {
    const int c = pick >= 0 ? pick : a.i;
    out_token[row] = c;
    out_logit[row] = lr[c];
  }
}

extern "C" int atoma_sample(const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                            const int32_t* top_k, const float* top_p, const float* uniform, float* weights,
                            int32_t* out_token, float* out_logit, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows, sample_splits(n_rows, vocab)), dim3(kSampThreads), 0, stream, logits, ld,
                     vocab, temperature, top_k, top_p, uniform, weights, out_token, out_logit);
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

// ---- the same draw with every row shared by several blocks -----------------------------------------------------
// One block walks a row of 128k logits in 10 us, and a row with top-k and top-p is walked seven times: 100 to 135 us
// for a step's sampler however few rows there are.  Here a row's vocabulary is cut into P parts, a block each, and
// what the blocks of a row must know of each other (the row's largest logit, the histograms of a search level, the
// kept mass of every part) goes through memory from one launch to the next: six short launches in a row instead
// of one long one.  The arithmetic is that of sample_kernel (integer masses, ties towards the lower index), so the
// tokens are the same.
//
// A row's scratch memory: a header and, for each of the three search levels, the histograms of sample_kernel.
constexpr int kMaxParts = 16;
// (the state of the threshold search, see split_search_step)
struct SplitSearch {
  uint32_t bits_k, bits_p, want_k, equal_k, equal_p, pad;
  u64 want_p;
};
static_assert(sizeof(SplitSearch) == 32, "eight words");
constexpr int kMaxPartLen = 16 * kSampThreads;    // values of a part: at most 16 a thread in the last launch
struct SplitRow {
  u64 total;                         // mass of all weights
  u64 part_mass[kMaxParts];          // of a part: the mass of its weights above the threshold (all, without a cut)
  uint32_t part_ties[kMaxParts];     // of a part: weights equal to the threshold
  float part_max_v[kMaxParts];       // of a part: largest logit and its index
  int32_t part_max_i[kMaxParts];
  SplitSearch search[3];             // what the search has found after each level (see split_search_step)
  uint32_t pad[6];
  uint32_t hist_k[3][kBins];         // top-k search: how many weights fall into each bin
  uint32_t hist_pn[3][kBins];        // top-p search: how many (level 0: hist_k says it), and their mass
  u64 hist_pm[3][kBins];
};
static_assert(sizeof(SplitRow) % 16 == 0, "rows of scratch stay aligned");

__device__ __forceinline__ void part_range(int vocab, int parts, int part, int& lo, int& hi) {
  const int len = ((vocab + parts * 4 - 1) / (parts * 4)) * 4;
  lo = part * len < vocab ? part * len : vocab;
  hi = lo + len < vocab ? lo + len : vocab;
}

// A part's values in registers, sixteen a thread at most (kMaxPartLen), asked for in one go: thread t holds the
// four neighbours at lo + (j * kSampThreads + t) * 4 for j = 0 .. 3.  What a launch needs from other blocks (the row's
// largest logit, its histograms) is asked for at the same time, so that a launch is one trip to memory long.
constexpr int kPartQuads = kMaxPartLen / (4 * kSampThreads);
struct PartValues {
  float v[kPartQuads][4];
};
__device__ __forceinline__ void load_part(const float* __restrict__ x, int lo, int hi, PartValues& pv) {
  const bool vec = (((uintptr_t)(x + lo)) & 15) == 0;
#pragma unroll
  for (int j = 0; j < kPartQuads; ++j) {
    const int i = lo + (j * kSampThreads + (int)threadIdx.x) * 4;
    if (i + 4 <= hi && vec) {
      const float4 q = *reinterpret_cast<const float4*>(x + i);
      pv.v[j][0] = q.x, pv.v[j][1] = q.y, pv.v[j][2] = q.z, pv.v[j][3] = q.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) pv.v[j][e] = i + e < hi ? x[i + e] : 0.f;
    }
  }
}
__device__ __forceinline__ void store_part(float* __restrict__ x, int lo, int hi, const PartValues& pv) {
  const bool vec = (((uintptr_t)(x + lo)) & 15) == 0;
#pragma unroll
  for (int j = 0; j < kPartQuads; ++j) {
    const int i = lo + (j * kSampThreads + (int)threadIdx.x) * 4;
    if (i + 4 <= hi && vec) {
      *reinterpret_cast<float4*>(x + i) = make_float4(pv.v[j][0], pv.v[j][1], pv.v[j][2], pv.v[j][3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i + e < hi) x[i + e] = pv.v[j][e];
    }
  }
}
// f(value, index in the row) for the values that exist
template <typename F> __device__ __forceinline__ void for_part(const PartValues& pv, int lo, int hi, F f) {
#pragma unroll
  for (int j = 0; j < kPartQuads; ++j) {
    const int i = lo + (j * kSampThreads + (int)threadIdx.x) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (i + e < hi) f(pv.v[j][e], i + e);
  }
}

// launch 1: a part's largest logit; the row's histograms and total start at zero
__global__ void __launch_bounds__(kSampThreads)
split_max_kernel(const float* __restrict__ logits, int ld, int vocab, SplitRow* __restrict__ rows) {
  __shared__ ArgMax am[kSampWaves];
  const int row = blockIdx.x, parts = gridDim.y, part = blockIdx.y, tid = threadIdx.x;
  SplitRow& r = rows[row];
  const float* lr = logits + (size_t)row * ld;
  int lo, hi;
  part_range(vocab, parts, part, lo, hi);
  // (the histograms are 12 K words of 32 bits: every part clears a share)
  uint32_t* words = &r.hist_k[0][0];
  constexpr int kWords = (int)((sizeof(r.hist_k) + sizeof(r.hist_pn) + sizeof(r.hist_pm)) / 4);
  for (int i = part * kSampThreads + tid; i < kWords; i += parts * kSampThreads) words[i] = 0;
  if (part == 0 && tid == 0) r.total = 0;
  ArgMax a = {-INFINITY, 0x7fffffff};
  if (lo < hi) sweep(lr + lo, hi - lo, [&](float v, int i) { a = better(a, ArgMax{v, i + lo}); });
  a = block_argmax(a, am);
  if (tid == 0) {
    r.part_max_v[part] = a.v;
    r.part_max_i[part] = a.i;
  }
}

// the row's largest logit from its parts' (the same in every thread)
__device__ __forceinline__ ArgMax split_row_max(const SplitRow& r, int parts, int vocab) {
  ArgMax a = {-INFINITY, 0x7fffffff};
  for (int p = 0; p < parts; ++p) a = better(a, ArgMax{r.part_max_v[p], r.part_max_i[p]});
  if ((unsigned)a.i >= (unsigned)vocab) a.i = 0;       // a row of NaN has no largest value: still name a token
  return a;
}

// this block's counts (and masses) of a level, added to the row's
__device__ __forceinline__ void flush_histograms(SplitRow& r, int level, bool cut_k, bool cut_p, bool same_counts,
                                                 const uint32_t* hist_k, const uint32_t* hist_pn, const u64* hist_pm) {
  const int tid = threadIdx.x;
  if (cut_k || same_counts) {
    const uint32_t n = hist_k[tid];
    if (n) atomicAdd(&r.hist_k[level][tid], n);
  }
  if (cut_p) {
    if (!same_counts) {
      const uint32_t n = hist_pn[tid];
      if (n) atomicAdd(&r.hist_pn[level][tid], n);
    }
    const u64 m = hist_pm[tid];
    if (m) atomicAdd(&r.hist_pm[level][tid], m);
  }
}

// launch 2: the part's weights, their mass, and the histograms of the first ten bits; the default answer
__global__ void __launch_bounds__(kSampThreads)
split_weights_kernel(const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
                     const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                     float* __restrict__ weights, SplitRow* __restrict__ rows, int32_t* __restrict__ out_token,
                     float* __restrict__ out_logit, int cuts) {
  __shared__ uint32_t hist_k[kBins];
  __shared__ u64 hist_pm[kBins];
  __shared__ u64 wave_u64[kSampWaves];
  const int row = blockIdx.x, parts = gridDim.y, part = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  SplitRow& r = rows[row];
  const float* lr = logits + (size_t)row * ld;
  float* w = weights + (size_t)row * vocab;
  int lo, hi;
  part_range(vocab, parts, part, lo, hi);
  PartValues pv;
  load_part(lr, lo, hi, pv);
  const float temp = temperature[row];
  const int k = top_k[row];
  const float p = top_p[row];
  const ArgMax a = split_row_max(r, parts, vocab);
  if (part == 0 && tid == 0) {       // the answer of a greedy row, and of a row whose weights are no numbers
    out_token[row] = a.i;
    out_logit[row] = lr[a.i];
  }
  if (!(temp > 0.f)) return;
  const bool cut_k = cuts && k > 0 && k < vocab, cut_p = cuts && p < 1.0f, cut = cut_k || cut_p;
  hist_k[tid] = 0;
  hist_pm[tid] = 0;
  __syncthreads();
  const float inv_t = 1.4426950408889634f / temp;
  uint32_t hi_sum = 0, lo_sum = 0;
#pragma unroll
  for (int j = 0; j < kPartQuads; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) pv.v[j][e] = __builtin_amdgcn_exp2f((pv.v[j][e] - a.v) * inv_t);
  store_part(w, lo, hi, pv);
  for_part(pv, lo, hi, [&](float o, int) {
    uint32_t fh, fl;
    fixed_parts(o, fh, fl);
    hi_sum += fh;
    lo_sum += fl;
    if (cut) {
      const uint32_t bin = (__float_as_uint(o) >> 20) & (kBins - 1);
      atomicAdd(&hist_k[bin], 1u);
      if (cut_p) atomicAdd(&hist_pm[bin], ((u64)fh << 20) + fl);
    }
  });
  const u64 mass = wave_total(((u64)hi_sum << 20) + lo_sum);
  if (lane == 0) wave_u64[wave] = mass;
  __syncthreads();
  if (tid == 0) {
    u64 all = 0;
    for (int i = 0; i < kSampWaves; ++i) all += wave_u64[i];
    if (cut_p && all) atomicAdd(&r.total, all);
    if (!cut) {                      // everything is kept: the draw needs no more than this
      r.part_mass[part] = all;
      r.part_ties[part] = 0;
    }
  }
  if (cut) flush_histograms(r, 0, cut_k, cut_p, true, hist_k, hist_k, hist_pm);
}

// What the search has found so far: the bits of the two thresholds, what is still wanted below them, and how many
// weights share the bits.  Every launch takes the search one level further, from the histograms that the launch
// before it filled (the same steps as in sample_kernel, the same result in every thread of every block of the row);
// the row's first block leaves the state after its level in the row's scratch memory for the next launch.
__device__ SplitSearch split_search_step(SplitRow& r, int level, bool cut_k, bool cut_p, int k, float p,
                                         uint32_t* hist_k, uint32_t* hist_pn, u64* hist_pm, u64* wave_u64,
                                         uint32_t* wave_u32, int* sel_s, u64* rest_u64, uint32_t* rest_u32) {
  const int tid = threadIdx.x;
  // (this thread's bins, the state and the total are asked for together: one trip to memory)
  const uint32_t bin_k = r.hist_k[level][tid];
  const uint32_t bin_pn = level == 0 ? 0u : r.hist_pn[level][tid];
  const u64 bin_pm = r.hist_pm[level][tid];
  SplitSearch s = {0, 0, cut_k ? (uint32_t)k : 0u, 0, 0, 0, 0};
  if (level > 0) {
    s = r.search[level - 1];
  } else if (cut_p) {
    const u64 total = r.total;
    const double need = ceil((double)p * (double)total);
    s.want_p = need < 1.0 ? 1ull : (u64)need;
    if (s.want_p > total) s.want_p = total;
  }
  __syncthreads();
  hist_k[tid] = bin_k;
  hist_pn[tid] = level == 0 ? bin_k : bin_pn;
  hist_pm[tid] = bin_pm;
  __syncthreads();
  int sel;
  if (cut_k) {
    select_bin<uint32_t>(hist_k, s.want_k, sel, s.want_k, wave_u32, sel_s, rest_u32);
    if (sel < 0) sel = 0, s.want_k = 0x7fffffff;          // cannot happen: k < vocab weights exist
    s.bits_k = (s.bits_k << 10) | (uint32_t)sel;
    s.equal_k = hist_k[sel];
  }
  if (cut_p) {
    select_bin<u64>(hist_pm, s.want_p, sel, s.want_p, wave_u64, sel_s, rest_u64);
    if (sel < 0) sel = 0;                                 // cannot happen: want_p <= total
    s.bits_p = (s.bits_p << 10) | (uint32_t)sel;
    s.equal_p = hist_pn[sel];
  }
  __syncthreads();
  // (a record for every level: the other blocks of the row may still be reading the one before)
  if (blockIdx.y == 0 && tid == 0) r.search[level] = s;
  return s;
}

#define ATOMA_SPLIT_SEARCH_LDS                                                                     \
  __shared__ uint32_t hist_k[kBins];                                                               \
  __shared__ uint32_t hist_pn[kBins];                                                              \
  __shared__ u64 hist_pm[kBins];                                                                   \
  __shared__ u64 wave_u64[kSampWaves];                                                             \
  __shared__ uint32_t wave_u32[kSampWaves];                                                        \
  __shared__ int sel_s;                                                                            \
  __shared__ u64 rest_u64;                                                                         \
  __shared__ uint32_t rest_u32

// launches 3 and 4 (level 1 and 2): the histograms of the next ten bits, of the part's weights that share the bits
// found so far
__global__ void __launch_bounds__(kSampThreads)
split_level_kernel(int level, int vocab, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
                   const float* __restrict__ top_p, const float* __restrict__ weights, SplitRow* __restrict__ rows) {
  ATOMA_SPLIT_SEARCH_LDS;
  const int row = blockIdx.x, parts = gridDim.y, part = blockIdx.y, tid = threadIdx.x;
  const float temp = temperature[row];
  const int k = top_k[row];
  const float p = top_p[row];
  const bool cut_k = k > 0 && k < vocab, cut_p = p < 1.0f;
  if (!(temp > 0.f) || (!cut_k && !cut_p)) return;
  SplitRow& r = rows[row];
  const float* w = weights + (size_t)row * vocab;
  int lo, hi;
  part_range(vocab, parts, part, lo, hi);
  PartValues pv;
  load_part(w, lo, hi, pv);
  const SplitSearch s = split_search_step(r, level - 1, cut_k, cut_p, k, p, hist_k, hist_pn, hist_pm, wave_u64,
                                          wave_u32, &sel_s, &rest_u64, &rest_u32);
  hist_k[tid] = 0;
  hist_pn[tid] = 0;
  hist_pm[tid] = 0;
  __syncthreads();
  const int shift = 20 - 10 * level;
  for_part(pv, lo, hi, [&](float v, int) {
    const uint32_t b = __float_as_uint(v);
    const uint32_t high = b >> (shift + 10), bin = (b >> shift) & (kBins - 1);
    if (cut_k && high == s.bits_k) atomicAdd(&hist_k[bin], 1u);
    if (cut_p && high == s.bits_p) {
      atomicAdd(&hist_pn[bin], 1u);
      atomicAdd(&hist_pm[bin], fixed_of(v));
    }
  });
  __syncthreads();
  flush_histograms(r, level, cut_k, cut_p, false, hist_k, hist_pn, hist_pm);
}

// The cut that the search ends in: the threshold (as float bits), how many of the weights equal to it are kept
// (those of lowest index), how many there are.  As in sample_kernel.
struct SplitCut {
  uint32_t tau, n_equal;
  u64 ties_kept;
  bool all_ties;
};
__device__ __forceinline__ SplitCut split_cut(const SplitSearch& s, bool cut_k, bool cut_p) {
  SplitCut c = {0, 0xffffffffu, ~0ull, true};
  if (cut_k) {
    c.tau = s.bits_k;
    c.ties_kept = s.want_k;
    c.n_equal = s.equal_k;
  }
  if (cut_p) {
    const u64 each = fixed_of(__uint_as_float(s.bits_p));
    u64 ties = each ? (s.want_p + each - 1) / each : (u64)s.equal_p;
    if (ties < 1) ties = 1;
    if (ties > s.equal_p) ties = s.equal_p;
    if (!cut_k || s.bits_p > c.tau || (s.bits_p == c.tau && ties < c.ties_kept)) {
      c.tau = s.bits_p;
      c.ties_kept = ties;
      c.n_equal = s.equal_p;
    }
  }
  c.all_ties = c.ties_kept >= (u64)c.n_equal;
  return c;
}

// launch 5: the part's mass above the threshold and its number of weights equal to it
__global__ void __launch_bounds__(kSampThreads)
split_mass_kernel(int vocab, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
                  const float* __restrict__ top_p, const float* __restrict__ weights, SplitRow* __restrict__ rows) {
  ATOMA_SPLIT_SEARCH_LDS;
  const int row = blockIdx.x, parts = gridDim.y, part = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float temp = temperature[row];
  const int k = top_k[row];
  const float p = top_p[row];
  const bool cut_k = k > 0 && k < vocab, cut_p = p < 1.0f;
  if (!(temp > 0.f) || (!cut_k && !cut_p)) return;
  SplitRow& r = rows[row];
  const float* w = weights + (size_t)row * vocab;
  int lo, hi;
  part_range(vocab, parts, part, lo, hi);
  PartValues pv;
  load_part(w, lo, hi, pv);
  const SplitSearch s = split_search_step(r, 2, cut_k, cut_p, k, p, hist_k, hist_pn, hist_pm, wave_u64, wave_u32,
                                          &sel_s, &rest_u64, &rest_u32);
  const SplitCut c = split_cut(s, cut_k, cut_p);
  uint32_t hi_sum = 0, lo_sum = 0, ties = 0;
  for_part(pv, lo, hi, [&](float v, int) {
    const uint32_t b = __float_as_uint(v);
    if (b > c.tau) {
      uint32_t fh, fl;
      fixed_parts(v, fh, fl);
      hi_sum += fh;
      lo_sum += fl;
    } else if (b == c.tau) {
      ++ties;
    }
  });
  const u64 mass = wave_total(((u64)hi_sum << 20) + lo_sum);
  ties = wave_total(ties);
  __syncthreads();
  if (lane == 0) {
    wave_u64[wave] = mass;
    wave_u32[wave] = ties;
  }
  __syncthreads();
  if (tid == 0) {
    u64 m = 0;
    uint32_t t = 0;
    for (int i = 0; i < kSampWaves; ++i) m += wave_u64[i], t += wave_u32[i];
    r.part_mass[part] = m;
    r.part_ties[part] = t;
  }
}

// launch 6, a block a row: the part that holds u * (kept mass), and in it the first index at which the running sum
// of kept weights exceeds that.  A thread takes a run of neighbouring weights of the part, at most 32.
__global__ void __launch_bounds__(kSampThreads)
split_draw_kernel(const float* __restrict__ logits, int ld, int vocab, int parts, const float* __restrict__ temperature,
                  const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                  const float* __restrict__ uniform, const float* __restrict__ weights,
                  SplitRow* __restrict__ rows, int32_t* __restrict__ out_token, float* __restrict__ out_logit,
                  int cuts) {
  __shared__ u64 wave_u64[kSampWaves];
  __shared__ uint32_t wave_u32[kSampWaves];
  __shared__ int pick_s;
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (!(temperature[row] > 0.f)) return;
  const int k = top_k[row];
  const float p = top_p[row];
  const bool cut_k = cuts && k > 0 && k < vocab, cut_p = cuts && p < 1.0f, cut = cut_k || cut_p;
  SplitRow& r = rows[row];
  SplitCut c = {0, 0xffffffffu, ~0ull, true};
  if (cut) c = split_cut(r.search[2], cut_k, cut_p);    // (the search ended in the launch before this one)
  const u64 tie_mass = fixed_of(__uint_as_float(c.tau));
  // kept mass of every part: what lies above the threshold, and its share of the kept ties (the first in the row)
  u64 kept = 0, before = 0, ties_before = 0;
  int chosen = -1;
  u64 part_kept[kMaxParts];
  {
    u64 ties_seen = 0;
#pragma unroll
    for (int q = 0; q < kMaxParts; ++q) {
      if (q >= parts) {
        part_kept[q] = 0;
        continue;
      }
      u64 t = r.part_ties[q];
      u64 keep_t = t;
      if (!c.all_ties) {
        const u64 left = c.ties_kept > ties_seen ? c.ties_kept - ties_seen : 0;
        keep_t = t < left ? t : left;
      }
      part_kept[q] = r.part_mass[q] + (cut ? keep_t * tie_mass : 0);
      kept += part_kept[q];
      ties_seen += t;
    }
  }
  if (kept == 0) return;                           // weights that are no numbers: the default answer stands
  u64 target = (u64)((double)uniform[row] * (double)kept);
  if (target >= kept) target = kept - 1;           // (kept >= 2^40: the largest weight is always kept)
  {
    u64 run = 0, ties_seen = 0;
#pragma unroll
    for (int q = 0; q < kMaxParts; ++q) {
      if (q >= parts) continue;
      if (chosen < 0 && target < run + part_kept[q]) {
        chosen = q;
        before = run;
        ties_before = ties_seen;
      }
      run += part_kept[q];
      ties_seen += r.part_ties[q];
    }
  }
  if (chosen < 0) return;                          // (cannot happen: kept > target)
  const float* lr = logits + (size_t)row * ld;
  const float* w = weights + (size_t)row * vocab;
  int lo, hi;
  part_range(vocab, parts, chosen, lo, hi);
  // Each wave owns a contiguous stretch of the part, in pieces of 256 values (four neighbours a lane), all of them
  // in registers: ties first (a tie's rank is the number of ties before it in the row), then kept masses, then the
  // wave that holds the target walks its pieces with running sums over its lanes.
  constexpr int kPieces = kMaxPartLen / (kSampWaves * 256);
  const int stretch = ((hi - lo + kSampWaves * 256 - 1) / (kSampWaves * 256)) * 256;
  const int begin = lo + wave * stretch < hi ? lo + wave * stretch : hi;
  const int end = begin + stretch < hi ? begin + stretch : hi;
  const bool vec_w = (((uintptr_t)w) & 15) == 0;
  float v[kPieces][4];
  int n[kPieces];
  uint32_t ties[kPieces];
  uint32_t wave_ties = 0;
#pragma unroll
  for (int j = 0; j < kPieces; ++j) {
    const int i = begin + j * 256 + lane * 4;
    n[j] = end - i < 0 ? 0 : end - i > 4 ? 4 : end - i;
    if (n[j] == 4 && vec_w) {
      const float4 q = *reinterpret_cast<const float4*>(w + i);
      v[j][0] = q.x, v[j][1] = q.y, v[j][2] = q.z, v[j][3] = q.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[j][e] = e < n[j] ? w[i + e] : 0.f;
    }
    ties[j] = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) ties[j] += e < n[j] && __float_as_uint(v[j][e]) == c.tau;
    wave_ties += ties[j];
  }
  if (tid == 0) pick_s = -1;
  uint32_t rank_run = (uint32_t)ties_before;           // (ties are weights of the row: fewer than 2^31)
  if (!c.all_ties) {                                   // (a tie's rank matters only where some ties are dropped)
    wave_ties = wave_total(wave_ties);
    if (lane == 0) wave_u32[wave] = wave_ties;
    __syncthreads();
    for (int i = 0; i < wave; ++i) rank_run += wave_u32[i];
  }
  // the kept mass of the lane's values of piece j (in two parts), given the rank of its first tie
  auto lane_mass = [&](int j, uint32_t rank, bool* keep, uint32_t& hi_sum, uint32_t& lo_sum) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t bits = __float_as_uint(v[j][e]);
      keep[e] = e < n[j] && (bits > c.tau || (bits == c.tau && (c.all_ties || (u64)rank < c.ties_kept)));
      if (e < n[j] && bits == c.tau) ++rank;
      if (keep[e]) {
        uint32_t fh, fl;
        fixed_parts(v[j][e], fh, fl);
        hi_sum += fh;
        lo_sum += fl;
      }
    }
  };
  uint32_t rank_of[kPieces];
  u64 mass_of[kPieces];
  u64 wave_mass = 0;
#pragma unroll
  for (int j = 0; j < kPieces; ++j) {
    rank_of[j] = 0;
    if (!c.all_ties) {
      const uint32_t incl = wave_prefix(ties[j]);
      rank_of[j] = rank_run + incl - ties[j];
      rank_run += __shfl(incl, 63, 64);
    }
    bool keep[4];
    uint32_t hi_sum = 0, lo_sum = 0;
    lane_mass(j, rank_of[j], keep, hi_sum, lo_sum);
    mass_of[j] = ((u64)hi_sum << 20) + lo_sum;
    wave_mass += mass_of[j];
  }
  wave_mass = wave_total(wave_mass);
  if (lane == 0) wave_u64[wave] = wave_mass;
  __syncthreads();
  u64 run = before;
  for (int i = 0; i < wave; ++i) run += wave_u64[i];
  if (run <= target && target < run + wave_mass) {       // one wave at most: the sums rise with the wave
    int pick = -1;
#pragma unroll
    for (int j = 0; j < kPieces; ++j) {
      if (pick >= 0) continue;
      const u64 li = wave_prefix(mass_of[j]);
      const u64 whole = __shfl(li, 63, 64);
      if (run + whole > target) {
        const u64 ahead = __ballot(run + li > target);
        const int first = __ffsll((long long)ahead) - 1;
        int found = -1;
        if (lane == first) {
          bool keep[4];
          uint32_t hi_sum = 0, lo_sum = 0;
          lane_mass(j, rank_of[j], keep, hi_sum, lo_sum);
          u64 at = run + li - mass_of[j];
          for (int e = 0; e < 4; ++e) {
            if (!keep[e]) continue;
            at += fixed_of(v[j][e]);
            if (at > target) {
              found = begin + j * 256 + lane * 4 + e;
              break;
            }
          }
        }
        pick = __shfl(found, first, 64);
      }
      run += whole;
    }
    if (lane == 0) pick_s = pick;
  }
  __syncthreads();
  if (tid == 0 && pick_s >= 0) {
    out_token[row] = pick_s;
    out_logit[row] = lr[pick_s];
  }
}

// parts a row: so many that the blocks of all rows fill the GPU, and that a part's weights fit the draw's registers
static int split_parts(int n_rows, int vocab) {
  int parts = (256 + n_rows - 1) / n_rows;
  const int least = (vocab + kMaxPartLen - 1) / kMaxPartLen;
  parts = parts < least ? least : parts;
  return parts > kMaxParts ? (least <= kMaxParts ? kMaxParts : 0) : parts;
}

extern "C" size_t atoma_sample_split_scratch_bytes(int n_rows) { return (size_t)(n_rows > 0 ? n_rows : 0) * sizeof(SplitRow); }

// atoma_sample for steps in which rows draw: the same tokens from six short launches (see above).  scratch: at
// least atoma_sample_split_scratch_bytes(n_rows) bytes, 16-byte aligned, whatever they hold.  Vocabularies too
// large for sixteen parts (above 262,144) are refused: atoma_sample takes them.  cuts == 0: the caller knows that
// no row has a top-k or top-p cut; the three launches of the search are left out, and top_k and top_p are not read
// (a row that has a cut all the same is drawn from all of its weights).
extern "C" int atoma_sample_split(const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                                  const int32_t* top_k, const float* top_p, const float* uniform, float* weights,
                                  void* scratch, int cuts, int32_t* out_token, float* out_logit, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab || scratch == nullptr || ((uintptr_t)scratch & 15) != 0) return ATOMA_ERR_SHAPE;
  const int parts = split_parts(n_rows, vocab);
  if (parts <= 0) return ATOMA_ERR_SHAPE;
  SplitRow* rows = static_cast<SplitRow*>(scratch);
  const dim3 grid(n_rows, parts), block(kSampThreads);
  hipLaunchKernelGGL(split_max_kernel, grid, block, 0, stream, logits, ld, vocab, rows);
  hipLaunchKernelGGL(split_weights_kernel, grid, block, 0, stream, logits, ld, vocab, temperature, top_k, top_p, weights,
                     rows, out_token, out_logit, cuts);
  if (cuts) {
    for (int level = 1; level <= 2; ++level)
      hipLaunchKernelGGL(split_level_kernel, grid, block, 0, stream, level, vocab, temperature, top_k, top_p, weights,
                         rows);
    hipLaunchKernelGGL(split_mass_kernel, grid, block, 0, stream, vocab, temperature, top_k, top_p, weights, rows);
  }
  hipLaunchKernelGGL(split_draw_kernel, dim3(n_rows), block, 0, stream, logits, ld, vocab, parts, temperature, top_k,
                     top_p, uniform, weights, rows, out_token, out_logit, cuts);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// ---- sampling without a workspace argument and without any allocation (declared in sample_static.h) ----------
// The weights exp((l - max) / T) of all rows, which atoma_sample keeps in the caller's workspace, live here in an
// array of the code object.  Every device that loads this library holds its own copy at its own address until the
// process ends; host code may not use the array's name as an address, so the address is asked for once per device
// and kept.  All calls on one device share the array: two that overlap in time (two streams, two threads) race.
// Nothing in it has to start at zero: a sampled row writes all of its weights before it reads any of them.
#include "sample_static.h"
#include <mutex>

static __device__ __align__(256) float scratch[ATOMA_SAMPLE_STATIC_MAX_FLOATS];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
float* scratch_of_device[kMaxDevices] = {};       // device address of `scratch` on each device, once known

// the address of the current device's copy of `scratch`; a HIP error code (positive) through rc otherwise
float* scratch_address(int& rc) {
  rc = 0;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    rc = (int)e;
    return nullptr;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    rc = ATOMA_ERR_SHAPE;
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(scratch_mutex);
  if (scratch_of_device[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      rc = e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
      return nullptr;
    }
    scratch_of_device[dev] = static_cast<float*>(p);
  }
  return scratch_of_device[dev];
}
}  // namespace

extern "C" int atoma_sample_static_init(void) {
  int rc;
  scratch_address(rc);
  return rc;
}

extern "C" int atoma_sample_static(const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                                   const int32_t* top_k, const float* top_p, const float* uniform,
                                   int32_t* out_token, float* out_logit, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || ld < vocab) return ATOMA_ERR_SHAPE;
  if ((unsigned long long)n_rows * (unsigned long long)vocab > (unsigned long long)ATOMA_SAMPLE_STATIC_MAX_FLOATS)
    return ATOMA_ERR_TOO_LARGE;
  int rc;
  float* weights = scratch_address(rc);
  if (weights == nullptr) return rc;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows, sample_splits(n_rows, vocab)), dim3(kSampThreads), 0, stream, logits, ld,
                     vocab, temperature, top_k, top_p, uniform, weights, out_token, out_logit);
  ATOMA_LAUNCH_CHECK();
  return 0;
}
