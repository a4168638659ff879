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
