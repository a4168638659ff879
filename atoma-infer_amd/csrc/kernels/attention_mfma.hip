// bfloat16 attention over the paged cache on the matrix cores, for prompts, portions and decoded tokens alike.
// Compiled once per head size and page size: -DATOMA_HD=<multiple of 16, at most 256>, -DATOMA_PAGE=<tokens a page, a
// multiple of 16; 16 if not given>.
//
// Work is cut on the host into tasks, one per wave: 32 query rows against a range of keys.  A row is a
// (token, query head) pair of one request and one KV head: row r of a tile is head r / qt, token tok0 + r % qt,
// so the heads of a group share every key and value that is read (the reference does this only for some of its
// kernels: csrc/src/lib.rs:69-100).  The four waves of a workgroup run four consecutive tasks; the host orders
// tasks so that these read the same keys (the heads of one tile, or neighbouring key ranges of one request) and
// meet in the L1 cache.  A task either covers all keys its rows may see and writes the output, or covers one
// chunk of 128 to 512 keys and writes a partial result (normalised output and log-sum-exp); the wave that finishes a
// row piece's last chunk merges them (or, without counters, the combine kernel does):
// the split keeps the GPU busy when few rows face many keys (csrc/kernels/flash_fwd_kernel.h:1131-1310 is the
// reference's combine).  Chunk borders are multiples of the chunk size, so a partial result covers the same keys
// whatever else the batch holds.
//
// Per block of 32 keys (two runs of 16 tokens: two pages of 16 tokens, or two runs of one or of two larger pages),
// with v_mfma_f32_32x32x16_bf16:
//   S^T[key, row] = K[key, :] . Q[row, :]     K page rows are the A operand straight from global memory,
//                                             Q the B operand, kept in registers for the whole task;
//   online softmax down the keys of each row in float32 (exp2 with the scale folded in), masked by the row's
//   own position and window (bottom-right aligned causal mask, csrc/kernels/mask.h:171-192);
//   O^T[d, row] += V^T[d, key] . P^T[key, row]  S^T's accumulator layout is already the B operand layout, so
//                                             P goes from registers to the MFMA as bfloat16 without a
//                                             transpose, and V^T is how the cache stores values.
#include "common.h"

using namespace atoma;

#ifndef ATOMA_HD
#error "compile with -DATOMA_HD=<head size>"
#endif

constexpr int HD = ATOMA_HD;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");
constexpr int KSTEPS = HD / 16;        // MFMA steps over the head dimension for S
constexpr int DTILES = (HD + 31) / 32; // 32-row tiles of O^T
#ifndef ATOMA_PAGE
#define ATOMA_PAGE 16
#endif
constexpr int PAGE = ATOMA_PAGE;       // tokens a page
static_assert(PAGE % 16 == 0 && PAGE >= 16, "pages hold a multiple of 16 tokens");
constexpr int RUNS = PAGE / 16;        // runs of 16 tokens a page; a run of values is laid out as a page of 16 (cache_layout.h)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kSlack = 8.0f;   // see the softmax in the kernel

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

struct Task {
  int32_t entry;    // row of the block tables; < 0: nothing to do
  int32_t tok0;     // first token of the tile, counted inside the entry
  int32_t qt;       // tokens per head in the tile
  int32_t row0;     // first of this task's 32 rows inside the tile
  int32_t k_begin;  // keys [k_begin, k_end) by absolute position; k_begin is a multiple of 32
  int32_t k_end;
  int32_t dest;     // < 0: write the output; else index of the partial result
  int32_t n_parts;  // combine tasks: number of partial results starting at dest; tasks that leave a partial result:
                    // index of their combine task (the record that says where the row piece's parts start and how many)
  int32_t tok_base; // row of the entry's first token in the step's batch
  int32_t count;    // tokens of the entry in this step
  int32_t pos0;     // absolute position of the entry's first token
  int32_t tiles;    // pieces of 32 rows that the task covers from row0 on: 2 in launches of two-tile waves, else 0 or 1
};

// x of the lane 32 away, by one cross-half register swap (no trip through LDS as a shuffle would take)
__device__ __forceinline__ float from_other_half(float x, bool upper) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(upper ? r[0] : r[1]);
}

__device__ __forceinline__ bf16x8 pack8(const float* v) {
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = (__bf16)v[i];
  return r;
}


// Stores and loads that go through to memory, past the L2 of this wave's XCD (which the other XCDs' waves do not
// see): what a wave hands to a wave of another workgroup inside one launch.
__device__ __forceinline__ void store_through(float* p, float4 v) {
  unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
  const unsigned long long lo = (unsigned long long)__float_as_uint(v.x) | ((unsigned long long)__float_as_uint(v.y) << 32);
  const unsigned long long hi = (unsigned long long)__float_as_uint(v.z) | ((unsigned long long)__float_as_uint(v.w) << 32);
  __hip_atomic_store(q, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(q + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_through(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float4 load_through(const float* p) {
  const unsigned long long* q = reinterpret_cast<const unsigned long long*>(p);
  const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_float4(__uint_as_float((unsigned)lo), __uint_as_float((unsigned)(lo >> 32)), __uint_as_float((unsigned)hi),
                     __uint_as_float((unsigned)(hi >> 32)));
}
__device__ __forceinline__ float load_through1(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge the partial results of one piece of 32 rows, by one wave: out = sum_s w_s O_s / sum_s w_s with
// w_s = exp2(lse_s - max).  The live rows' values are dealt to the lanes four at a time; a lane walks the parts in the
// order of their index, BATCH in flight (each round a trip to memory: the fewer rounds the better, but the parts in
// flight need registers, and the launches that prompts use must not pay for them with a wave less a SIMD), and follows the
// running maximum as the attention loop does, so the result depends on the parts alone.  comb: the piece's combine record (dest: first part, n_parts: how many).
template <int BATCH>
__device__ __forceinline__ void merge_parts(const float* __restrict__ part_o, const float* __restrict__ part_lse,
                                            uint16_t* __restrict__ out, int out_stride, const Task& comb, int kvh,
                                            int nh, int nkv, int lane) {
  constexpr int Q = HD / 4;                        // pieces of four values in a row
  const int g = nh / nkv;
  const size_t part_stride = (size_t)nkv * 32;     // rows between two parts of the same (KV head, row)
  const size_t base0 = ((size_t)comb.dest * nkv + kvh) * 32;
  const int n_parts = comb.n_parts;
  for (int idx = lane; idx < 32 * Q; idx += 64) {
    const int c = idx / Q, d = (idx % Q) * 4;
    const int r = comb.row0 + c;
    const int hq = r / comb.qt, tok = comb.tok0 + r % comb.qt;
    if (hq >= g || tok >= comb.count) continue;
    const float* pl = part_lse + base0 + c;
    const float* po = part_o + (base0 + c) * HD + d;
    float m = -INFINITY, wsum = 0.f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < n_parts; s0 += BATCH) {
      float ls[BATCH];
      float4 v[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int sp = s0 + u < n_parts ? s0 + u : n_parts - 1;
        ls[u] = load_through1(pl + (size_t)sp * part_stride);
        v[u] = load_through(po + (size_t)sp * part_stride * HD);
      }
      float mb = m;
#pragma unroll
      for (int u = 0; u < BATCH; ++u)
        if (s0 + u < n_parts) mb = fmaxf(mb, ls[u]);
      const float m_use = (mb == -INFINITY) ? 0.f : mb;
      const float corr = __builtin_amdgcn_exp2f(m - m_use);      // exp2(-inf) = 0 on the first round
      wsum *= corr;
      acc.x *= corr, acc.y *= corr, acc.z *= corr, acc.w *= corr;
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        if (s0 + u < n_parts) {
          const float w = __builtin_amdgcn_exp2f(ls[u] - m_use);
          wsum += w;
          acc.x += w * v[u].x, acc.y += w * v[u].y, acc.z += w * v[u].z, acc.w += w * v[u].w;
        }
      }
      m = mb;
    }
    const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
    uint2 pk;
    pk.x = (uint32_t)f32_to_bf16_bits(acc.x * inv) | ((uint32_t)f32_to_bf16_bits(acc.y * inv) << 16);
    pk.y = (uint32_t)f32_to_bf16_bits(acc.z * inv) | ((uint32_t)f32_to_bf16_bits(acc.w * inv) << 16);
    *reinterpret_cast<uint2*>(out + (size_t)(comb.tok_base + tok) * out_stride + (size_t)(kvh * g + hq) * HD + d) = pk;
  }
}

// KSPLIT waves share a task: wave h of them takes the blocks of 32 keys number h, h + KSPLIT, ... of the task's
// range, and the KSPLIT partial results are merged through LDS at the end.  A wave walks its blocks one after the
// other at a pace set by latencies (MFMA, exponentials, cross-lane moves), not by any unit's throughput, and a
// launch lasts as long as its longest wave: with two waves per task the last tile of a long prompt, which sees
// all keys, takes half the time.  A workgroup runs TASKS tasks, so it has TASKS * KSPLIT waves:
//   4 x 1  decode steps of few requests: the tasks are short chunks of keys, merged by the second kernel;
//   4 x 2  prompts and mixed steps;
//   1 x 8  decode steps of many requests: a task is all keys of a request's token, so nothing is left to the
//          second kernel (there are enough requests and KV heads to fill the GPU without cutting keys into tasks).
// RT: pieces of 32 rows a wave works on, against the same keys: with two, every fragment of keys and values that a
// wave fetches, and the page and loop arithmetic of a block, serve 64 rows.  A wave's pace is set by its vector
// instructions (about a hundred a block and piece, a third of their time the sixteen exponentials), so portions
// behind long prefixes gain (2,048 tokens behind 30,720: 741 -> 682 us at head size 64, behind 63,488: 1,495 ->
// 1,355, behind 14,336: 376 -> 363); short prompts lose, because twice as few waves, each with a chain twice as
// long, fill the GPU worse.  The host asks for two pieces from 16,384 keys on.
template <int TASKS, int KSPLIT, int RT = 1>
__global__ void __launch_bounds__(64 * TASKS * KSPLIT)
attention_mfma_kernel(const Task* __restrict__ tasks, int n_tasks, int nkv, const uint16_t* __restrict__ q,
                      int q_stride, int nh, const int32_t* __restrict__ block_tables, int max_blocks, int window,
                      const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                      uint16_t* __restrict__ out, int out_stride, float* __restrict__ part_o,
                      float* __restrict__ part_lse, float scale, int32_t* __restrict__ counters) {
  // (the arguments come in the order in which a wave needs them: the first fourteen words, up to kcache, are in
  // scalar registers when the wave starts, the others are fetched from memory, a trip that the task record, the
  // queries, the page numbers and the first keys need not wait for)
  // (a wave's number is the same in all its lanes; saying so keeps what follows from it in scalar registers)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slot = wave % TASKS, part = wave / TASKS;   // which of the workgroup's tasks, which share of its keys
  // workgroups are numbered with the KV head running fastest: neighbours read the same block tables and finish
  // together, and the longest tasks (which come first) start first.  The GPU deals workgroups to its eight XCDs in
  // turn, so with eight KV heads (or a multiple) all tiles of a prompt that read one head's keys and values run on
  // one XCD and find them in its L2 (with the KV head running slowest a prompt of 2,048 tokens takes 48 us instead
  // of 37, a portion of 2,048 tokens behind 14,336 others 373 instead of 359; from 30,000 keys on it is all one).
  const int kvh = blockIdx.x % nkv;
  const int ti = (blockIdx.x / nkv) * TASKS + slot;
  // with KSPLIT > 1 every wave must reach the barrier below: a wave without work runs an empty range
  // (one load of the record: an empty one has an empty key range of its own)
  const Task task = tasks[ti < n_tasks ? ti : 0];
  const bool has_task = ti < n_tasks && task.entry >= 0;
  // (the record of the row piece that a chunk belongs to, for the wave that will merge the piece's chunks: asked for
  // now, it is a trip to memory less behind the last chunk)
  const Task comb = tasks[(has_task && task.dest >= 0 && counters != nullptr) ? n_tasks + task.n_parts : 0];
  if (KSPLIT == 1 && !has_task) return;
  const int g = nh / nkv;
  const int c = lane & 31, hg = lane >> 5;
  // the same in every lane; saying so keeps loop control and page arithmetic in scalar registers
  const int k_begin = __builtin_amdgcn_readfirstlane(task.k_begin);
  const int k_end = has_task ? __builtin_amdgcn_readfirstlane(task.k_end) : k_begin;
  const int entry = has_task ? __builtin_amdgcn_readfirstlane(task.entry) : 0;

  // this lane's row in each piece
  bool row_ok[RT];
  int trow[RT], p_row[RT], lo_row[RT], head[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int r = task.row0 + 32 * t + c;
    const int hq = r / task.qt, tok = task.tok0 + r % task.qt;
    row_ok[t] = has_task && hq < g && tok < task.count && (t == 0 || task.tiles > t);
    trow[t] = row_ok[t] ? task.tok_base + tok : 0;
    p_row[t] = row_ok[t] ? task.pos0 + tok : -1;
    lo_row[t] = (window > 0 && p_row[t] - window + 1 > 0) ? p_row[t] - window + 1 : 0;
    head[t] = kvh * g + (row_ok[t] ? hq : 0);
  }
  // a piece without a live row is skipped altogether (the same for all lanes)
  bool piece_on[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) piece_on[t] = RT == 1 || __ballot(row_ok[t]) != 0;

  // page numbers: lane i asks for page (kb / PAGE + i) of the task's request; lanes 0 and 1 hold the pages that the two
  // runs of 16 keys of the block at kb may lie in (with pages of 32, 64, ... tokens both in lane 0's).  Asked for at the
  // top of every turn for the next one, before anything else, so that waiting for the answer leaves the loads of
  // fragments behind it in flight.
  const int32_t* table = block_tables + (size_t)entry * max_blocks;
  auto page_window = [&](int kb) {
    int b = kb / PAGE + lane;
    if (b > max_blocks - 1) b = max_blocks - 1;
    return table[b];
  };
  // the second run's page among those lanes, and each run's place in its page (all the same in every lane)
  auto second_lane = [&](int kb) { return RUNS == 1 ? 1 : (kb + 16) / PAGE - kb / PAGE; };
  auto run_of = [&](int key) { return RUNS == 1 ? 0 : (key / 16) % RUNS; };

  // Q fragments: B operand, lane (row c, k half hg) holds 8 consecutive d per step
  bf16x8 qf[RT][KSTEPS];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const uint16_t* qp = q + (size_t)trow[t] * q_stride + (size_t)head[t] * HD + hg * 8;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) qf[t][s] = *reinterpret_cast<const bf16x8*>(qp + s * 16);
  }

  // the lowest own position and the highest window start among this wave's live rows: blocks wholly between
  // them need no mask.  (A lane without a live row must stay out of the minimum: with a zero of its own, every block
  // of a decode step, where 4 of a wave's 32 rows are live, would take the masked path.)
  int p_lo = 0x7fffffff, lo_hi = 0;
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (row_ok[t]) {
      p_lo = min(p_lo, p_row[t]);
      lo_hi = max(lo_hi, lo_row[t]);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    p_lo = min(p_lo, __shfl_xor(p_lo, off, 64));
    lo_hi = max(lo_hi, __shfl_xor(lo_hi, off, 64));
  }
  p_lo = __builtin_amdgcn_readfirstlane(p_lo);       // (all lanes hold the same by now)
  lo_hi = __builtin_amdgcn_readfirstlane(lo_hi);

  const float sc2 = scale * kLog2e;
  float m[RT], l[RT];
  f32x16 o[RT][DTILES];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    m[t] = -INFINITY, l[t] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[t][dt][i] = 0.f;
  }

  const size_t kv_head_stride = (size_t)PAGE * HD;            // one (page, head) tile
  const size_t page_stride = (size_t)nkv * kv_head_stride;

  // Page numbers are the same in all lanes, so a tile's address is scalar arithmetic and a lane adds its own
  // offset, which never changes: tile order (cache_layout.h): keys: for each 16 columns, the 8-column pieces of all 16
  // tokens side by side; values: this lane's eight key slots of column d are one 16-byte piece.
  const uint16_t* const k_tiles = kcache + (size_t)kvh * kv_head_stride;
  const uint16_t* const v_tiles = vcache + (size_t)kvh * kv_head_stride;
  const uint32_t k_lane = (uint32_t)(hg * PAGE + (c & 15)) * 8;
  auto load_keys = [&](int kb, int p0, int p1, bf16x8* kf) {
    // (a key's 8-column pieces lie PAGE * 8 elements apart, the tokens of a piece side by side: a run starts 16 * 8 in)
    const uint16_t* const t0 = k_tiles + (size_t)__builtin_amdgcn_readfirstlane(p0) * page_stride + run_of(kb) * 128;
    const uint16_t* const t1 = k_tiles + (size_t)__builtin_amdgcn_readfirstlane(p1) * page_stride + run_of(kb + 16) * 128;
    const uint16_t* kp = ((c < 16) ? t0 : t1) + k_lane;
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) kf[st] = *reinterpret_cast<const bf16x8*>(kp + st * (2 * PAGE * 8));
  };
  // V^T fragments of both pages: lane (d = dt*32 + c, key slots hg*4..+4 and 8 + hg*4..+4 of each page)
  auto load_vals = [&](int kb, int p0, int p1, bf16x8 (*vf)[DTILES]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint16_t* const tile = v_tiles + (size_t)__builtin_amdgcn_readfirstlane(j ? p1 : p0) * page_stride +
                                   run_of(kb + 16 * j) * (16 * HD);
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt) {
        const int d = dt * 32 + c;
        if (HD % 32 == 0 || d < HD) {
          constexpr int last_rows = HD % 32 == 0 ? 32 : HD % 32;
          const int rows = (HD % 32 == 0 || dt < DTILES - 1) ? 32 : last_rows;
          const uint32_t v_lane = (uint32_t)(dt * 512 + (hg * rows + c) * 8);
          vf[j][dt] = *reinterpret_cast<const bf16x8*>(tile + v_lane);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) vf[j][dt][i] = (__bf16)0.f;
        }
      }
    }
  };

  // Keys run one block ahead of the values.  A block's values are asked for when its turn begins and arrive while
  // S^T and the softmax run; the next block's keys are asked for as soon as S^T has used the registers of this
  // block's, and arrive while the softmax and the P.V products run.  So no fragment needs registers of its own to wait
  // in.  Every turn but the last issues the same loads, none of them under a condition (the last turn is a copy of
  // the code without them), which lets the compiler wait for exactly the loads a product needs and leave the younger
  // ones in flight.
  constexpr int STRIDE = 32 * KSPLIT;
  const int k_first = k_begin + 32 * part;
  bf16x8 kf[KSTEPS];
  bf16x8 vf[2][DTILES];
  int p0 = 0, p1 = 0;
  if (k_first < k_end) {
    const int pw = page_window(k_first);
    p0 = __builtin_amdgcn_readlane(pw, 0);
    p1 = __builtin_amdgcn_readlane(pw, second_lane(k_first));
    load_keys(k_first, p0, p1, kf);
  }
  auto turn = [&](int kb, auto more) {
    constexpr bool MORE = decltype(more)::value;
    int pw = 0;
    if constexpr (MORE) pw = page_window(kb + STRIDE);
    load_vals(kb, p0, p1, vf);
    // (no instruction: it keeps the compiler from moving these loads down to where their values are used)
    asm volatile("" ::: "memory");
    // S^T = K Q^T, for each piece of rows against the same fragments of the keys
    f32x16 s[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[t][i] = 0.f;
      if (piece_on[t]) {
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st)
          s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[st], qf[t][st], s[t], 0, 0, 0);
      }
    }
    if constexpr (MORE) {
      p0 = __builtin_amdgcn_readlane(pw, 0);
      p1 = __builtin_amdgcn_readlane(pw, second_lane(kb + STRIDE));
      load_keys(kb + STRIDE, p0, p1, kf);
      asm volatile("" ::: "memory");
    }

    // Online softmax; accumulator element i is key kb + (i/4)*8 + hg*4 + i%4.  The running maximum is kept in
    // units of the scaled score (score * scale * log2 e), so one fused multiply-add feeds exp2.  Only blocks
    // that touch a row's own position, the window's edge or the end of the key range need the mask.
    const bool edge = kb + 31 > p_lo || kb < lo_hi || kb + 32 > k_end;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      if (!piece_on[t]) continue;
      float sv[16];
      float bmax = -INFINITY;
      if (edge) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kb + (i >> 2) * 8 + hg * 4 + (i & 3);
          const bool ok = key <= p_row[t] && key >= lo_row[t] && key < k_end;
          sv[i] = ok ? s[t][i] : -INFINITY;
          bmax = fmaxf(bmax, sv[i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          sv[i] = s[t][i];
          bmax = fmaxf(bmax, sv[i]);
        }
      }
      bmax = fmaxf(bmax, from_other_half(bmax, hg != 0)) * sc2;
      // The reference point m of a row's exponentials follows its maximum only in jumps: as long as no row of the
      // wave has grown by more than kSlack (in powers of two) beyond its m, m stays, the weights may exceed one (by
      // at most 2^kSlack, nothing to float32 sums or to bfloat16 weights, whose precision is relative) and the
      // accumulators need no rescaling, which is most of a block's vector work.  out = o / l does not depend on m.
      const float m_new = fmaxf(m[t], bmax);
      const bool grew = __ballot(m_new > m[t] + kSlack) != 0;    // (-inf + kSlack = -inf: a row's first key always counts)
      if (grew) {
        const float corr = __builtin_amdgcn_exp2f(m[t] - ((m_new == -INFINITY) ? 0.f : m_new));
        l[t] *= corr;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[t][dt][i] *= corr;
        m[t] = m_new;
      }
      const float m_use = (m[t] == -INFINITY) ? 0.f : m[t];
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        sv[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], sc2, -m_use));
        psum += sv[i];
      }
      l[t] += psum;      // this lane's half of the row's sum; the halves meet after the last block

      // O^T += V^T P^T
      const bf16x8 pf0 = pack8(sv), pf1 = pack8(sv + 8);
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt) {
        o[t][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[0][dt], pf0, o[t][dt], 0, 0, 0);
        o[t][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[1][dt], pf1, o[t][dt], 0, 0, 0);
      }
    }
  };
  int kb = k_first;
  for (; kb + STRIDE < k_end; kb += STRIDE) turn(kb, std::true_type{});
  if (kb < k_end) turn(kb, std::false_type{});

  if constexpr (KSPLIT > 1) {
    // Merge the shares of a task: the waves with part > 0 lay down (m, l, o), lane by lane; the wave with part 0
    // rescales all to the common maximum and adds them in order.  Same lanes hold the same (row, column) in all.
    // (the launch asks for (KSPLIT - 1) * TASKS * PER_LANE * 64 floats of LDS: more than the 64 KB that a kernel may
    // declare for itself when heads are wide, hence not declared here)
    constexpr int PER_LANE = RT * (DTILES * 16 + 2);
    extern __shared__ float merge[];
    if (part > 0) {
      float* dst = merge + (size_t)((part - 1) * TASKS + slot) * PER_LANE * 64 + lane;
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        float* d2 = dst + (size_t)t * (DTILES * 16 + 2) * 64;
        d2[0] = m[t];
        d2[64] = l[t];
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) d2[(2 + dt * 16 + i) * 64] = o[t][dt][i];
      }
    }
    __syncthreads();
    if (part > 0 || !has_task) return;
#pragma unroll
    for (int h = 1; h < KSPLIT; ++h) {
      const float* src = merge + (size_t)((h - 1) * TASKS + slot) * PER_LANE * 64 + lane;
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const float* s2 = src + (size_t)t * (DTILES * 16 + 2) * 64;
        const float m2 = s2[0], l2 = s2[64];
        const float m_all = fmaxf(m[t], m2);
        const float m_use = (m_all == -INFINITY) ? 0.f : m_all;
        const float a = __builtin_amdgcn_exp2f(m[t] - m_use), b2 = __builtin_amdgcn_exp2f(m2 - m_use);
        l[t] = l[t] * a + l2 * b2;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[t][dt][i] = o[t][dt][i] * a + s2[(2 + dt * 16 + i) * 64] * b2;
        m[t] = m_all;
      }
    }
  }

  // a row's sum of weights: its two lanes have each summed the keys they hold (both scaled by the same m)
#pragma unroll
  for (int t = 0; t < RT; ++t) l[t] += from_other_half(l[t], hg != 0);

  // accumulator element i of tile dt is d = dt*32 + (i/4)*8 + hg*4 + i%4 of row c
  if (task.dest < 0) {
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      if (!row_ok[t]) continue;
      const float inv = l[t] > 0.f ? 1.0f / l[t] : 0.f;
      uint16_t* op = out + (size_t)trow[t] * out_stride + (size_t)head[t] * HD;
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int d = dt * 32 + q4 * 8 + hg * 4;
          if (HD % 32 == 0 || d < HD) {
            uint2 v;
            v.x = (uint32_t)f32_to_bf16_bits(o[t][dt][q4 * 4 + 0] * inv) |
                  ((uint32_t)f32_to_bf16_bits(o[t][dt][q4 * 4 + 1] * inv) << 16);
            v.y = (uint32_t)f32_to_bf16_bits(o[t][dt][q4 * 4 + 2] * inv) |
                  ((uint32_t)f32_to_bf16_bits(o[t][dt][q4 * 4 + 3] * inv) << 16);
            *reinterpret_cast<uint2*>(op + d) = v;
          }
        }
    }
  } else {
    // a partial result is one piece of 32 rows (the host gives such tasks one piece, whatever RT is);
    // rows that are not live are never read by the merge (their log-sum-exp is, and says -inf)
    const float inv = l[0] > 0.f ? 1.0f / l[0] : 0.f;
    float* po = part_o + (((size_t)task.dest * nkv + kvh) * 32 + c) * HD;
    const bool merge_here = counters != nullptr;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = dt * 32 + q4 * 8 + hg * 4;
        if (row_ok[0] && (HD % 32 == 0 || d < HD)) {
          float4 v = make_float4(o[0][dt][q4 * 4 + 0] * inv, o[0][dt][q4 * 4 + 1] * inv, o[0][dt][q4 * 4 + 2] * inv,
                                 o[0][dt][q4 * 4 + 3] * inv);
          if (merge_here) store_through(po + d, v);
          else *reinterpret_cast<float4*>(po + d) = v;
        }
      }
    const float lse = l[0] > 0.f ? m[0] + __builtin_amdgcn_logf(l[0]) : -INFINITY;
    float* pl = part_lse + ((size_t)task.dest * nkv + kvh) * 32 + c;
    if (hg == 0) {
      if (merge_here) store_through(pl, lse);
      else *pl = lse;
    }
    if (merge_here) {
      // The wave that finishes the last chunk of a row piece merges all of its chunks.  The parts go through to memory
      // (stores and loads that pass the L2 of this wave's XCD, which other XCDs do not see), this wave's stores have
      // arrived before it counts itself in, and the counter is a device-wide atomic: no fence that would write back or
      // invalidate a whole cache is needed.  The parts are added in the order of their index, whoever comes last.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0);
      int32_t* counter = counters + (size_t)task.n_parts * nkv + kvh;
      int before = 0;
      if (lane == 0) before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      before = __builtin_amdgcn_readfirstlane(before);
      if (before + 1 == comb.n_parts) {
        if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        // (a wave a task: the launches of decoded tokens alone, which have registers to spare)
        merge_parts<(KSPLIT == 1 ? 16 : 12)>(part_o, part_lse, out, out_stride, comb, kvh, nh, nkv, lane);
      }
    }
  }
}

// Merge partial results: out = sum_s w_s O_s / sum_s w_s with w_s = exp2(lse_s - max lse).
// The kernel of its own, for callers that bring no counters (the attention kernel then leaves the parts to it).
// With counters the last wave to finish a row piece's chunks merges them inside the attention kernel: done with
// device-scope fences around the counter that measured far dearer than this second launch (a decode step 1.6 times as
// long: such fences write back and invalidate the L2 of the wave's XCD), done with stores and loads that go through
// to memory it saves the launch.
// One block per (combine task, KV head).  The log-sum-exps of all parts are first brought into LDS by all
// threads at once and turned into weights there; then the valid rows of the task (group x tokens, at most 32)
// times HD output values are spread over the 256 threads, and each adds its parts in order of their index with
// eight loads in flight.
constexpr int kCombineParts = 128;   // parts whose weights fit in LDS at once; more are merged in rounds

__global__ void __launch_bounds__(256)
attention_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_lse,
                         uint16_t* __restrict__ out, int out_stride, const Task* __restrict__ tasks, int nh,
                         int nkv) {
  __shared__ float wts[kCombineParts][32];
  __shared__ float row_max[32];
  const Task task = tasks[blockIdx.x];
  if (task.entry < 0) return;
  const int kvh = blockIdx.y, g = nh / nkv;
  const int tok_base = task.tok_base, count = task.count;
  const size_t part_stride = (size_t)nkv * 32;   // rows between two partial results of the same (KV head, row)
  const size_t base0 = ((size_t)task.dest * nkv + kvh) * 32;
  const int tid = threadIdx.x;

  // the largest log-sum-exp of every row, over all parts
  {
    const int c = tid & 31, lane_part = tid >> 5;   // 8 parts at a time per row
    float mx = -INFINITY;
    for (int s = lane_part; s < task.n_parts; s += 8) mx = fmaxf(mx, part_lse[base0 + s * part_stride + c]);
    wts[lane_part][c] = mx;
    __syncthreads();
    if (tid < 32) {
      float m2 = wts[0][tid];
#pragma unroll
      for (int i = 1; i < 8; ++i) m2 = fmaxf(m2, wts[i][tid]);
      row_max[tid] = m2;
    }
    __syncthreads();
  }

  float acc[(32 * HD + 255) / 256];
  float wsum[(32 * HD + 255) / 256];
#pragma unroll
  for (int i = 0; i < (32 * HD + 255) / 256; ++i) acc[i] = wsum[i] = 0.f;

  for (int p0 = 0; p0 < task.n_parts; p0 += kCombineParts) {
    const int np = task.n_parts - p0 < kCombineParts ? task.n_parts - p0 : kCombineParts;
    __syncthreads();
    for (int i = tid; i < np * 32; i += 256) {
      const int s = i >> 5, c = i & 31;
      wts[s][c] = __builtin_amdgcn_exp2f(part_lse[base0 + (size_t)(p0 + s) * part_stride + c] - row_max[c]);
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < (32 * HD + 255) / 256; ++it) {
      const int idx = tid + it * 256;
      const int c = idx / HD, d = idx % HD;
      const int r = task.row0 + c;
      const int hq = r / task.qt, tok = task.tok0 + r % task.qt;
      if (idx >= 32 * HD || hq >= g || tok >= count) continue;
      const float* po = part_o + (base0 + (size_t)p0 * part_stride + c) * HD + d;
      int s = 0;
      for (; s + 8 <= np; s += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = po[(size_t)(s + u) * part_stride * HD];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          acc[it] += wts[s + u][c] * v[u];
          wsum[it] += wts[s + u][c];
        }
      }
      for (; s < np; ++s) {
        acc[it] += wts[s][c] * po[(size_t)s * part_stride * HD];
        wsum[it] += wts[s][c];
      }
    }
  }
#pragma unroll
  for (int it = 0; it < (32 * HD + 255) / 256; ++it) {
    const int idx = tid + it * 256;
    const int c = idx / HD, d = idx % HD;
    const int r = task.row0 + c;
    const int hq = r / task.qt, tok = task.tok0 + r % task.qt;
    if (idx >= 32 * HD || hq >= g || tok >= count) continue;
    out[(size_t)(tok_base + tok) * out_stride + (size_t)(kvh * g + hq) * HD + d] =
        f32_to_bf16_bits(acc[it] / wsum[it]);
  }
}

// the merge needs (DTILES * 16 + 2) floats per lane of (KSPLIT - 1) * TASKS waves in LDS: 4 waves for 4 x 2, 7 for 1 x 8;
// a workgroup may have the 160 KB of a CU
constexpr size_t kLdsBytes = 160 * 1024;
constexpr size_t kMerge2Bytes = (DTILES * 16 + 2) * 64 * 4 * sizeof(float);
constexpr size_t kMerge4Bytes = (DTILES * 16 + 2) * 64 * 6 * sizeof(float);      // two tasks, three waves each
constexpr size_t kMerge8Bytes = (DTILES * 16 + 2) * 64 * 7 * sizeof(float);
constexpr bool kSplit2Fits = kMerge2Bytes <= kLdsBytes;
constexpr bool kSplit4Fits = kMerge4Bytes <= kLdsBytes;
constexpr bool kSplit8Fits = kMerge8Bytes <= kLdsBytes;
// two pieces of rows a wave: where the accumulators of both fit the registers of eight waves a workgroup, and the
// merge of two waves a task (twice as large) lets two workgroups share a CU
constexpr bool kTwoPieces = HD <= 64;

// A kernel that wants more than 64 KB of LDS at launch must be told so once per device: every instance of the
// template keeps, per device, whether it has been (a driver call per launch would sit on the path of every layer of
// every step, and inside the recording of decode graphs).  An instance always asks for the same number of bytes.
constexpr int kMaxDevices = 64;
template <typename K> static int allow_lds(K kernel, size_t bytes) {
  if (bytes <= 65536) return 0;
  static bool told[kMaxDevices] = {};
  int dev = 0;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev >= 0 && dev < kMaxDevices && told[dev]) return 0;
  const int rc = (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (rc == 0 && dev >= 0 && dev < kMaxDevices) told[dev] = true;
  return rc;
}

extern "C" int atoma_attention_mfma_head_size() { return HD; }
extern "C" int atoma_attention_mfma_page_size() { return PAGE; }
extern "C" int atoma_attention_mfma_max_ksplit() { return kSplit8Fits ? 8 : kSplit2Fits ? 2 : 1; }
extern "C" int atoma_attention_mfma_max_row_tiles() { return kTwoPieces ? 2 : 1; }

// tasks: device array of n_tasks Task records (main kernel), followed by n_combine records of the row pieces whose
// keys are cut into chunks.  counters: null, or n_combine * nkv zeros (left as zeros again): the attention kernel then
// merges the chunks itself and the combine kernel does not run.
extern "C" int atoma_attention_mfma(const void* q, int q_stride, const void* kcache, const void* vcache, void* out,
                                    int out_stride, float* part_o, float* part_lse, const int32_t* tasks, int n_tasks,
                                    int n_combine, const int32_t* block_tables, int max_blocks, float scale,
                                    int window, int nh, int nkv, int ksplit, int row_tiles, int32_t* counters,
                                    hipStream_t stream) {
  if (n_tasks <= 0) return 0;
  // row_tiles: 1, or 2: the tasks that write the output cover 64 rows (Task::tiles says so), two waves a task
  if (row_tiles != 1 && !(row_tiles == 2 && kTwoPieces && ksplit == 2)) return ATOMA_ERR_SHAPE;
  if (nkv <= 0 || nh % nkv || nkv > 65535 || max_blocks <= 0 || (q_stride & 7) || (out_stride & 3) ||
      ((uintptr_t)q & 15) || ((uintptr_t)out & 7))
    return ATOMA_ERR_SHAPE;
  const Task* t = reinterpret_cast<const Task*>(tasks);
  // ksplit: waves that share a task's keys: 1, 2 (four tasks a workgroup) or 8 (one task a workgroup), the latter
  // two for head sizes whose merge fits in LDS
#define ATOMA_ATTN(T, KS, BYTES, ...)                                                                              \
  do {                                                                                                             \
    const int rc_lds = allow_lds(attention_mfma_kernel<T, KS, ##__VA_ARGS__>, BYTES);                              \
    if (rc_lds != 0) return rc_lds;                                                                                \
    hipLaunchKernelGGL((attention_mfma_kernel<T, KS, ##__VA_ARGS__>), dim3(((n_tasks + T - 1) / T) * nkv),        \
                       dim3(64 * T * KS), BYTES,                                                                   \
                       stream, t, n_tasks, nkv, (const uint16_t*)q, q_stride, nh, block_tables, max_blocks,        \
                       window, (const uint16_t*)kcache, (const uint16_t*)vcache, (uint16_t*)out, out_stride,       \
                       part_o, part_lse, scale, counters);                                                         \
  } while (0)
  if (ksplit == 1) ATOMA_ATTN(4, 1, 0);
  else if (ksplit == 2 && row_tiles == 2) ATOMA_ATTN(4, 2, 2 * kMerge2Bytes, (kTwoPieces ? 2 : 1));
  else if (ksplit == 2 && kSplit2Fits) ATOMA_ATTN(4, (kSplit2Fits ? 2 : 1), kMerge2Bytes);
  else if (ksplit == 4 && kSplit4Fits) ATOMA_ATTN(2, (kSplit4Fits ? 4 : 1), kMerge4Bytes);
  else if (ksplit == 8 && kSplit8Fits) ATOMA_ATTN(1, (kSplit8Fits ? 8 : 1), kMerge8Bytes);
  else return ATOMA_ERR_SHAPE;
#undef ATOMA_ATTN
  ATOMA_LAUNCH_CHECK();
  if (n_combine > 0 && counters == nullptr) {
    hipLaunchKernelGGL(attention_combine_kernel, dim3(n_combine, nkv), dim3(256), 0, stream, part_o, part_lse,
                       (uint16_t*)out, out_stride, t + n_tasks, nh, nkv);
    ATOMA_LAUNCH_CHECK();
  }
  return 0;
}
