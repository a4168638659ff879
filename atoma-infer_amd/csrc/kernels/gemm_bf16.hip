// bfloat16 x bfloat16 products on the matrix cores for few rows of activations (decode and short portions):
// C[M, N] = A[M, K] * W[N, K]^T with float32 accumulation, W streamed from HBM once.
//
// The product is bound by the bytes of W.  A wave owns RT tiles of 16 rows of W and multiplies them against up to
// MT tiles of 16 rows of A with v_mfma_f32_16x16x32_bf16: the W tile is the MFMA's A operand (lane l: row l%16,
// eight consecutive k at (l/16)*8), the activations its B operand (lane l: row of A l%16, the same eight k), so
// both are 16-byte loads straight from global memory and nothing passes through LDS on the way in.
// The waves of a workgroup either take different rows of W (WK = 1, four waves) or split K four or eight ways for
// the same rows and add their accumulators in LDS (WK = 4, 8), which keeps enough loads in flight when N is small.
// K can additionally be split across blockIdx.y; then each slice writes its own float32 plane
// C[slice][M][N] and the consumer adds the planes (the fused residual-add + RMSNorm kernel does).
// Each output's sum order depends only on (K, WK, slices), never on M or on the row's place in the batch.
//
// Needs K % (32 * WK * slices) == 0 and 16-byte aligned rows; the host wrapper checks and otherwise refuses.
#include "common.h"
#include "cache_layout.h"

using namespace atoma;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// What the rotary epilogue needs beside the product: see the ROPE branch below.
struct RopeArgs {
  const int32_t* positions;      // [M]
  const float* cos_t;            // [positions, hd / 2]
  const float* sin_t;
  uint16_t* kcache;              // [pages, nkv, page_size * hd] tiles, bfloat16
  uint16_t* vcache;
  const int32_t* slot_mapping;   // [M]; negative: no cache write for the row
  int page_size, nh, nkv, hd;
};

// Outputs n0 .. n0 + 3 of row `row` of the fused q, k, v projection (float32 sums x0 .. x3), with the rows of every q
// and k head ordered so that the members of rotary pair i = (column i, column i + hd/2) are outputs 2i and 2i + 1 of
// the head: the four are two whole pairs, i and i + 1.  They are rotated here and go to their own columns: q to
// q_out [M, nh * hd], k into the row's slot of the paged cache (the order inside a tile: cache_layout.h); v heads are
// copied into theirs.  The same arithmetic as the rotary kernel (csrc/kernels/rotary.h:116-131 of the reference), on
// the float32 sums before they are rounded.
__device__ __forceinline__ void rope_store4(float x0, float x1, float x2, float x3, int row, int n0, const RopeArgs& ra,
                                            uint16_t* __restrict__ q_out, int ldq) {
  const int hd = ra.hd, half = hd >> 1;
  const int head = n0 / hd, d0 = n0 % hd;
  if (head >= ra.nh + ra.nkv) {
    const int slot = ra.slot_mapping[row];
    if (slot < 0) return;
    const int page = slot / ra.page_size, off = slot % ra.page_size;
    uint16_t* tile = ra.vcache + ((size_t)page * ra.nkv + (head - ra.nh - ra.nkv)) * ra.page_size * hd;
    tile[value_offset(d0, off, hd, ra.page_size)] = f32_to_bf16_bits(x0);
    tile[value_offset(d0 + 1, off, hd, ra.page_size)] = f32_to_bf16_bits(x1);
    tile[value_offset(d0 + 2, off, hd, ra.page_size)] = f32_to_bf16_bits(x2);
    tile[value_offset(d0 + 3, off, hd, ra.page_size)] = f32_to_bf16_bits(x3);
    return;
  }
  const int i = d0 >> 1;                       // even: columns i, i + 1 and their partners lie together
  const size_t at = (size_t)ra.positions[row] * half + i;
  const float c0 = ra.cos_t[at], s0 = ra.sin_t[at], c1 = ra.cos_t[at + 1], s1 = ra.sin_t[at + 1];
  const uint32_t lo = (uint32_t)f32_to_bf16_bits(x0 * c0 - x1 * s0) |
                      ((uint32_t)f32_to_bf16_bits(x2 * c1 - x3 * s1) << 16);      // columns i, i + 1
  const uint32_t hi = (uint32_t)f32_to_bf16_bits(x1 * c0 + x0 * s0) |
                      ((uint32_t)f32_to_bf16_bits(x3 * c1 + x2 * s1) << 16);      // i + half, i + half + 1
  if (head < ra.nh) {
    uint16_t* q = q_out + (size_t)row * ldq + (size_t)head * hd;
    *reinterpret_cast<uint32_t*>(q + i) = lo;
    *reinterpret_cast<uint32_t*>(q + i + half) = hi;
    return;
  }
  const int slot = ra.slot_mapping[row];
  if (slot < 0) return;
  const int page = slot / ra.page_size, off = slot % ra.page_size;
  uint16_t* tile = ra.kcache + ((size_t)page * ra.nkv + (head - ra.nh)) * ra.page_size * hd;
  *reinterpret_cast<uint32_t*>(tile + key_offset(off, i, ra.page_size)) = lo;
  *reinterpret_cast<uint32_t*>(tile + key_offset(off, i + half, ra.page_size)) = hi;
}

// A norm that is finished by its neighbours (at most 16 rows of activations).
//   In: the rows of A are residual rows times the norm's weight, not yet divided by their root mean square; the
//   sums of squares of the residual rows arrive as ss_in [parts_in][16] (a part per producing wave), and every sum
//   of this product is multiplied by 1 / sqrt(sum_p ss_in[p][row] / width_in + eps_in) before its epilogue: the
//   product is linear in its rows, so this is the product of the normed rows.
//   Out (resid != null): the product is not stored; it is added to the float32 residual rows resid [M][N] in
//   place, u_out [M][N] receives residual times gamma as bfloat16 (the A of the next product) and ss_out
//   [waves][16] each wave's share of the rows' sums of squares (the next product's ss_in).
struct FuseArgs {
  const float* ss_in;
  int parts_in;
  float eps_in, inv_width_in;
  float* resid;
  const void* gamma;       // [N] norm weight of the following norm
  int gamma_is_bf16;
  uint16_t* u_out;
  float* ss_out;
};

// HALF (one tile of W, at most 16 rows of A, the residual epilogue): a wave owns 8 rows of W, not 16, so that twice
// as many workgroups share a small N; what a workgroup may have in flight, not the matrix cores, is what bounds
// these products.  The lanes of the tile's other 8 rows load the same 8 rows of W 32 values of K further on, so a
// step covers 64 values of K and every lane's load is used: the step's two MFMAs take the one fragment of W
// against the activations of its first and of its second 32 values, into two accumulators; rows 0..7 of the first
// and rows 8..15 of the second are the wave's sums (the other halves are products of mismatched K and are dropped),
// and they meet once, after the last step.
// PACK (half tiles, at most 8 rows of A): the activations are packed the same way, lanes 8..15 holding rows 0..7 of
// A 32 values of K further on, so one fragment of A and one MFMA a step serve both halves: the quadrant (rows 0..7 of
// W, rows 0..7 of A) holds the sums over the first 32 values of every step, the quadrant (8..15, 8..15) those over the
// second, and they meet once, after the last step.  Half as many loads of the activations, which every workgroup
// fetches whole.
// TILED: W is not row-major but laid out at load time in the order in which this kernel's waves read it (see
// atoma_gemm_bf16_tiled_offset): tiles of 16 rows x 32 values of K in the lanes' order (1 KB, one load of a wave),
// ordered by batch of U steps, then workgroup, wave, step, tile.  All the workgroups of a launch walk their batches at
// about the same pace, so at any moment the loads in flight cover one stretch of memory that moves from the front of
// the matrix to its back, as a plain streaming read does, where row-major rows have every wave fetch 64-byte
// pieces 2 * K bytes apart (loads alone, the gate-up matrix of Llama 1B: 11.5 against 13.3 us).
// The arguments of gemm_skinny_kernel behind k_len as they lie in its argument segment (the layout of a C struct of
// the parameters in their order): three pointers and eight ints lie before them.
struct SkinnyLateArgs {
  size_t plane;
  RopeArgs ra;
  FuseArgs fa;
};
constexpr int kSkinnyLateArgsOffset = 3 * 8 + 8 * 4;
static_assert(kSkinnyLateArgsOffset % alignof(SkinnyLateArgs) == 0, "plane follows k_len without padding");

template <int MT, int RT, int WN, int WK, typename TC, bool SWIGLU = false, bool ROPE = false, int UO = 0,
          bool HALF = false, bool PACK = false, int TILED = 0>
__global__ void __launch_bounds__(64 * WN * WK)
gemm_skinny_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, TC* __restrict__ c, int M, int N,
                   int K, int lda, int ldw, int ldc, int grid_slices, int k_len, size_t plane_arg, RopeArgs ra_arg,
                   FuseArgs fa_arg) {
  // (The first arguments, up to grid_slices, are what a wave needs for the addresses of its first loads: the module
  // is compiled so that they are in scalar registers when the wave starts, where the others, and the grid's sizes,
  // are fetched from memory, a trip of its own that the first loads must not wait for.  Hence grid_slices, which
  // says what gridDim.y would, k_len = K / (grid_slices * WK), the values of K that a wave walks (a division less on
  // the way to the first load), and no use of gridDim.  The later arguments are not taken from the parameters, which
  // the compiler fetches at the kernel's entry (into scalar registers that it then wants for something else, so
  // that it waits for them after all), but read from the argument segment by fetch_late_args() below, behind the
  // first loads.)
  size_t plane = 0;
  RopeArgs ra;
  FuseArgs fa;
  auto fetch_late_args = [&]() {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const __attribute__((address_space(4))) char* seg_bytes;
    typedef const __attribute__((address_space(4))) SkinnyLateArgs* seg_late;
    const seg_late seg = (seg_late)((seg_bytes)__builtin_amdgcn_kernarg_segment_ptr() + kSkinnyLateArgsOffset);
    plane = seg->plane;
    ra.positions = seg->ra.positions, ra.cos_t = seg->ra.cos_t, ra.sin_t = seg->ra.sin_t;
    ra.kcache = seg->ra.kcache, ra.vcache = seg->ra.vcache, ra.slot_mapping = seg->ra.slot_mapping;
    ra.page_size = seg->ra.page_size, ra.nh = seg->ra.nh, ra.nkv = seg->ra.nkv, ra.hd = seg->ra.hd;
    fa.ss_in = seg->fa.ss_in, fa.parts_in = seg->fa.parts_in, fa.eps_in = seg->fa.eps_in;
    fa.inv_width_in = seg->fa.inv_width_in, fa.resid = seg->fa.resid, fa.gamma = seg->fa.gamma;
    fa.gamma_is_bf16 = seg->fa.gamma_is_bf16, fa.u_out = seg->fa.u_out, fa.ss_out = seg->fa.ss_out;
#else
    plane = plane_arg, ra = ra_arg, fa = fa_arg;
#endif
  };
  (void)plane_arg, (void)ra_arg, (void)fa_arg;
  // loads of U steps of K are issued together before their MFMAs, so that a wave keeps U * (RT + MT) 16-byte
  // loads per lane in flight: the product is bound by memory latency and bandwidth, not by arithmetic
  // (eight waves of many tiles have 256 registers each: one step)
  constexpr int U = UO ? UO : (RT + MT <= 2) ? 4 : (RT + MT > 5 && WK > 4) ? 1 : 2;     // (batch_depth() says the same)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wn = wave % WN, wk = wave / WN;
  const int r16 = lane & 15, kg = lane >> 4;
  static_assert(!HALF || (RT == 1 && MT == 1 && !SWIGLU && !ROPE), "half tiles: one tile, residual epilogue");
  static_assert(!PACK || HALF, "packed activations go with half tiles");
  static_assert(!TILED || (WN == 1 && (!HALF || TILED == 1)),
                "the tiled layout: K split over a workgroup's waves");
  const int n_base = (blockIdx.x * WN + wn) * (HALF ? 8 : RT * 16);
  constexpr int KSTEP = HALF ? 64 : 32;               // values of K that a wave's step covers
  const int k_slices = grid_slices * WK;
  const int k_begin = (blockIdx.y * WK + wk) * k_len;

  // row pointers; rows past the end are clamped to the last valid row and never stored
  const uint16_t* wp[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    int n = n_base + r * 16 + (HALF ? (r16 & 7) : r16);
    if (n > N - 1) n = N - 1;
    wp[r] = w + (size_t)n * ldw + k_begin + kg * 8 + ((HALF && r16 >= 8) ? 32 : 0);
  }
  const uint16_t* ap[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    int row = m * 16 + (PACK ? (r16 & 7) : r16);
    if (row > M - 1) row = M - 1;
    ap[m] = a + (size_t)row * lda + k_begin + kg * 8 + ((PACK && r16 >= 8) ? 32 : 0);
  }

  // the tiled layout: this lane's piece of the wave's first tile, and the elements between two batches
  // (TILED is the number of tiles of a wave that the layout was made for: it divides RT, and a wave of more tiles
  // reads those of RT / TILED neighbouring groups of the layout)
  constexpr int LRT = TILED ? TILED : 1;
  static_assert(RT % LRT == 0, "a wave covers whole groups of the layout");
  // (with K split over the grid too, every slice of K counts as a wave of the layout: k_slices of them a group)
  const uint16_t* const wt =
      w + ((size_t)(blockIdx.x * (RT / LRT) * k_slices + blockIdx.y * WK + wk) * U * LRT) * 512 + lane * 8;
  const size_t wt_batch = (size_t)(N / (HALF ? 8 : 16 * RT)) * k_slices * U * RT * 512;   // (groups of the layout)
  const size_t wt_group = (size_t)k_slices * U * LRT * 512;      // between the layout's groups that a wave covers

  f32x4 acc[RT][MT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x4 acc_hi = f32x4{0.f, 0.f, 0.f, 0.f};           // HALF: the sums over the second 32 values of every step

  // what the fused norm needs from memory is asked for first, so that it has arrived when the sums are done
  // The shares of the rows' sums of squares are added by all waves of the workgroup, up to sixteen per lane and row,
  // and meet in LDS (behind the barrier that the K-split needs anyway).  They are asked for after the first loads
  // of the weight (below) and added after the last MFMA, so that nothing waits for them.
  __shared__ float ss_red[WN * WK][16];
  // (fa lives in the later arguments: nothing may ask for it before the first loads of the weight are on their way)
  auto is_scaled = [&]() { return MT == 1 && fa.ss_in != nullptr; };
  constexpr int SS_STRIDE = 4 * WN * WK;
  float ss_v[16];
  auto load_shares = [&]() {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int p = wave * 4 + kg + j * SS_STRIDE;
      ss_v[j] = (is_scaled() && p < fa.parts_in) ? fa.ss_in[p * 16 + r16] : 0.f;
    }
  };
  f32x4 res_in[RT];
  auto load_resid = [&]() {
    if (MT == 1 && fa.resid != nullptr && wk == 0) {
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        const int n0 = n_base + r * 16 + kg * 4;
        res_in[r] = (r16 < M && n0 + 3 < N && (!HALF || kg < 2))
                        ? *reinterpret_cast<const f32x4*>(fa.resid + (size_t)r16 * N + n0)
                        : f32x4{0.f, 0.f, 0.f, 0.f};
      }
    }
  };

  // two buffers of U steps each: while the MFMAs of one run, the loads of the other are in flight
  bf16x8 wf[2][U][RT], af[2][U][MT], af_hi[2][U];
  auto load = [&](int buf, int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        if constexpr (TILED)
          wf[buf][u][r] = *reinterpret_cast<const bf16x8*>(wt + (size_t)(k0 / (KSTEP * U)) * wt_batch +
                                                           (r / LRT) * wt_group + (u * LRT + r % LRT) * 512);
        else
          wf[buf][u][r] = *reinterpret_cast<const bf16x8*>(wp[r] + k0 + u * KSTEP);
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) af[buf][u][m] = *reinterpret_cast<const bf16x8*>(ap[m] + k0 + u * KSTEP);
      if constexpr (HALF && !PACK) af_hi[buf][u] = *reinterpret_cast<const bf16x8*>(ap[0] + k0 + u * KSTEP + 32);
    }
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[r][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[buf][u][r], af[buf][u][m], acc[r][m], 0, 0, 0);
      if constexpr (HALF && !PACK)
        acc_hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[buf][u][0], af_hi[buf][u], acc_hi, 0, 0, 0);
    }
  };
  constexpr int STEP = KSTEP * U;
  const int n_batches = k_len / STEP;
  int k = 0;
  if (n_batches > 0) {
    load(0, 0);
    __builtin_amdgcn_sched_barrier(0);      // (what follows needs the later arguments: behind the first loads)
    fetch_late_args();
    load_resid();
    if constexpr (MT == 1) load_shares();
    int b = 0;
    for (; b + 2 <= n_batches; b += 2) {
      load(1, (b + 1) * STEP);
      multiply(0);
      if (b + 2 < n_batches) load(0, (b + 2) * STEP);
      multiply(1);
    }
    if (b < n_batches) multiply(0);
    k = n_batches * STEP;
  }
  if (n_batches <= 0) {
    fetch_late_args();
    load_resid();
  }
  for (; k < k_len; k += KSTEP) {
    bf16x8 wt[RT], at[MT];
#pragma unroll
    for (int r = 0; r < RT; ++r) wt[r] = *reinterpret_cast<const bf16x8*>(wp[r] + k);
#pragma unroll
    for (int m = 0; m < MT; ++m) at[m] = *reinterpret_cast<const bf16x8*>(ap[m] + k);
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[r][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wt[r], at[m], acc[r][m], 0, 0, 0);
    if constexpr (HALF && !PACK) {
      const bf16x8 at_hi = *reinterpret_cast<const bf16x8*>(ap[0] + k + 32);
      acc_hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wt[0], at_hi, acc_hi, 0, 0, 0);
    }
  }
  if constexpr (PACK) {
    // (row n of W, row r of A), n and r below 8: the lane of (n + 8, r + 8), 32 + 8 lanes further, has the other half
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[0][0][i] += __shfl(acc[0][0][i], (lane + 40) & 63, 64);
  } else if constexpr (HALF) {
    // rows 0..7 of the tile (lanes kg < 2) take the sums of the second halves from rows 8..15 (the lane 32 further)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc_hi[i]), __float_as_uint(acc_hi[i]), false,
                                                       false);
      acc[0][0][i] += __uint_as_float(sw[1]);
    }
  }

  if (is_scaled()) {
    if (n_batches <= 0) load_shares();
    float ss_mine = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) ss_mine += ss_v[j];
    for (int p = wave * 4 + kg + 16 * SS_STRIDE; p < fa.parts_in; p += SS_STRIDE) ss_mine += fa.ss_in[p * 16 + r16];
    ss_mine += __shfl_xor(ss_mine, 16, 64);
    ss_mine += __shfl_xor(ss_mine, 32, 64);
    if (kg == 0) ss_red[wave][r16] = ss_mine;
    if constexpr (WK == 1) __syncthreads();
  }

  if constexpr (WK > 1) {
    // add the WK partial accumulators of the same rows: waves wk > 0 write, wave wk == 0 sums in fixed order
    __shared__ float red[(WK - 1) * WN * RT * MT * 4 * 64];
    constexpr int per_wave = RT * MT * 4 * 64;
    if (wk > 0) {
      float* dst = red + ((wk - 1) * WN + wn) * per_wave;
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[((r * MT + m) * 4 + i) * 64 + lane] = acc[r][m][i];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int s = 0; s < WK - 1; ++s) {
      const float* src = red + (s * WN + wn) * per_wave;
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[r][m][i] += src[((r * MT + m) * 4 + i) * 64 + lane];
    }
  }

  if constexpr (MT == 1) {
    if (is_scaled()) {
      float t = 0.f;
#pragma unroll
      for (int i = 0; i < WN * WK; ++i) t += ss_red[i][r16];
      const float row_scale = 1.0f / sqrtf(t * fa.inv_width_in + fa.eps_in);
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[r][0][i] *= row_scale;
    }
    if constexpr (!SWIGLU && !ROPE) {
      if (fa.resid != nullptr) {
        // lane (row r16, columns n0 .. n0 + 3 of each of its RT tiles): residual, next activations, squares
        float ssq = 0.f;
#pragma unroll
        for (int r = 0; r < RT; ++r) {
          const int n0 = n_base + r * 16 + kg * 4;
          if (r16 >= M || n0 + 3 >= N || (HALF && kg >= 2)) continue;
          float g[4];
          if (fa.gamma_is_bf16) {
            const uint2 t = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(fa.gamma) + n0);
            g[0] = bf16_bits_to_f32((uint16_t)(t.x & 0xffff)), g[1] = bf16_bits_to_f32((uint16_t)(t.x >> 16));
            g[2] = bf16_bits_to_f32((uint16_t)(t.y & 0xffff)), g[3] = bf16_bits_to_f32((uint16_t)(t.y >> 16));
          } else {
            const f32x4 t = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(fa.gamma) + n0);
            g[0] = t[0], g[1] = t[1], g[2] = t[2], g[3] = t[3];
          }
          f32x4 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            v[i] = res_in[r][i] + acc[r][0][i];
            ssq += v[i] * v[i];
          }
          *reinterpret_cast<f32x4*>(fa.resid + (size_t)r16 * N + n0) = v;
          uint2 o;
          o.x = (uint32_t)f32_to_bf16_bits(v[0] * g[0]) | ((uint32_t)f32_to_bf16_bits(v[1] * g[1]) << 16);
          o.y = (uint32_t)f32_to_bf16_bits(v[2] * g[2]) | ((uint32_t)f32_to_bf16_bits(v[3] * g[3]) << 16);
          *reinterpret_cast<uint2*>(fa.u_out + (size_t)r16 * N + n0) = o;
        }
        ssq += __shfl_xor(ssq, 16, 64);
        ssq += __shfl_xor(ssq, 32, 64);
        if (kg == 0) fa.ss_out[(size_t)(blockIdx.x * WN + wn) * 16 + r16] = ssq;
        return;
      }
    }
  }

  if constexpr (SWIGLU) {
    // W holds, for every 16 outputs, 16 gate rows followed by 16 up rows: row tile r is a gate tile, r + 1 its
    // up tile, and the lane that holds gate value (n, row) holds up value (n, row) too.
    // C[row][n] = silu(gate) * up, with N / 2 columns (the reference: models/src/llama.rs:364).
    static_assert(!SWIGLU || (RT % 2 == 0 && sizeof(TC) == 2), "swiglu epilogue needs pairs of tiles, bf16 out");
#pragma unroll
    for (int r = 0; r < RT; r += 2) {
      const int n0 = (n_base + r * 16) / 2 + kg * 4;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int row = m * 16 + r16;
        if (row >= M || n0 + 3 >= N / 2) continue;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float g = acc[r][m][i];
          v[i] = g / (1.0f + expf(-g)) * acc[r + 1][m][i];
        }
        uint2 o;
        o.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
        o.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(c) + (size_t)row * ldc + n0) = o;
      }
    }
    return;
  }

  if constexpr (ROPE) {
    // the fused q, k, v projection: rotate q and k, store k and v in the cache (rope_store4)
    static_assert(!ROPE || sizeof(TC) == 2, "the rotary epilogue writes bfloat16");
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      const int n0 = n_base + r * 16 + kg * 4;
      if (n0 + 3 >= N) continue;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int row = m * 16 + r16;
        if (row >= M) continue;
        rope_store4(acc[r][m][0], acc[r][m][1], acc[r][m][2], acc[r][m][3], row, n0, ra,
                    reinterpret_cast<uint16_t*>(c), ldc);
      }
    }
    return;
  }

  // D[n = kg*4 + i][row of A = r16]: four consecutive columns of C per lane
  TC* cp = c + (size_t)blockIdx.y * plane;
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int n0 = n_base + r * 16 + kg * 4;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const int row = m * 16 + r16;
      if (row >= M) continue;
      TC* dst = cp + (size_t)row * ldc + n0;
      if (n0 + 3 < N && (ldc & 3) == 0) {
        if (sizeof(TC) == 4) {
          *reinterpret_cast<f32x4*>(dst) = acc[r][m];
        } else {
          uint2 v;
          v.x = (uint32_t)f32_to_bf16_bits(acc[r][m][0]) | ((uint32_t)f32_to_bf16_bits(acc[r][m][1]) << 16);
          v.y = (uint32_t)f32_to_bf16_bits(acc[r][m][2]) | ((uint32_t)f32_to_bf16_bits(acc[r][m][3]) << 16);
          *reinterpret_cast<uint2*>(dst) = v;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n0 + i < N) dst[i] = from_f32<TC>(acc[r][m][i]);
      }
    }
  }
}

template <int MT, int RT, int WN, int WK>
static int launch(const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc,
                  int slices, const FuseArgs& fa, hipStream_t stream) {
  dim3 grid((N + WN * RT * 16 - 1) / (WN * RT * 16), slices), block(64 * WN * WK);
  const size_t plane = (size_t)M * ldc;
  if (c_dtype == kF32)
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, float>), grid, block, 0, stream, (const uint16_t*)a,
                       (const uint16_t*)w, (float*)c, M, N, K, lda, ldw, ldc, slices, K / (slices * WK), plane, RopeArgs{}, fa);
  else if (c_dtype == kBF16)
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, bf16_t>), grid, block, 0, stream, (const uint16_t*)a,
                       (const uint16_t*)w, (bf16_t*)c, M, N, K, lda, ldw, ldc, slices, K / (slices * WK), plane, RopeArgs{}, fa);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// The depth of a wave's batches of loads for (tiles of rows, tiles of the weight, waves splitting K), as the kernel
// chooses it; the tiled layout of a weight is made for one such triple.
static constexpr int batch_depth(int mt, int rt, int wk) { return (rt + mt <= 2) ? 4 : (rt + mt > 5 && wk > 4) ? 1 : 2; }

// Where element (row n, column k) of a weight [N, K] lies in the tiled layout made for waves of rt tiles, wk waves a
// workgroup and batches of u steps (see the kernel's TILED): N % (16 rt) == 0 and K % (32 wk u) == 0.
extern "C" long long atoma_gemm_bf16_tiled_offset(long long n, long long k, long long N, long long K, int rt, int wk,
                                                  int u) {
  const long long k_len = K / wk, wg = n / (16 * rt), r = (n / 16) % rt, row = n % 16;
  const long long slice = k / k_len, kk = k % k_len, batch = kk / (32 * u), step = (kk / 32) % u, kg = (kk % 32) / 8;
  const long long groups = N / (16 * rt);
  return ((((batch * groups + wg) * wk + slice) * u + step) * rt + r) * 512 + (kg * 16 + row) * 8 + k % 8;
}

template <int MT>
static int launch_mt(const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, int lda, int ldw,
                     int ldc, int rt, int wk, int slices, const FuseArgs& fa, hipStream_t stream) {
#define ATOMA_CASE(R, WN_, WK_)                                                                                   \
  if (rt == R && wk == WK_)                                                                                       \
  return launch<MT, R, WN_, WK_>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, slices, fa, stream)
  ATOMA_CASE(1, 4, 1);
  ATOMA_CASE(2, 4, 1);
  ATOMA_CASE(4, 4, 1);
  ATOMA_CASE(1, 1, 4);
  ATOMA_CASE(2, 1, 4);
  ATOMA_CASE(1, 1, 8);
  ATOMA_CASE(2, 1, 8);
  ATOMA_CASE(4, 1, 4);
#undef ATOMA_CASE
  return ATOMA_ERR_SHAPE;
}

// a [M <= 64, K] bf16, w [N, K] bf16 -> c [slices][M, N] (bf16 only with slices == 1, or float32).
// rt: tiles of 16 rows of W per wave (1, 2, 4); wk: 1 (four waves on different rows), 4 or 8 (that many waves
// split K for the same rows; four tiles only with 4); slices: K split across the grid.
static bool fuse_in_ok(const float* ss_in, int parts_in, float eps_in, int width_in, int M) {
  return ss_in == nullptr || (M <= 16 && parts_in > 0 && width_in > 0 && eps_in >= 0.f);
}

static FuseArgs fuse_in(const float* ss_in, int parts_in, float eps_in, int width_in) {
  FuseArgs fa{};
  fa.ss_in = ss_in;
  fa.parts_in = parts_in;
  fa.eps_in = eps_in;
  fa.inv_width_in = width_in > 0 ? 1.0f / (float)width_in : 0.f;
  return fa;
}

static int skinny_dispatch(const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, int lda, int ldw,
                           int ldc, int rt, int wk, int slices, const FuseArgs& fa, hipStream_t stream) {
  const int mt = (M + 15) / 16;
  switch (mt) {
    case 1: return launch_mt<1>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, fa, stream);
    case 2: return launch_mt<2>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, fa, stream);
    case 3: return launch_mt<3>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, fa, stream);
    default: return launch_mt<4>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, fa, stream);
  }
}

extern "C" int atoma_gemm_bf16_skinny(const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                                      int lda, int ldw, int ldc, int rt, int wk, int slices, const float* ss_in,
                                      int parts_in, float eps_in, int width_in, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || slices <= 0 || K % (32 * wk * slices) || (lda & 7) || (ldw & 7) || lda < K || ldw < K ||
      ldc < N || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || (slices > 1 && c_dtype != kF32) || slices > 65535 ||
      !fuse_in_ok(ss_in, parts_in, eps_in, width_in, M) || (ss_in && slices > 1))
    return ATOMA_ERR_SHAPE;
  return skinny_dispatch(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices,
                         fuse_in(ss_in, parts_in, eps_in, width_in), stream);
}

// The same product over a weight in the tiled layout (at most 16 rows of a; rt tiles a wave, wk waves a workgroup: 2
// and 8, or 4 and 4; N % (16 rt) == 0, K % (32 wk u) == 0 with u the kernel's batch depth): float32 or bfloat16 out.
extern "C" int atoma_gemm_bf16_skinny_tiled(const void* a, const void* w_tiled, void* c, int c_dtype, int M, int N, int K,
                                            int lda, int ldc, int rt, int wk, const float* ss_in, int parts_in,
                                            float eps_in, int width_in, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K <= 0 || wk <= 0 || rt <= 0 || N % (16 * rt) || K % (32 * wk * batch_depth(1, rt, wk)) || (lda & 7) ||
      lda < K || ldc < N || ((uintptr_t)a & 15) || ((uintptr_t)w_tiled & 15) ||
      !fuse_in_ok(ss_in, parts_in, eps_in, width_in, M))
    return ATOMA_ERR_SHAPE;
  const FuseArgs fa = fuse_in(ss_in, parts_in, eps_in, width_in);
  dim3 grid(N / (16 * rt), 1);
#define ATOMA_TILED(R, WK_, TC_)                                                                                      \
  do {                                                                                                               \
    hipLaunchKernelGGL((gemm_skinny_kernel<1, R, 1, WK_, TC_, false, false, 0, false, false, R>), grid,              \
                       dim3(64 * WK_), 0, stream, (const uint16_t*)a, (const uint16_t*)w_tiled, (TC_*)c, M, N, K,    \
                       lda, K, ldc, 1, K / WK_, (size_t)0, RopeArgs{}, fa);                                             \
    ATOMA_LAUNCH_CHECK();                                                                                            \
    return 0;                                                                                                        \
  } while (0)
  if (rt == 2 && wk == 8 && c_dtype == kF32) ATOMA_TILED(2, 8, float);
  if (rt == 2 && wk == 8 && c_dtype == kBF16) ATOMA_TILED(2, 8, bf16_t);
  if (rt == 4 && wk == 4 && c_dtype == kF32) ATOMA_TILED(4, 4, float);
  if (rt == 2 && wk == 4 && c_dtype == kF32) ATOMA_TILED(2, 4, float);
  if (rt == 2 && wk == 4 && c_dtype == kBF16) ATOMA_TILED(2, 4, bf16_t);
#undef ATOMA_TILED
  return ATOMA_ERR_SHAPE;
}

template <int MT>
static int launch_swiglu_tiled(const void* a, const void* w_tiled, void* c, int M, int N, int K, int lda, int ldc, int rt,
                               int layout_rt, const FuseArgs& fa, hipStream_t stream) {
  dim3 grid(N / (16 * rt), 1);
#define ATOMA_SWIGLU_TILED(R, L)                                                                                      \
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, R, 1, 4, bf16_t, true, false, 0, false, false, L>), grid, dim3(256), 0,  \
                     stream, (const uint16_t*)a, (const uint16_t*)w_tiled, (bf16_t*)c, M, N, K, lda, K, ldc,         \
                     1, K / 4, (size_t)0, RopeArgs{}, fa)
  if (rt == 2 && layout_rt == 2) ATOMA_SWIGLU_TILED(2, 2);
  else if (rt == 4 && layout_rt == 2) ATOMA_SWIGLU_TILED(4, 2);
  else if (rt == 4 && layout_rt == 4) ATOMA_SWIGLU_TILED(4, 4);
  else return ATOMA_ERR_SHAPE;
#undef ATOMA_SWIGLU_TILED
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <int MT, int RT>
static int launch_tiled_planes(const void* a, const void* w_tiled, float* c, int M, int N, int K, int lda, int ldc,
                               int slices, hipStream_t stream) {
  dim3 grid(N / (16 * RT), slices);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, 1, 4, float, false, false, 0, false, false, RT>), grid, dim3(256), 0,
                     stream, (const uint16_t*)a, (const uint16_t*)w_tiled, c, M, N, K, lda, K, ldc, slices, K / (slices * 4), (size_t)M * ldc,
                     RopeArgs{}, FuseArgs{});
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// Float32 planes c [slices][M, N] of a product of 17 to 64 rows, K split over four waves a workgroup and ``slices``
// ways over the grid, over a weight in the tiled layout made for waves of rt tiles (2 or 4) and 4 * slices slices of K.
extern "C" int atoma_gemm_bf16_skinny_tiled_planes(const void* a, const void* w_tiled, float* c, int M, int N, int K,
                                                   int lda, int ldc, int rt, int slices, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  static_assert(batch_depth(2, 2, 4) == 2 && batch_depth(4, 4, 4) == 2 && batch_depth(2, 4, 4) == 2 &&
                batch_depth(4, 2, 4) == 2, "one layout for 17 to 64 rows");
  if (M <= 16 || M > 64 || K <= 0 || (rt != 2 && rt != 4) || slices <= 0 || slices > 65535 || N % (16 * rt) ||
      K % (32 * 4 * slices * 2) || (lda & 7) || lda < K || ldc < N || ((uintptr_t)a & 15) || ((uintptr_t)w_tiled & 15))
    return ATOMA_ERR_SHAPE;
  const int mt = (M + 15) / 16;
#define ATOMA_PLANES(MT_)                                                                                             \
  return rt == 2 ? launch_tiled_planes<MT_, 2>(a, w_tiled, c, M, N, K, lda, ldc, slices, stream)                     \
                 : launch_tiled_planes<MT_, 4>(a, w_tiled, c, M, N, K, lda, ldc, slices, stream)
  if (mt == 2) ATOMA_PLANES(2);
  if (mt == 3) ATOMA_PLANES(3);
  ATOMA_PLANES(4);
#undef ATOMA_PLANES
}

// The gate-up product with SiLU(gate) * up in its epilogue over a weight in the tiled layout (gate and up rows
// interleaved in blocks of 16 before the tiling): at most 64 rows of a; waves of rt tiles (2 or 4) read a layout made
// for waves of layout_rt tiles (rt or, with rt 4, also 2), wk 4.  The depth of the batches of loads, and with it the
// layout, is the same for every number of rows.
extern "C" int atoma_gemm_bf16_skinny_swiglu_tiled(const void* a, const void* w_tiled, void* c, int M, int N, int K,
                                                   int lda, int ldc, int rt, int layout_rt, int wk, const float* ss_in,
                                                   int parts_in, float eps_in, int width_in, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  static_assert(batch_depth(1, 2, 4) == batch_depth(4, 2, 4) && batch_depth(1, 4, 4) == batch_depth(4, 4, 4) &&
                batch_depth(2, 2, 4) == batch_depth(3, 4, 4), "one layout for every number of rows");
  if (M > 64 || K <= 0 || wk != 4 || (rt != 2 && rt != 4) || N % (16 * rt) || K % (32 * wk * batch_depth(1, rt, wk)) ||
      (lda & 7) || lda < K || ldc < N / 2 || (ldc & 3) || ((uintptr_t)a & 15) || ((uintptr_t)w_tiled & 15) ||
      ((uintptr_t)c & 7) || !fuse_in_ok(ss_in, parts_in, eps_in, width_in, M))
    return ATOMA_ERR_SHAPE;
  const FuseArgs fa = fuse_in(ss_in, parts_in, eps_in, width_in);
  switch ((M + 15) / 16) {
    case 1: return launch_swiglu_tiled<1>(a, w_tiled, c, M, N, K, lda, ldc, rt, layout_rt, fa, stream);
    case 2: return launch_swiglu_tiled<2>(a, w_tiled, c, M, N, K, lda, ldc, rt, layout_rt, fa, stream);
    case 3: return launch_swiglu_tiled<3>(a, w_tiled, c, M, N, K, lda, ldc, rt, layout_rt, fa, stream);
    default: return launch_swiglu_tiled<4>(a, w_tiled, c, M, N, K, lda, ldc, rt, layout_rt, fa, stream);
  }
}

extern "C" int atoma_gemm_bf16_batch_depth(int mt, int rt, int wk) { return batch_depth(mt, rt, wk); }

// The product of at most 16 rows added to the residual stream, with the following norm begun (see FuseArgs):
// resid [M][N] float32 += a w^T in place, u_out [M][N] bfloat16 = resid * gamma, ss_out [parts][16] the shares of
// the rows' sums of squares, parts = atoma_gemm_bf16_resid_parts(N, rt, wk, half).  half: 8 rows of W a wave (see the kernel).  depth: steps of K whose loads a wave
// issues together (two such batches are in flight).  The rows of a may themselves be an
// unfinished norm (ss_in).  K is split over the waves of a workgroup only, so every sum has one owner.
extern "C" int atoma_gemm_bf16_resid_parts(int N, int rt, int wk, int half) {
  const int wn = wk == 1 ? 4 : 1;
  const int cols = half ? wn * 8 : wn * rt * 16;
  return ((N + cols - 1) / cols) * wn;
}

template <int R, int WN, int WK, int U, bool H>
static void resid_kernels(bool tiled, const void* a, const void* w, int M, int N, int K, int lda, int ldw, float* resid,
                          const FuseArgs& fa, hipStream_t stream) {
  const int cols = H ? WN * 8 : WN * R * 16;
  dim3 grid((N + cols - 1) / cols, 1), block(64 * WN * WK);
#define ATOMA_RESID_KERNEL(PACK_, TILED_)                                                                             \
  hipLaunchKernelGGL((gemm_skinny_kernel<1, R, WN, WK, float, false, false, U, H, PACK_, TILED_>), grid, block, 0,    \
                     stream, (const uint16_t*)a, (const uint16_t*)w, resid, M, N, K, lda, ldw, N, 1, K / WK,          \
                     (size_t)0, RopeArgs{}, fa)
  if constexpr (WN == 1 && WK == 8 && (U == 4 || U == 8)) {
    if (tiled) {
      if (H && M <= 8) ATOMA_RESID_KERNEL(H, 1);
      else ATOMA_RESID_KERNEL(false, 1);
      return;
    }
  }
  if (H && M <= 8) ATOMA_RESID_KERNEL(H, 0);        // (activations packed as the half tiles are)
  else ATOMA_RESID_KERNEL(false, 0);
#undef ATOMA_RESID_KERNEL
}

static int launch_resid(const void* a, const void* w, bool tiled, int M, int N, int K, int lda, int ldw, int rt, int wk,
                        int depth, int half, const float* ss_in, int parts_in, float eps_in, int width_in, float* resid,
                        const void* gamma, int gamma_dtype, void* u_out, float* ss_out, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  // the tiled layout: eight waves a workgroup, batches of 4 or 8 steps; whole tiles (atoma_gemm_bf16_tiled_offset with
  // one tile a wave) or half tiles (8 rows x 64 values of K in the lanes' order, atoma_gemm_bf16_tiled_offset_half)
  if (tiled && (wk != 8 || (depth != 4 && depth != 8) || rt != 1 || N % (half ? 8 : 16) ||
                K % ((half ? 64 : 32) * wk * depth)))
    return ATOMA_ERR_SHAPE;
  if (M > 16 || K <= 0 || K % ((half ? 64 : 32) * wk) || (lda & 7) || (ldw & 7) || lda < K || ldw < K || (N & 3) ||
      ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || !resid || !gamma || !u_out || !ss_out ||
      ((uintptr_t)resid & 15) || ((uintptr_t)gamma & 15) || ((uintptr_t)u_out & 7) ||
      (gamma_dtype != kF32 && gamma_dtype != kBF16) || !fuse_in_ok(ss_in, parts_in, eps_in, width_in, M))
    return ATOMA_ERR_SHAPE;
  FuseArgs fa = fuse_in(ss_in, parts_in, eps_in, width_in);
  fa.resid = resid;
  fa.gamma = gamma;
  fa.gamma_is_bf16 = gamma_dtype == kBF16;
  fa.u_out = (uint16_t*)u_out;
  fa.ss_out = ss_out;
  // (the float32 instance; nothing is stored through c)
#define ATOMA_RESID(R, WN_, WK_, U_, H_)                                                                           \
  if (rt == R && wk == WK_ && depth == U_ && (half != 0) == H_) {                                                  \
    resid_kernels<R, WN_, WK_, U_, H_>(tiled, a, w, M, N, K, lda, ldw, resid, fa, stream);                         \
    ATOMA_LAUNCH_CHECK();                                                                                          \
    return 0;                                                                                                      \
  }
  ATOMA_RESID(1, 1, 4, 4, false)
  ATOMA_RESID(1, 1, 8, 4, false)
  ATOMA_RESID(1, 1, 8, 2, false)
  ATOMA_RESID(1, 1, 8, 8, false)
  ATOMA_RESID(1, 4, 1, 4, false)
  ATOMA_RESID(1, 1, 4, 4, true)
  ATOMA_RESID(1, 1, 4, 8, true)
  ATOMA_RESID(1, 1, 8, 4, true)
  ATOMA_RESID(1, 1, 8, 8, true)
  ATOMA_RESID(1, 1, 8, 2, true)
  ATOMA_RESID(1, 4, 1, 4, true)
#undef ATOMA_RESID
  return ATOMA_ERR_SHAPE;
}

extern "C" int atoma_gemm_bf16_skinny_resid(const void* a, const void* w, int M, int N, int K, int lda, int ldw,
                                            int rt, int wk, int depth, int half, const float* ss_in, int parts_in, float eps_in,
                                            int width_in, float* resid, const void* gamma, int gamma_dtype,
                                            void* u_out, float* ss_out, hipStream_t stream) {
  return launch_resid(a, w, false, M, N, K, lda, ldw, rt, wk, depth, half, ss_in, parts_in, eps_in, width_in, resid,
                      gamma, gamma_dtype, u_out, ss_out, stream);
}

// The same over a weight in the tiled layout: eight waves a workgroup, one tile or half tile a wave, batches of
// ``depth`` steps (4 or 8).
extern "C" int atoma_gemm_bf16_skinny_resid_tiled(const void* a, const void* w_tiled, int M, int N, int K, int lda,
                                                  int depth, int half, const float* ss_in, int parts_in, float eps_in,
                                                  int width_in, float* resid, const void* gamma, int gamma_dtype,
                                                  void* u_out, float* ss_out, hipStream_t stream) {
  return launch_resid(a, w_tiled, true, M, N, K, lda, K, 1, 8, depth, half, ss_in, parts_in, eps_in, width_in, resid,
                      gamma, gamma_dtype, u_out, ss_out, stream);
}

// Where element (row n, column k) of a weight [N, K] lies in the tiled layout of half tiles: tiles of 8 rows x 64
// values of K (lane l holds row l % 8 and the 8 values from 8 (l / 16) + 32 (l / 8 % 2) on), ordered by batch of u
// steps, workgroup (8 rows), wave (K / wk values each), step.  N % 8 == 0 and K % (64 wk u) == 0.
extern "C" long long atoma_gemm_bf16_tiled_offset_half(long long n, long long k, long long N, long long K, int wk,
                                                       int u) {
  const long long k_len = K / wk, wg = n / 8, row = n % 8;
  const long long slice = k / k_len, kk = k % k_len, batch = kk / (64 * u), step = (kk / 64) % u, p = kk % 64;
  const long long lane = ((p % 32) / 8) * 16 + (p / 32) * 8 + row;
  return (((batch * (N / 8) + wg) * wk + slice) * u + step) * 512 + lane * 8 + k % 8;
}

template <int MT, int RT, int WN, int WK>
static int launch_swiglu(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                         const FuseArgs& fa, hipStream_t stream) {
  dim3 grid((N + WN * RT * 16 - 1) / (WN * RT * 16), 1), block(64 * WN * WK);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, bf16_t, true>), grid, block, 0, stream, (const uint16_t*)a,
                     (const uint16_t*)w, (bf16_t*)c, M, N, K, lda, ldw, ldc, 1, K / WK, (size_t)0, RopeArgs{}, fa);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <int MT>
static int launch_swiglu_mt(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                            int rt, int wk, const FuseArgs& fa, hipStream_t stream) {
  if (rt == 2 && wk == 1) return launch_swiglu<MT, 2, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, fa, stream);
  if (rt == 4 && wk == 1) return launch_swiglu<MT, 4, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, fa, stream);
  if (rt == 2 && wk == 4) return launch_swiglu<MT, 2, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, fa, stream);
  if constexpr (MT < 4) {   // with four tiles of rows the epilogue does not fit the registers of eight waves
    if (rt == 2 && wk == 8) return launch_swiglu<MT, 2, 1, 8>(a, w, c, M, N, K, lda, ldw, ldc, fa, stream);
  }
  if (rt == 4 && wk == 4) return launch_swiglu<MT, 4, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, fa, stream);
  return ATOMA_ERR_SHAPE;
}

// The gate-up product with SiLU(gate) * up in its epilogue.  w [N, K] holds gate and up rows interleaved in blocks
// of 16 (16 gate rows, then the 16 up rows of the same outputs); c is [M, N / 2] bfloat16.  N % 32 == 0.
extern "C" int atoma_gemm_bf16_skinny_swiglu(const void* a, const void* w, void* c, int M, int N, int K, int lda,
                                             int ldw, int ldc, int rt, int wk, const float* ss_in, int parts_in,
                                             float eps_in, int width_in, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % (32 * wk) || (N & 31) || (lda & 7) || (ldw & 7) || lda < K || ldw < K || ldc < N / 2 ||
      (ldc & 3) || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || ((uintptr_t)c & 7) ||
      !fuse_in_ok(ss_in, parts_in, eps_in, width_in, M))
    return ATOMA_ERR_SHAPE;
  const FuseArgs fa = fuse_in(ss_in, parts_in, eps_in, width_in);
  switch ((M + 15) / 16) {
    case 1: return launch_swiglu_mt<1>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, fa, stream);
    case 2: return launch_swiglu_mt<2>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, fa, stream);
    case 3: return launch_swiglu_mt<3>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, fa, stream);
    default: return launch_swiglu_mt<4>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, fa, stream);
  }
}

template <int MT, int RT, int WN, int WK, int TILED = 0>
static int launch_rope(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                       const RopeArgs& ra, const FuseArgs& fa, hipStream_t stream) {
  dim3 grid((N + WN * RT * 16 - 1) / (WN * RT * 16), 1), block(64 * WN * WK);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, bf16_t, false, true, 0, false, false, TILED>), grid, block, 0, stream,
                     (const uint16_t*)a, (const uint16_t*)w, (bf16_t*)c, M, N, K, lda, ldw, ldc, 1, K / WK, (size_t)0, ra, fa);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <int MT>
static int launch_rope_mt(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                          int rt, int wk, const RopeArgs& ra, const FuseArgs& fa, hipStream_t stream) {
  if (rt == 1 && wk == 4) return launch_rope<MT, 1, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, ra, fa, stream);
  if (rt == 2 && wk == 4) return launch_rope<MT, 2, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, ra, fa, stream);
  if (rt == 1 && wk == 8) return launch_rope<MT, 1, 1, 8>(a, w, c, M, N, K, lda, ldw, ldc, ra, fa, stream);
  if constexpr (MT < 4) {   // with four tiles of rows the epilogue does not fit the registers of eight waves
    if (rt == 2 && wk == 8) return launch_rope<MT, 2, 1, 8>(a, w, c, M, N, K, lda, ldw, ldc, ra, fa, stream);
  }
  if (rt == 1 && wk == 1) return launch_rope<MT, 1, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, ra, fa, stream);
  if (rt == 2 && wk == 1) return launch_rope<MT, 2, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, ra, fa, stream);
  return ATOMA_ERR_SHAPE;
}

// The fused q, k, v projection of at most 64 rows with rotary encoding and the cache write in its epilogue.
// w [(nh + 2 nkv) hd, K] with the rows of q and k heads in pair order (pair i: rows 2i, 2i + 1 of the head);
// c [M, ldc >= nh hd] receives the rotated q in its own column order; rotated k and v go to the rows' slots of
// the caches ([pages, nkv, page_size * hd] bfloat16 tiles).  hd % 4 == 0 (then hd / 2 is even and 4-byte stores
// are aligned).
extern "C" int atoma_gemm_bf16_skinny_rope(const void* a, const void* w, void* c, int M, int K, int lda, int ldw,
                                           int ldc, int rt, int wk, const int32_t* positions, const float* cos_t,
                                           const float* sin_t, void* kcache, void* vcache,
                                           const int32_t* slot_mapping, int page_size, int nh, int nkv, int hd,
                                           const float* ss_in, int parts_in, float eps_in, int width_in,
                                           hipStream_t stream) {
  if (M <= 0) return 0;
  const int N = (nh + 2 * nkv) * hd;
  if (!fuse_in_ok(ss_in, parts_in, eps_in, width_in, M)) return ATOMA_ERR_SHAPE;
  const FuseArgs fa = fuse_in(ss_in, parts_in, eps_in, width_in);
  if (M > 64 || K <= 0 || wk <= 0 || K % (32 * wk) || (lda & 7) || (ldw & 7) || lda < K || ldw < K ||
      ldc < nh * hd || (ldc & 1) || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || ((uintptr_t)c & 3) || (hd & 3) ||
      nh <= 0 || nkv <= 0 || page_size <= 0 || !positions || !cos_t || !sin_t || !kcache || !vcache ||
      !slot_mapping || ((uintptr_t)kcache & 3))
    return ATOMA_ERR_SHAPE;
  const RopeArgs ra{positions, cos_t, sin_t, (uint16_t*)kcache, (uint16_t*)vcache, slot_mapping, page_size, nh, nkv, hd};
  switch ((M + 15) / 16) {
    case 1: return launch_rope_mt<1>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, fa, stream);
    case 2: return launch_rope_mt<2>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, fa, stream);
    case 3: return launch_rope_mt<3>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, fa, stream);
    default: return launch_rope_mt<4>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, fa, stream);
  }
}

// The same for at most 16 rows over a weight in the tiled layout made for waves of rt tiles (1 or 2) and 4 waves a
// workgroup.
extern "C" int atoma_gemm_bf16_skinny_rope_tiled(const void* a, const void* w_tiled, void* c, int M, int K, int lda,
                                                 int ldc, int rt, int wk, const int32_t* positions, const float* cos_t,
                                                 const float* sin_t, void* kcache, void* vcache,
                                                 const int32_t* slot_mapping, int page_size, int nh, int nkv, int hd,
                                                 const float* ss_in, int parts_in, float eps_in, int width_in,
                                                 hipStream_t stream) {
  if (M <= 0) return 0;
  const int N = (nh + 2 * nkv) * hd;
  if (!fuse_in_ok(ss_in, parts_in, eps_in, width_in, M)) return ATOMA_ERR_SHAPE;
  const FuseArgs fa = fuse_in(ss_in, parts_in, eps_in, width_in);
  if (M > 16 || K <= 0 || wk != 4 || (rt != 1 && rt != 2) || N % (16 * rt) || K % (32 * wk * batch_depth(1, rt, wk)) ||
      (lda & 7) || lda < K || ldc < nh * hd || (ldc & 1) || ((uintptr_t)a & 15) || ((uintptr_t)w_tiled & 15) ||
      ((uintptr_t)c & 3) || (hd & 3) || nh <= 0 || nkv <= 0 || page_size <= 0 || !positions || !cos_t || !sin_t ||
      !kcache || !vcache || !slot_mapping || ((uintptr_t)kcache & 3))
    return ATOMA_ERR_SHAPE;
  const RopeArgs ra{positions, cos_t, sin_t, (uint16_t*)kcache, (uint16_t*)vcache, slot_mapping, page_size, nh, nkv, hd};
  if (rt == 1) return launch_rope<1, 1, 1, 4, 1>(a, w_tiled, c, M, N, K, lda, K, ldc, ra, fa, stream);
  return launch_rope<1, 2, 1, 4, 2>(a, w_tiled, c, M, N, K, lda, K, ldc, ra, fa, stream);
}

// The fused q, k, v projection of 17 to 64 rows as float32 planes of a K-split product (which about 256 workgroups
// share, each fetching an eighth of the activations, where the product with the rotary epilogue has 192 that each
// fetch all of them), summed here in the order of the planes, rotated and stored: a thread takes four outputs of a row.
constexpr int kMaxPlanes = 8;
__global__ void __launch_bounds__(256)
rope_from_planes_kernel(const float* __restrict__ planes, int slices, size_t plane, int M, int N, uint16_t* __restrict__ q_out,
                        int ldq, RopeArgs ra) {
  const int row = blockIdx.x;
  const int n0 = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (n0 + 3 >= N) return;
  const float* p = planes + (size_t)row * N + n0;
  // (all planes are asked for at once: each load is a trip to memory)
  f32x4 v[kMaxPlanes];
#pragma unroll
  for (int s = 0; s < kMaxPlanes; ++s) v[s] = *reinterpret_cast<const f32x4*>(p + (size_t)(s < slices ? s : 0) * plane);
  f32x4 sum = v[0];
#pragma unroll
  for (int s = 1; s < kMaxPlanes; ++s)
    if (s < slices) sum[0] += v[s][0], sum[1] += v[s][1], sum[2] += v[s][2], sum[3] += v[s][3];
  rope_store4(sum[0], sum[1], sum[2], sum[3], row, n0, ra, q_out, ldq);
}

// planes [slices][M][N] float32 with N = (nh + 2 nkv) hd, the columns of q and k heads in pair order; q_out
// [M, ldq >= nh hd] bfloat16.  hd % 4 == 0.
extern "C" int atoma_rope_from_planes(const float* planes, int slices, int M, void* q_out, int ldq,
                                      const int32_t* positions, const float* cos_t, const float* sin_t, void* kcache,
                                      void* vcache, const int32_t* slot_mapping, int page_size, int nh, int nkv, int hd,
                                      hipStream_t stream) {
  if (M <= 0) return 0;
  const int N = (nh + 2 * nkv) * hd;
  if (slices <= 0 || slices > kMaxPlanes || M > 65535 || ldq < nh * hd || (ldq & 1) || ((uintptr_t)planes & 15) || ((uintptr_t)q_out & 3) ||
      (hd & 3) || nh <= 0 || nkv <= 0 || page_size <= 0 || !positions || !cos_t || !sin_t || !kcache || !vcache ||
      !slot_mapping || ((uintptr_t)kcache & 3))
    return ATOMA_ERR_SHAPE;
  const RopeArgs ra{positions, cos_t, sin_t, (uint16_t*)kcache, (uint16_t*)vcache, slot_mapping, page_size, nh, nkv, hd};
  dim3 grid(M, (N / 4 + 255) / 256);
  hipLaunchKernelGGL(rope_from_planes_kernel, grid, dim3(256), 0, stream, planes, slices, (size_t)M * N, M, N,
                     (uint16_t*)q_out, ldq, ra);
  ATOMA_LAUNCH_CHECK();
  return 0;
}
