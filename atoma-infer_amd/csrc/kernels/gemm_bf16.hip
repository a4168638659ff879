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

template <int MT, int RT, int WN, int WK, typename TC, bool SWIGLU = false, bool ROPE = false>
__global__ void __launch_bounds__(64 * WN * WK)
gemm_skinny_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, TC* __restrict__ c, int M, int N,
                   int K, int lda, int ldw, int ldc, size_t plane, RopeArgs ra) {
  // loads of U steps of K are issued together before their MFMAs, so that a wave keeps U * (RT + MT) 16-byte
  // loads per lane in flight: the product is bound by memory latency and bandwidth, not by arithmetic
  // (eight waves of many tiles have 256 registers each: one step)
  constexpr int U = (RT + MT <= 2) ? 4 : (RT + MT > 5 && WK > 4) ? 1 : 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wn = wave % WN, wk = wave / WN;
  const int r16 = lane & 15, kg = lane >> 4;
  const int n_base = (blockIdx.x * WN + wn) * (RT * 16);
  const int k_slices = gridDim.y * WK;
  const int k_len = K / k_slices;
  const int k_begin = (blockIdx.y * WK + wk) * k_len;

  // row pointers; rows past the end are clamped to the last valid row and never stored
  const uint16_t* wp[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    int n = n_base + r * 16 + r16;
    if (n > N - 1) n = N - 1;
    wp[r] = w + (size_t)n * ldw + k_begin + kg * 8;
  }
  const uint16_t* ap[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    int row = m * 16 + r16;
    if (row > M - 1) row = M - 1;
    ap[m] = a + (size_t)row * lda + k_begin + kg * 8;
  }

  f32x4 acc[RT][MT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = f32x4{0.f, 0.f, 0.f, 0.f};

  // two buffers of U steps each: while the MFMAs of one run, the loads of the other are in flight
  bf16x8 wf[2][U][RT], af[2][U][MT];
  auto load = [&](int buf, int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int r = 0; r < RT; ++r) wf[buf][u][r] = *reinterpret_cast<const bf16x8*>(wp[r] + k0 + u * 32);
#pragma unroll
      for (int m = 0; m < MT; ++m) af[buf][u][m] = *reinterpret_cast<const bf16x8*>(ap[m] + k0 + u * 32);
    }
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[r][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[buf][u][r], af[buf][u][m], acc[r][m], 0, 0, 0);
  };
  constexpr int STEP = 32 * U;
  const int n_batches = k_len / STEP;
  int k = 0;
  if (n_batches > 0) {
    load(0, 0);
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
  for (; k < k_len; k += 32) {
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
    // W is the fused q, k, v projection with the rows of every q and k head ordered so that the members of
    // rotary pair i = (column i, column i + hd/2) are outputs 2i and 2i + 1 of the head: a lane's four outputs are
    // two whole pairs, i and i + 1.  They are rotated here and go to their own columns: q to C [M, nh * hd], k
    // into the row's slot of the paged cache (the order inside a tile: cache_layout.h); v heads are copied into
    // theirs.  The same arithmetic as the rotary kernel (csrc/kernels/rotary.h:116-131 of the reference), on the
    // float32 sums before they are rounded.
    static_assert(!ROPE || sizeof(TC) == 2, "the rotary epilogue writes bfloat16");
    const int hd = ra.hd, half = hd >> 1;
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      const int n0 = n_base + r * 16 + kg * 4;
      if (n0 + 3 >= N) continue;
      const int head = n0 / hd, d0 = n0 % hd;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int row = m * 16 + r16;
        if (row >= M) continue;
        const float x0 = acc[r][m][0], x1 = acc[r][m][1], x2 = acc[r][m][2], x3 = acc[r][m][3];
        if (head >= ra.nh + ra.nkv) {
          const int slot = ra.slot_mapping[row];
          if (slot < 0) continue;
          const int page = slot / ra.page_size, off = slot % ra.page_size;
          uint16_t* tile = ra.vcache + ((size_t)page * ra.nkv + (head - ra.nh - ra.nkv)) * ra.page_size * hd;
          tile[value_offset(d0, off, hd, ra.page_size)] = f32_to_bf16_bits(x0);
          tile[value_offset(d0 + 1, off, hd, ra.page_size)] = f32_to_bf16_bits(x1);
          tile[value_offset(d0 + 2, off, hd, ra.page_size)] = f32_to_bf16_bits(x2);
          tile[value_offset(d0 + 3, off, hd, ra.page_size)] = f32_to_bf16_bits(x3);
          continue;
        }
        const int i = d0 >> 1;                       // even: columns i, i + 1 and their partners lie together
        const size_t at = (size_t)ra.positions[row] * half + i;
        const float c0 = ra.cos_t[at], s0 = ra.sin_t[at], c1 = ra.cos_t[at + 1], s1 = ra.sin_t[at + 1];
        const uint32_t lo = (uint32_t)f32_to_bf16_bits(x0 * c0 - x1 * s0) |
                            ((uint32_t)f32_to_bf16_bits(x2 * c1 - x3 * s1) << 16);      // columns i, i + 1
        const uint32_t hi = (uint32_t)f32_to_bf16_bits(x1 * c0 + x0 * s0) |
                            ((uint32_t)f32_to_bf16_bits(x3 * c1 + x2 * s1) << 16);      // i + half, i + half + 1
        if (head < ra.nh) {
          uint16_t* q = reinterpret_cast<uint16_t*>(c) + (size_t)row * ldc + (size_t)head * hd;
          *reinterpret_cast<uint32_t*>(q + i) = lo;
          *reinterpret_cast<uint32_t*>(q + i + half) = hi;
          continue;
        }
        const int slot = ra.slot_mapping[row];
        if (slot < 0) continue;
        const int page = slot / ra.page_size, off = slot % ra.page_size;
        uint16_t* tile = ra.kcache + ((size_t)page * ra.nkv + (head - ra.nh)) * ra.page_size * hd;
        *reinterpret_cast<uint32_t*>(tile + key_offset(off, i, ra.page_size)) = lo;
        *reinterpret_cast<uint32_t*>(tile + key_offset(off, i + half, ra.page_size)) = hi;
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
                  int slices, hipStream_t stream) {
  dim3 grid((N + WN * RT * 16 - 1) / (WN * RT * 16), slices), block(64 * WN * WK);
  const size_t plane = (size_t)M * ldc;
  if (c_dtype == kF32)
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, float>), grid, block, 0, stream, (const uint16_t*)a,
                       (const uint16_t*)w, (float*)c, M, N, K, lda, ldw, ldc, plane, RopeArgs{});
  else if (c_dtype == kBF16)
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, bf16_t>), grid, block, 0, stream, (const uint16_t*)a,
                       (const uint16_t*)w, (bf16_t*)c, M, N, K, lda, ldw, ldc, plane, RopeArgs{});
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <int MT>
static int launch_mt(const void* a, const void* w, void* c, int c_dtype, int M, int N, int K, int lda, int ldw,
                     int ldc, int rt, int wk, int slices, hipStream_t stream) {
#define ATOMA_CASE(R, WN_, WK_)                                                                                   \
  if (rt == R && wk == WK_) return launch<MT, R, WN_, WK_>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, slices, stream)
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
extern "C" int atoma_gemm_bf16_skinny(const void* a, const void* w, void* c, int c_dtype, int M, int N, int K,
                                      int lda, int ldw, int ldc, int rt, int wk, int slices, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || slices <= 0 || K % (32 * wk * slices) || (lda & 7) || (ldw & 7) || lda < K || ldw < K ||
      ldc < N || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || (slices > 1 && c_dtype != kF32) || slices > 65535)
    return ATOMA_ERR_SHAPE;
  const int mt = (M + 15) / 16;
  switch (mt) {
    case 1: return launch_mt<1>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, stream);
    case 2: return launch_mt<2>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, stream);
    case 3: return launch_mt<3>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, stream);
    default: return launch_mt<4>(a, w, c, c_dtype, M, N, K, lda, ldw, ldc, rt, wk, slices, stream);
  }
}

template <int MT, int RT, int WN, int WK>
static int launch_swiglu(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                         hipStream_t stream) {
  dim3 grid((N + WN * RT * 16 - 1) / (WN * RT * 16), 1), block(64 * WN * WK);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, bf16_t, true>), grid, block, 0, stream, (const uint16_t*)a,
                     (const uint16_t*)w, (bf16_t*)c, M, N, K, lda, ldw, ldc, (size_t)0, RopeArgs{});
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <int MT>
static int launch_swiglu_mt(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                            int rt, int wk, hipStream_t stream) {
  if (rt == 2 && wk == 1) return launch_swiglu<MT, 2, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, stream);
  if (rt == 4 && wk == 1) return launch_swiglu<MT, 4, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, stream);
  if (rt == 2 && wk == 4) return launch_swiglu<MT, 2, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, stream);
  if constexpr (MT < 4) {   // with four tiles of rows the epilogue does not fit the registers of eight waves
    if (rt == 2 && wk == 8) return launch_swiglu<MT, 2, 1, 8>(a, w, c, M, N, K, lda, ldw, ldc, stream);
  }
  if (rt == 4 && wk == 4) return launch_swiglu<MT, 4, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, stream);
  return ATOMA_ERR_SHAPE;
}

// The gate-up product with SiLU(gate) * up in its epilogue.  w [N, K] holds gate and up rows interleaved in blocks
// of 16 (16 gate rows, then the 16 up rows of the same outputs); c is [M, N / 2] bfloat16.  N % 32 == 0.
extern "C" int atoma_gemm_bf16_skinny_swiglu(const void* a, const void* w, void* c, int M, int N, int K, int lda,
                                             int ldw, int ldc, int rt, int wk, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % (32 * wk) || (N & 31) || (lda & 7) || (ldw & 7) || lda < K || ldw < K || ldc < N / 2 ||
      (ldc & 3) || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || ((uintptr_t)c & 7))
    return ATOMA_ERR_SHAPE;
  switch ((M + 15) / 16) {
    case 1: return launch_swiglu_mt<1>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, stream);
    case 2: return launch_swiglu_mt<2>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, stream);
    case 3: return launch_swiglu_mt<3>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, stream);
    default: return launch_swiglu_mt<4>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, stream);
  }
}

template <int MT, int RT, int WN, int WK>
static int launch_rope(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                       const RopeArgs& ra, hipStream_t stream) {
  dim3 grid((N + WN * RT * 16 - 1) / (WN * RT * 16), 1), block(64 * WN * WK);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, WN, WK, bf16_t, false, true>), grid, block, 0, stream,
                     (const uint16_t*)a, (const uint16_t*)w, (bf16_t*)c, M, N, K, lda, ldw, ldc, (size_t)0, ra);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <int MT>
static int launch_rope_mt(const void* a, const void* w, void* c, int M, int N, int K, int lda, int ldw, int ldc,
                          int rt, int wk, const RopeArgs& ra, hipStream_t stream) {
  if (rt == 1 && wk == 4) return launch_rope<MT, 1, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, ra, stream);
  if (rt == 2 && wk == 4) return launch_rope<MT, 2, 1, 4>(a, w, c, M, N, K, lda, ldw, ldc, ra, stream);
  if (rt == 1 && wk == 8) return launch_rope<MT, 1, 1, 8>(a, w, c, M, N, K, lda, ldw, ldc, ra, stream);
  if constexpr (MT < 4) {   // with four tiles of rows the epilogue does not fit the registers of eight waves
    if (rt == 2 && wk == 8) return launch_rope<MT, 2, 1, 8>(a, w, c, M, N, K, lda, ldw, ldc, ra, stream);
  }
  if (rt == 1 && wk == 1) return launch_rope<MT, 1, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, ra, stream);
  if (rt == 2 && wk == 1) return launch_rope<MT, 2, 4, 1>(a, w, c, M, N, K, lda, ldw, ldc, ra, stream);
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
                                           hipStream_t stream) {
  if (M <= 0) return 0;
  const int N = (nh + 2 * nkv) * hd;
  if (M > 64 || K <= 0 || wk <= 0 || K % (32 * wk) || (lda & 7) || (ldw & 7) || lda < K || ldw < K ||
      ldc < nh * hd || (ldc & 1) || ((uintptr_t)a & 15) || ((uintptr_t)w & 15) || ((uintptr_t)c & 3) || (hd & 3) ||
      nh <= 0 || nkv <= 0 || page_size <= 0 || !positions || !cos_t || !sin_t || !kcache || !vcache ||
      !slot_mapping || ((uintptr_t)kcache & 3))
    return ATOMA_ERR_SHAPE;
  const RopeArgs ra{positions, cos_t, sin_t, (uint16_t*)kcache, (uint16_t*)vcache, slot_mapping, page_size, nh, nkv, hd};
  switch ((M + 15) / 16) {
    case 1: return launch_rope_mt<1>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, stream);
    case 2: return launch_rope_mt<2>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, stream);
    case 3: return launch_rope_mt<3>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, stream);
    default: return launch_rope_mt<4>(a, w, c, M, N, K, lda, ldw, ldc, rt, wk, ra, stream);
  }
}
