// C[M, N] = A[M, K] * W[N, K]^T in true float32: plain fused multiply-adds, no matrix-core instruction and no
// reduced-precision mode.  A and W may be float32 or bfloat16 (widened exactly on load); C float32 or bfloat16.
// Any M, N, K.  It is the product of the 32-bit path and the fallback for shapes the MFMA kernels refuse.
//
// Weights are [out, in] row-major as checkpoints store them (models/src/llama.rs:322-325), so both operands
// are contiguous along K.  Tile 64x64, K step 16, 256 threads, 4x4 outputs per thread.  Every output sums its K
// products in ascending order of k, so a row's result does not depend on M or on its place in the batch.
#include "common.h"

using namespace atoma;

constexpr int kTile = 64;
constexpr int kStepK = 16;

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const TA* __restrict__ a, const TW* __restrict__ w, TC* __restrict__ c, int M, int N, int K,
                    int lda, int ldw, int ldc) {
  __shared__ float as[kStepK][kTile + 4];
  __shared__ float ws[kStepK][kTile + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  float acc[4][4] = {};

  for (int k0 = 0; k0 < K; k0 += kStepK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread; consecutive threads walk along k
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + i * 256;
      const int r = e >> 4, kk = e & 15;
      const int k = k0 + kk;
      as[kk][r] = (m0 + r < M && k < K) ? to_f32(a[(size_t)(m0 + r) * lda + k]) : 0.f;
      ws[kk][r] = (n0 + r < N && k < K) ? to_f32(w[(size_t)(n0 + r) * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kStepK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) c[(size_t)m * ldc + n] = from_f32<TC>(acc[i][j]);
    }
  }
}

template <typename TA, typename TW>
static int launch_c(const TA* a, const TW* w, void* c, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc,
                    hipStream_t stream) {
  dim3 grid((N + kTile - 1) / kTile, (M + kTile - 1) / kTile), block(256);
  if (c_dtype == kF32)
    hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, float>), grid, block, 0, stream, a, w, (float*)c, M, N, K, lda,
                       ldw, ldc);
  else if (c_dtype == kBF16)
    hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, bf16_t>), grid, block, 0, stream, a, w, (bf16_t*)c, M, N, K, lda,
                       ldw, ldc);
  else
    return ATOMA_ERR_DTYPE;
  ATOMA_LAUNCH_CHECK();
  return 0;
}

template <typename TA>
static int launch_w(const TA* a, const void* w, int w_dtype, void* c, int c_dtype, int M, int N, int K, int lda,
                    int ldw, int ldc, hipStream_t stream) {
  if (w_dtype == kF32) return launch_c<TA, float>(a, (const float*)w, c, c_dtype, M, N, K, lda, ldw, ldc, stream);
  if (w_dtype == kBF16) return launch_c<TA, bf16_t>(a, (const bf16_t*)w, c, c_dtype, M, N, K, lda, ldw, ldc, stream);
  return ATOMA_ERR_DTYPE;
}

extern "C" int atoma_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, void* c, int c_dtype, int M,
                                  int N, int K, int lda, int ldw, int ldc, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return ATOMA_ERR_SHAPE;
  if ((M + kTile - 1) / kTile > 65535) return ATOMA_ERR_SHAPE;
  if (a_dtype == kF32) return launch_w<float>((const float*)a, w, w_dtype, c, c_dtype, M, N, K, lda, ldw, ldc, stream);
  if (a_dtype == kBF16)
    return launch_w<bf16_t>((const bf16_t*)a, w, w_dtype, c, c_dtype, M, N, K, lda, ldw, ldc, stream);
  return ATOMA_ERR_DTYPE;
}
