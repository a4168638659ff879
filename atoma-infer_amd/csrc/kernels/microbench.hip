// What this GPU delivers, measured: a read stream and a copy over device memory, and a loop of bfloat16 MFMAs.
// bench.py prints these beside the published peaks (8 TB/s, 2.5 PFLOP/s), which stay the yardstick of its fractions.
// And what a chain of dependent kernels costs beyond its bytes: the read stream launched over and over inside a
// graph (with no bytes: an empty kernel behind another), and, for comparison, a barrier over the whole grid inside
// one kernel, the thing a single persistent kernel would put in a launch's place.
#include "common.h"

using namespace atoma;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// every thread reads 16-byte words with a stride of the whole grid, U in flight; all of what is read is folded into
// one word (so that the loads stay 16 bytes wide) that is stored only if it has a value it practically never has
template <int U>
__global__ void __launch_bounds__(256)
probe_read_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink) {
  uint32_t acc = 0;
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + (U - 1) * stride < n16; i += U * stride) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = src[i + u * stride];
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const uint4 a = src[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

__global__ void __launch_bounds__(256)
probe_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    dst[i] = a, dst[i + stride] = b, dst[i + 2 * stride] = c, dst[i + 3 * stride] = d;
  }
  for (; i < n16; i += stride) dst[i] = src[i];
}

// four independent accumulators a wave, so that the matrix core's pipeline stays full
__global__ void __launch_bounds__(256)
probe_mfma_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(float)((threadIdx.x + i) & 3);
    b[i] = (__bf16)(float)((threadIdx.x * 3 + i) & 1);
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int it = 0; it < iters; ++it) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == -1.0f) sink[0] = s;      // sums of non-negative products: never
}

// grid: workgroups of 256 threads.  src (and dst) hold `bytes` bytes, a multiple of 16.  in_flight: 4, 8 or 16
// loads of 16 bytes a thread.
extern "C" int atoma_probe_read(const void* src, size_t bytes, int grid, int in_flight, void* sink,
                                hipStream_t stream) {
  if (grid <= 0 || bytes % 16 || ((uintptr_t)src & 15)) return ATOMA_ERR_SHAPE;
#define ATOMA_READ(U)                                                                                          \
  hipLaunchKernelGGL(probe_read_kernel<U>, dim3(grid), dim3(256), 0, stream, (const uint4*)src, bytes / 16,   \
                     (uint32_t*)sink)
  if (in_flight == 4) ATOMA_READ(4);
  else if (in_flight == 8) ATOMA_READ(8);
  else if (in_flight == 16) ATOMA_READ(16);
  else return ATOMA_ERR_SHAPE;
#undef ATOMA_READ
  ATOMA_LAUNCH_CHECK();
  return 0;
}

extern "C" int atoma_probe_copy(const void* src, void* dst, size_t bytes, int grid, hipStream_t stream) {
  if (grid <= 0 || bytes % 16 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(probe_copy_kernel, dim3(grid), dim3(256), 0, stream, (const uint4*)src, (uint4*)dst, bytes / 16);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// floating-point operations of one launch: grid * 4 waves * iters * 4 MFMAs * (2 * 32 * 32 * 16)
extern "C" int atoma_probe_mfma(int iters, int grid, void* sink, hipStream_t stream) {
  if (grid <= 0 || iters <= 0) return ATOMA_ERR_SHAPE;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(grid), dim3(256), 0, stream, iters, (float*)sink);
  ATOMA_LAUNCH_CHECK();
  return 0;
}

// A barrier over the whole grid, nb times in one kernel: every workgroup counts itself in at a device-wide counter and
// polls it until all have (relaxed atomics that go through to memory; no fence that would write back or invalidate a
// cache).  Every wait is bounded: past kSpinLimit polls a workgroup writes an error word and no wait spins again.
constexpr unsigned kSpinLimit = 1u << 18;

__global__ void __launch_bounds__(512)
probe_barrier_kernel(unsigned* __restrict__ counter, unsigned* __restrict__ err, int nb) {
  for (int b = 0; b < nb; ++b) {
    __syncthreads();
    if (threadIdx.x == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
      const unsigned target = (unsigned)(b + 1) * gridDim.x;
      __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      unsigned spins = 0;
      while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
        __builtin_amdgcn_s_sleep(1);
        if (++spins > kSpinLimit) {
          __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
      }
    }
    __syncthreads();
  }
}

// ctrl: 128 zeroed 32-bit words (word 0: the counter, word 64: set if a wait ran out).  grid workgroups of 512 threads,
// which must all be resident at once: refused if the device cannot hold them.
extern "C" int atoma_probe_barrier(void* ctrl, int grid, int nb, hipStream_t stream) {
  if (grid <= 0 || nb <= 0 || ((uintptr_t)ctrl & 3)) return ATOMA_ERR_SHAPE;
  int dev = 0, cus = 0, per_cu = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, probe_barrier_kernel, 512, 0);
  if (e != hipSuccess) return (int)e;
  if ((long long)grid > (long long)cus * per_cu) return ATOMA_ERR_SHAPE;
  unsigned* c = (unsigned*)ctrl;
  hipLaunchKernelGGL(probe_barrier_kernel, dim3(grid), dim3(512), 0, stream, c, c + 64, nb);
  ATOMA_LAUNCH_CHECK();
  return 0;
}
