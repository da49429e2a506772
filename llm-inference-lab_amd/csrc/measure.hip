// What the machine gives, measured with the simplest kernels that can reach it: the
// denominators of the roofline fractions that the benchmark reports beside the published
// peaks.  gfx950 only.  Not on the product path: bench.py loads this library in a child
// process before anything else is timed.
//
//   read stream     every lane reads 16 bytes at a time over a large buffer and keeps an
//                   xor of what it read (nothing is written)
//   copy stream     the same with one 16-byte store per load
//   MFMA issue      waves that do nothing but matrix instructions on registers:
//                   v_mfma_f32_16x16x32_bf16 (the engine's bfloat16 products) and
//                   v_mfma_f32_32x32x2_f32 (32-bit products and sums)
//   grid barrier    one block per compute unit, all meeting at a counter in memory again
//                   and again: what a device-wide barrier inside a kernel would cost
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_m;
typedef __attribute__((ext_vector_type(4))) float floatx4_m;
typedef __attribute__((ext_vector_type(16))) float floatx16_m;

constexpr int STREAM_THREADS = 256;
constexpr int STREAM_UNROLL = 8;

__global__ __launch_bounds__(STREAM_THREADS) void read_stream_kernel(const uint4* __restrict__ src, size_t n16,
                                                                     uint4* __restrict__ sink) {
  uint4 acc = {0u, 0u, 0u, 0u};
  const size_t stride = (size_t)gridDim.x * STREAM_THREADS;
  size_t i = (size_t)blockIdx.x * STREAM_THREADS + threadIdx.x;
  for (; i + (STREAM_UNROLL - 1) * stride < n16; i += STREAM_UNROLL * stride) {
    uint4 v[STREAM_UNROLL];
#pragma unroll
    for (int u = 0; u < STREAM_UNROLL; ++u) v[u] = src[i + u * stride];
#pragma unroll
    for (int u = 0; u < STREAM_UNROLL; ++u) {
      acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w;
    }
  }
  for (; i < n16; i += stride) {
    const uint4 v = src[i];
    acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
  }
  // (a store that depends on everything read, taken by next to no lane)
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[threadIdx.x] = acc;
}

__global__ __launch_bounds__(STREAM_THREADS) void copy_stream_kernel(const uint4* __restrict__ src,
                                                                     uint4* __restrict__ dst, size_t n16) {
  const size_t stride = (size_t)gridDim.x * STREAM_THREADS;
  size_t i = (size_t)blockIdx.x * STREAM_THREADS + threadIdx.x;
  for (; i + (STREAM_UNROLL - 1) * stride < n16; i += STREAM_UNROLL * stride) {
    uint4 v[STREAM_UNROLL];
#pragma unroll
    for (int u = 0; u < STREAM_UNROLL; ++u) v[u] = src[i + u * stride];
#pragma unroll
    for (int u = 0; u < STREAM_UNROLL; ++u) dst[i + u * stride] = v[u];
  }
  for (; i < n16; i += stride) dst[i] = src[i];
}

// Eight independent accumulators per wave, so that no instruction waits for the one before.
__global__ __launch_bounds__(256) void mfma_bf16_kernel(int iterations, float* __restrict__ sink) {
  bf16x8_m a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(0.001f * (float)((threadIdx.x + i) & 7));
    b[i] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + i) & 7));
  }
  floatx4_m acc[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) acc[k] = floatx4_m{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[k], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) total += acc[k][0] + acc[k][1] + acc[k][2] + acc[k][3];
  if (total == 12345.678f) sink[threadIdx.x] = total;
}

__global__ __launch_bounds__(256) void mfma_f32_kernel(int iterations, float* __restrict__ sink) {
  const float a = 0.001f * (float)(threadIdx.x & 7), b = 0.002f * (float)((threadIdx.x * 3) & 7);
  floatx16_m acc[4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[k], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) total += acc[k][i];
  if (total == 12345.678f) sink[threadIdx.x] = total;
}

// What a device-wide barrier costs inside one kernel: every block counts itself in with an
// atomic of device scope and reads the counter (device scope too, so the read passes the L2
// of its die by) until all have arrived, `rounds` times.  The wait is bounded: a block that
// has read the counter `spin_limit` times in one round without seeing it full sets `*failed`
// and leaves, and so, each at its own limit, do the others.  One block per compute unit at
// most, so that all of them are resident at once.
__global__ __launch_bounds__(64) void barrier_rounds_kernel(int rounds, int* counter, int* failed,
                                                            long spin_limit) {
  if (threadIdx.x != 0) return;
  for (int r = 0; r < rounds; ++r) {
    const int full = (r + 1) * (int)gridDim.x;
    __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    long spins = 0;
    while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < full) {
      if (++spins > spin_limit) {
        __hip_atomic_store(failed, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
      }
      __builtin_amdgcn_s_sleep(1);
    }
  }
}

static int check_launch() { return hipGetLastError() == hipSuccess ? 0 : 1; }

// counter and failed: two ints that are zero now.  blocks: at most the number of compute units.
extern "C" int llmlab_measure_barrier(int blocks, int rounds, int* counter, int* failed, long spin_limit,
                                      hipStream_t stream) {
  if (counter == nullptr || failed == nullptr || blocks <= 0 || blocks > 1024 || rounds <= 0 || spin_limit < 0)
    return 1;
  hipLaunchKernelGGL(barrier_rounds_kernel, dim3(blocks), dim3(64), 0, stream, rounds, counter, failed, spin_limit);
  return check_launch();
}

// bytes: a multiple of 16; sink: at least 4 KB.  Reads `bytes` once.
extern "C" int llmlab_measure_read(const void* src, size_t bytes, void* sink, int blocks, hipStream_t stream) {
  if (src == nullptr || sink == nullptr || bytes % 16 != 0 || blocks <= 0) return 1;
  hipLaunchKernelGGL(read_stream_kernel, dim3(blocks), dim3(STREAM_THREADS), 0, stream, (const uint4*)src,
                     bytes / 16, (uint4*)sink);
  return check_launch();
}

// Reads `bytes` and writes `bytes`.
extern "C" int llmlab_measure_copy(const void* src, void* dst, size_t bytes, int blocks, hipStream_t stream) {
  if (src == nullptr || dst == nullptr || bytes % 16 != 0 || blocks <= 0) return 1;
  hipLaunchKernelGGL(copy_stream_kernel, dim3(blocks), dim3(STREAM_THREADS), 0, stream, (const uint4*)src,
                     (uint4*)dst, bytes / 16);
  return check_launch();
}

// `blocks` blocks of four waves; returns the floating-point operations of the launch through
// *flops (2 m n k per instruction).  sink: at least 1 KB.
extern "C" int llmlab_measure_mfma(int f32, int blocks, int iterations, float* sink, double* flops,
                                   hipStream_t stream) {
  if (sink == nullptr || blocks <= 0 || iterations <= 0) return 1;
  if (f32) {
    hipLaunchKernelGGL(mfma_f32_kernel, dim3(blocks), dim3(256), 0, stream, iterations, sink);
    if (flops) *flops = (double)blocks * 4 * iterations * 4 * (2.0 * 32 * 32 * 2);
  } else {
    hipLaunchKernelGGL(mfma_bf16_kernel, dim3(blocks), dim3(256), 0, stream, iterations, sink);
    if (flops) *flops = (double)blocks * 4 * iterations * 8 * (2.0 * 16 * 16 * 32);
  }
  return check_launch();
}
