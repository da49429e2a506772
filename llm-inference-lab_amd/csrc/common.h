// Shared definitions of the gfx950 kernel sources: vector types, conversions,
// wave and block reductions, and the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

typedef __bf16 bf16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define WAVE 64

// dtype codes shared with the Python side
#define DT_F32 0
#define DT_BF16 1

// Every entry point returns 0, or a non-zero code after storing a message
// that the library's llmlab_last_error() hands out.  The buffer is one per
// library and thread and is not visible to other libraries.
__attribute__((visibility("hidden"))) inline thread_local char g_llmlab_error[512] = "";

__attribute__((visibility("hidden"))) inline void llmlab_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_llmlab_error, sizeof(g_llmlab_error), fmt, ap);
  va_end(ap);
}

#define LLMLAB_REQUIRE(cond, ...)        \
  do {                                   \
    if (!(cond)) {                       \
      llmlab_set_error(__VA_ARGS__);     \
      return 1;                          \
    }                                    \
  } while (0)

#define LLMLAB_LAUNCH_CHECK(name)                                              \
  do {                                                                         \
    hipError_t e_ = hipGetLastError();                                         \
    if (e_ != hipSuccess) {                                                    \
      llmlab_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
      return 2;                                                                \
    }                                                                          \
  } while (0)

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return (bf16_t)v; }

// A vector (norm weight, bias) may be stored in float32 or in bfloat16.
__device__ __forceinline__ float load_vec(const void* p, int is_bf16, int i) {
  return is_bf16 ? (float)((const bf16_t*)p)[i] : ((const float*)p)[i];
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `red` is shared memory of at least 17 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    red[16] = t;
  }
  __syncthreads();
  return red[16];
}

// ------------------------------------------------------------------ cache order
// One page of one kv head holds P keys of d numbers, and as many values.  Both are
// kept in the order in which the matrix cores read them in the attention products
// (v_mfma_f32_16x16x32_bf16, lane l = 16 g + c), so that a wave instruction reads
// consecutive memory:
//   keys:    [16-key block][octet of d][key in block][8]     (A operand of K . Q^T:
//            lane (c, g) takes key c, numbers 8 g .. 8 g + 7 of a 32-wide piece of d;
//            the 1 KB of a (key block, piece) is lane-contiguous)
//   values:  [16-key block][16-wide block of d][group of 4 keys][number in block][4]
//            (A operand of V^T . P^T: lane (c, g) takes number c of the block and the
//            keys 4 g .. 4 g + 3; the 512 bytes of a (key block, d block) are
//            lane-contiguous)
// k = key within the page, dd = number within the head, d a multiple of 16.
__host__ __device__ inline size_t kcache_index(int k, int dd, int d) {
  return ((size_t)((k >> 4) * (d >> 3) + (dd >> 3)) * 16 + (k & 15)) * 8 + (dd & 7);
}
__host__ __device__ inline size_t vcache_index(int k, int dd, int d) {
  return ((size_t)(((k >> 4) * (d >> 4) + (dd >> 4)) * 4 + ((k & 15) >> 2)) * 16 + (dd & 15)) * 4 + (k & 3);
}
