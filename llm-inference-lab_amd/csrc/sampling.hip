// Token selection over float32 logits [rows, vocab]: greedy argmax and
// temperature sampling by inverse CDF.  One block of 1024 threads per row; any
// vocabulary size.  gfx950 only.
//
// argmax: the largest value, ties to the smallest index; NaN never wins; a row of
// nothing but NaN gives -1 (the host turns that into an error).
// sample: with temperature t <= 0 the argmax; else p = softmax(logits / t) in
// float32 and the token is the smallest index whose cumulative sum reaches
// u * total, u in [0, 1) given by the host (a seeded counter-based generator), so
// a request's choices do not depend on the batch it ran in.  Each thread owns one
// contiguous stretch of the row, so the cumulative sum has one fixed order.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

constexpr int SAMPLE_THREADS = 1024;

struct Best {
  float v;
  int i;
};

__device__ __forceinline__ Best better(Best a, Best b) {
  // b replaces a if larger, or equal with a smaller index; i < 0 means "none yet"
  if (b.i < 0) return a;
  if (a.i < 0) return b;
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ Best block_argmax(const float* __restrict__ row, int vocab, float inv_t, Best* red) {
  Best best{0.f, -1};
  int i0 = 0;
  if (((uintptr_t)row & 15) == 0) {
    // four at a time where the row allows it; a thread's candidates come in rising
    // index order, so "larger wins, equal keeps the earlier" is the tie rule here too
    const int quads = vocab >> 2;
    for (int q = threadIdx.x; q < quads; q += blockDim.x) {
      const floatx4 v4 = *(const floatx4*)(row + 4 * q);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v = v4[j] * inv_t;
        if (v == v && (best.i < 0 || v > best.v)) best = Best{v, 4 * q + j};
      }
    }
    i0 = quads << 2;
  }
  for (int i = i0 + threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i] * inv_t;
    if (v != v) continue;  // NaN
    best = better(best, Best{v, i});
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o{__shfl_xor(best.v, off, WAVE), __shfl_xor(best.i, off, WAVE)};
    best = better(best, o);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    Best t = red[0];
    for (int w = 1; w < nw; ++w) t = better(t, red[w]);
    red[16] = t;
  }
  __syncthreads();
  return red[16];
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits,
                                                                 long row_stride, int vocab,
                                                                 const float* __restrict__ temperature,
                                                                 const float* __restrict__ uniform,
                                                                 int* __restrict__ out) {
  __shared__ Best red[17];
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ float fred[17];
  __shared__ int chosen;
  const int b = blockIdx.x;
  const float* row = logits + (size_t)b * row_stride;
  const float t = temperature ? temperature[b] : 0.f;
  if (!(t > 0.f)) {
    const Best best = block_argmax(row, vocab, 1.f, red);
    if (threadIdx.x == 0) out[b] = best.i;
    return;
  }
  const float inv_t = 1.f / t;
  const Best best = block_argmax(row, vocab, inv_t, red);
  if (best.i < 0) {
    if (threadIdx.x == 0) out[b] = -1;
    return;
  }
  // contiguous stretch per thread
  const int per = (vocab + blockDim.x - 1) / blockDim.x;
  const int begin = min(vocab, (int)threadIdx.x * per), end = min(vocab, begin + per);
  float mine = 0.f;
  for (int i = begin; i < end; ++i) {
    const float v = row[i] * inv_t;
    if (v == v) mine += __expf(v - best.v);
  }
  sums[threadIdx.x] = mine;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  // thread 0 walks the 1024 partial sums: a fixed order
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int i = 0; i < (int)blockDim.x; ++i) total += sums[i];
    const float target = uniform[b] * total;
    float run = 0.f;
    int owner = -1;
    for (int i = 0; i < (int)blockDim.x; ++i) {
      if (sums[i] > 0.f) owner = i;                 // last non-empty stretch so far
      if (run + sums[i] >= target && sums[i] > 0.f) { owner = i; break; }
      run += sums[i];
    }
    fred[0] = target - run;   // what is left to cover inside the owner's stretch
    chosen = owner;
  }
  __syncthreads();
  if ((int)threadIdx.x == chosen) {
    const float left = fred[0];
    float run = 0.f;
    int pick = -1, last = -1;
    for (int i = begin; i < end; ++i) {
      const float v = row[i] * inv_t;
      if (!(v == v)) continue;
      const float p = __expf(v - best.v);
      if (p > 0.f) last = i;
      run += p;
      if (run >= left && p > 0.f) { pick = i; break; }
    }
    out[b] = pick >= 0 ? pick : (last >= 0 ? last : best.i);
  }
}

// Greedy rows in two stages so that a row's scan is spread over many blocks:
// each block takes ARGMAX_CHUNK logits and leaves (value, index); one block per
// row picks among those with the same rule, so ties still go to the smallest index.
constexpr int ARGMAX_CHUNK = 8192;

__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits,
                                                             long row_stride, int vocab,
                                                             float* __restrict__ pvals,
                                                             int* __restrict__ pidx, int chunks) {
  __shared__ Best red[17];
  const int b = blockIdx.y, ch = blockIdx.x;
  const int begin = ch * ARGMAX_CHUNK;
  const int count = min(ARGMAX_CHUNK, vocab - begin);
  const Best best = block_argmax(logits + (size_t)b * row_stride + begin, count, 1.f, red);
  if (threadIdx.x == 0) {
    pvals[(size_t)b * chunks + ch] = best.v;
    pidx[(size_t)b * chunks + ch] = best.i < 0 ? -1 : begin + best.i;
  }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pvals,
                                                          const int* __restrict__ pidx, int chunks,
                                                          int* __restrict__ out) {
  const int b = blockIdx.x;
  Best best{0.f, -1};
  for (int i = threadIdx.x; i < chunks; i += 64)
    best = better(best, Best{pvals[(size_t)b * chunks + i], pidx[(size_t)b * chunks + i]});
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o{__shfl_xor(best.v, off, WAVE), __shfl_xor(best.i, off, WAVE)};
    best = better(best, o);
  }
  if (threadIdx.x == 0) out[b] = best.i;
}

// Both stages in one kernel: every block leaves its (value, index) with stores of device
// scope (written through to memory, past the L2 of its die), waits until they are done and
// counts itself in at the row's counter; the block that arrives last picks among all of
// them and sets the counter back to zero.  No fence, and nobody waits for anybody.
__global__ __launch_bounds__(256) void argmax_one_pass_kernel(const float* __restrict__ logits,
                                                              long row_stride, int vocab,
                                                              float* pvals, int* pidx, int chunks,
                                                              int* arrived, int* __restrict__ out) {
  __shared__ Best red[17];
  __shared__ int s_last;
  const int b = blockIdx.y, ch = blockIdx.x;
  const int begin = ch * ARGMAX_CHUNK;
  const int count = min(ARGMAX_CHUNK, vocab - begin);
  const Best best = block_argmax(logits + (size_t)b * row_stride + begin, count, 1.f, red);
  if (threadIdx.x == 0) {
    __hip_atomic_store(&pvals[(size_t)b * chunks + ch], best.v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&pidx[(size_t)b * chunks + ch], best.i < 0 ? -1 : begin + best.i, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0);
    const int before = __hip_atomic_fetch_add(&arrived[b], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = before == chunks - 1;
    if (s_last) __hip_atomic_store(&arrived[b], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last || threadIdx.x >= 64) return;
  Best all{0.f, -1};
  for (int i = threadIdx.x; i < chunks; i += 64)
    all = better(all, Best{__hip_atomic_load(&pvals[(size_t)b * chunks + i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT),
                           __hip_atomic_load(&pidx[(size_t)b * chunks + i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)});
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o{__shfl_xor(all.v, off, WAVE), __shfl_xor(all.i, off, WAVE)};
    all = better(all, o);
  }
  if (threadIdx.x == 0) out[b] = all.i;
}

// workspace: at least rows * ceil(vocab / 8192) * 2 words.  arrived (may be null: two
// kernels then): at least `rows` counters that are zero now and are left zero.
extern "C" int llmlab_argmax(const float* logits, long row_stride, int rows, int vocab, int* out,
                             float* workspace, size_t workspace_floats, int* arrived, size_t arrived_ints,
                             hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax: bad sizes rows=%d vocab=%d",
                 rows, vocab);
  if (rows == 0) return 0;
  const int chunks = (vocab + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
  LLMLAB_REQUIRE(workspace != nullptr && (size_t)rows * chunks * 2 <= workspace_floats,
                 "argmax: workspace too small");
  LLMLAB_REQUIRE(rows <= 65535, "argmax: too many rows");
  float* pvals = workspace;
  int* pidx = (int*)(workspace + (size_t)rows * chunks);
  if (arrived != nullptr && (size_t)rows <= arrived_ints && chunks > 1) {
    hipLaunchKernelGGL(argmax_one_pass_kernel, dim3(chunks, rows), dim3(256), 0, stream, logits, row_stride,
                       vocab, pvals, pidx, chunks, arrived, out);
    LLMLAB_LAUNCH_CHECK("argmax (one pass)");
    return 0;
  }
  hipLaunchKernelGGL(argmax_partial_kernel, dim3(chunks, rows), dim3(256), 0, stream, logits, row_stride,
                     vocab, pvals, pidx, chunks);
  LLMLAB_LAUNCH_CHECK("argmax (partial)");
  hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(64), 0, stream, pvals, pidx, chunks, out);
  LLMLAB_LAUNCH_CHECK("argmax (final)");
  return 0;
}

// The same selection for callers that cannot allocate: the partial maxima go to a
// device array of this file.  The array's name is only a handle in host code; the
// address on each GPU comes from hipGetSymbolAddress, asked for once per device with
// that device current, and the kernels take that address as an argument.
constexpr int STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) float scratch[2 * LLMLAB_ARGMAX_STATIC_PAIRS];
static float* g_scratch_ptr[STATIC_MAX_DEVICES] = {};
static std::mutex g_scratch_mutex;

static int static_scratch(float** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  LLMLAB_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
  LLMLAB_REQUIRE(device >= 0 && device < STATIC_MAX_DEVICES, "argmax_static: device %d is beyond %d",
                 device, STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    LLMLAB_REQUIRE(e == hipSuccess && p != nullptr, "argmax_static: hipGetSymbolAddress failed: %s",
                   hipGetErrorString(e));
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  return 0;
}

extern "C" int llmlab_argmax_static(const float* logits, long row_stride, int rows, int vocab, int* out,
                                    hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab,
                 "argmax_static: bad sizes rows=%d vocab=%d", rows, vocab);
  if (rows == 0) return 0;
  LLMLAB_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: null logits or output");
  const int chunks = (vocab + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
  LLMLAB_REQUIRE(rows <= 65535, "argmax_static: too many rows");
  LLMLAB_REQUIRE((size_t)rows * chunks <= (size_t)LLMLAB_ARGMAX_STATIC_PAIRS,
                 "argmax_static: %d rows of %d logits need %zu partial results, the static array "
                 "holds %d", rows, vocab, (size_t)rows * chunks, LLMLAB_ARGMAX_STATIC_PAIRS);
  float* base = nullptr;
  if (static_scratch(&base) != 0) return 1;
  float* pvals = base;
  int* pidx = (int*)(base + (size_t)rows * chunks);
  hipLaunchKernelGGL(argmax_partial_kernel, dim3(chunks, rows), dim3(256), 0, stream, logits, row_stride,
                     vocab, pvals, pidx, chunks);
  LLMLAB_LAUNCH_CHECK("argmax_static (partial)");
  hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(64), 0, stream, pvals, pidx, chunks, out);
  LLMLAB_LAUNCH_CHECK("argmax_static (final)");
  return 0;
}

extern "C" int llmlab_sample(const float* logits, long row_stride, int rows, int vocab,
                             const float* temperature, const float* uniform, int* out,
                             hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample: bad sizes rows=%d vocab=%d",
                 rows, vocab);
  LLMLAB_REQUIRE(temperature == nullptr || uniform != nullptr,
                 "sample: temperatures need uniform numbers");
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride,
                     vocab, temperature, uniform, out);
  LLMLAB_LAUNCH_CHECK("sample");
  return 0;
}
