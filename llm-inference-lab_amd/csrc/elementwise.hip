// Embedding gather, RMSNorm, and rotary position encoding fused with the
// write of keys and values into the paged cache.  gfx950 only.
#include "common.h"

extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

extern "C" int llmlab_abi_version() { return 6; }

// --------------------------------------------------------------- embedding
// out[r, :] = float(table[ids[r], :]); an id outside [0, vocab) is clamped (the
// host has already refused such ids; the clamp keeps a stale device-side id
// from reading outside the table).
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int hidden, int vocab) {
  const int r = blockIdx.x;
  int id = ids[r];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + (size_t)id * hidden;
  float* dst = out + (size_t)r * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = to_float(src[c]);
}

// The same from a bfloat16 table packed in MFMA fragment order (see
// llmlab_pack_weight): row `id` is lane column id % 16 of strip id / 16, its
// columns 8 ch .. 8 ch + 7 the 16 bytes of lane (ch % 4) * 16 + id % 16 in tile ch / 4.
__global__ void embed_packed_kernel(const bf16_t* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int hidden, int vocab) {
  const int r = blockIdx.x;
  int id = ids[r];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const int tiles = (hidden + 31) >> 5;
  const bf16_t* strip = table + (size_t)(id >> 4) * tiles * 512;
  float* dst = out + (size_t)r * hidden;
  for (int ch = threadIdx.x; ch < (hidden >> 3); ch += blockDim.x) {
    const bf16x8 v = *(const bf16x8*)(strip + (size_t)(ch >> 2) * 512 + (((ch & 3) << 4) + (id & 15)) * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) dst[ch * 8 + j] = (float)v[j];
  }
}

// dtype DT_BF16 + packed != 0: the table is in fragment order (hidden a multiple of 8).
extern "C" int llmlab_embed(const void* table, int dtype, int packed, const int* ids, float* out, int rows,
                            int hidden, int vocab, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes rows=%d hidden=%d vocab=%d",
                 rows, hidden, vocab);
  LLMLAB_REQUIRE(!packed || (dtype == DT_BF16 && hidden % 8 == 0), "embed: a packed table is bfloat16, %d wide", hidden);
  if (rows == 0) return 0;
  dim3 grid(rows), block(256);
  if (packed)
    hipLaunchKernelGGL(embed_packed_kernel, grid, dim3(128), 0, stream, (const bf16_t*)table, ids, out,
                       hidden, vocab);
  else if (dtype == DT_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, ids, out,
                       hidden, vocab);
  else
    hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, (const float*)table, ids, out,
                       hidden, vocab);
  LLMLAB_LAUNCH_CHECK("embed");
  return 0;
}

// ----------------------------------------------------------------- RMSNorm
// out[i, :] = x[row_i, :] * rsqrt(mean(x[row_i]^2) + eps) * w, row_i = rows[i] or
// i.  The square, the mean, the rsqrt and both products are float32; one
// rounding to T at the end.
// With pieces that a product left for the stream (pend[s][row, :], s < splits), the
// row is first made whole, x[r] += sum_s pend[s][r] (written back: every element
// belongs to one thread), and then normed; rows must not be gathered then.
// A thread keeps its first KEEP groups of W elements (and their weights) in
// registers, so a row of up to KEEP * W * blockDim.x elements costs one trip to
// memory; what lies beyond is read again after the reduction.  VEC: groups of four
// (hidden % 4 == 0 and 16-byte aligned rows).
template <typename T, bool VEC, int G>
__global__ void rmsnorm_kernel(float* __restrict__ x, const void* __restrict__ w, int w_bf16,
                               float eps, T* __restrict__ out, const int* __restrict__ rows,
                               int hidden, const float* __restrict__ pend, int splits, size_t pend_stride) {
  constexpr int KEEP = 4, W = VEC ? 4 : 1;
  __shared__ float red[17];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* src = x + (size_t)r * hidden;
  const float* prow = pend + (size_t)r * hidden;
  const int stride = blockDim.x * W;
  float keep[KEEP][W], wk[KEEP][W];
  float ss = 0.f;
  // Pieces come G at a time, loads unconditional (past the last piece: the last one again,
  // not added), so that they travel together instead of one after the other: G = 4 for
  // the many pieces that few rows bring (a step bound by latency).  One or two pieces,
  // which many rows bring, are taken one by one (G = 1, a kernel of its own): that step
  // is bound by the memory rate, and the registers of a group would cost it waves (2,048
  // rows of 896 with two pieces: 8.8 us one by one, 10.7 in pairs).
  auto fetch = [&](int c, float* v) {       // the whole values of elements c .. c+W-1, written back if pieces came in
    if constexpr (VEC) {
      floatx4 t = *(const floatx4*)(src + c);
      for (int s0 = 0; s0 < splits; s0 += G) {
        floatx4 p[G];
#pragma unroll
        for (int j = 0; j < G; ++j) p[j] = *(const floatx4*)(prow + (size_t)min(s0 + j, splits - 1) * pend_stride + c);
#pragma unroll
        for (int j = 0; j < G; ++j)
          if (s0 + j < splits) t += p[j];
      }
      if (splits > 0) *(floatx4*)(src + c) = t;
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] = t[e];
    } else {
      float t = src[c];
      for (int s0 = 0; s0 < splits; s0 += G) {
        float p[G];
#pragma unroll
        for (int j = 0; j < G; ++j) p[j] = prow[(size_t)min(s0 + j, splits - 1) * pend_stride + c];
#pragma unroll
        for (int j = 0; j < G; ++j) t += s0 + j < splits ? p[j] : 0.f;
      }
      if (splits > 0) src[c] = t;
      v[0] = t;
    }
  };
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = threadIdx.x * W + j * stride;
    if (c < hidden) {
      fetch(c, keep[j]);
#pragma unroll
      for (int e = 0; e < W; ++e) { wk[j][e] = load_vec(w, w_bf16, c + e); ss += keep[j][e] * keep[j][e]; }
    }
  }
  for (int c = threadIdx.x * W + KEEP * stride; c < hidden; c += stride) {
    float v[W];
    fetch(c, v);
#pragma unroll
    for (int e = 0; e < W; ++e) ss += v[e] * v[e];
  }
  ss = block_sum(ss, red);      // (a barrier; below a thread reads back only what it wrote itself)
  const float inv = rsqrtf(ss / (float)hidden + eps);
  T* dst = out + (size_t)i * hidden;
#pragma unroll
  for (int j = 0; j < KEEP; ++j) {
    const int c = threadIdx.x * W + j * stride;
    if (c < hidden) {
      if constexpr (VEC) {
        typedef T outx4 __attribute__((ext_vector_type(4)));
        outx4 o;
#pragma unroll
        for (int e = 0; e < W; ++e) o[e] = from_float<T>(keep[j][e] * inv * wk[j][e]);
        *(outx4*)(dst + c) = o;
      } else {
        dst[c] = from_float<T>(keep[j][0] * inv * wk[j][0]);
      }
    }
  }
  for (int c = threadIdx.x * W + KEEP * stride; c < hidden; c += stride)
#pragma unroll
    for (int e = 0; e < W; ++e) dst[c + e] = from_float<T>(src[c + e] * inv * load_vec(w, w_bf16, c + e));
}

extern "C" int llmlab_rmsnorm(float* x, const void* w, int w_dtype, float eps, void* out,
                              int out_dtype, const int* rows, int n_out, int hidden,
                              const float* pend, int splits, size_t pend_stride, hipStream_t stream) {
  LLMLAB_REQUIRE(n_out >= 0 && hidden > 0, "rmsnorm: bad sizes n=%d hidden=%d", n_out, hidden);
  LLMLAB_REQUIRE(splits == 0 || (pend != nullptr && rows == nullptr && pend_stride >= (size_t)n_out * hidden),
                 "rmsnorm: pending sums go with all rows in order");
  if (n_out == 0) return 0;
  const bool vec = hidden % 4 == 0 && pend_stride % 4 == 0 &&
                   (((uintptr_t)x | (uintptr_t)pend | (uintptr_t)out) & 15) == 0;
  // few rows are bound by latency, not by the memory rate: then a row is spread over as
  // many threads as it has groups of four numbers, so that every thread's loads (its
  // numbers and the pieces owed to them) are one round
  int threads = hidden >= 8192 ? 512 : 256;
  if (n_out <= 128)
    while (threads < 1024 && threads * 4 < hidden) threads *= 2;
  dim3 grid(n_out), block(threads);
#define LLMLAB_RMSNORM(T, VEC)                                                                             \
  do {                                                                                                     \
    if (splits > 2)                                                                                        \
      hipLaunchKernelGGL((rmsnorm_kernel<T, VEC, 4>), grid, block, 0, stream, x, w, w_dtype == DT_BF16, eps, \
                         (T*)out, rows, hidden, pend, splits, pend_stride);                                \
    else                                                                                                   \
      hipLaunchKernelGGL((rmsnorm_kernel<T, VEC, 1>), grid, block, 0, stream, x, w, w_dtype == DT_BF16, eps, \
                         (T*)out, rows, hidden, pend, splits, pend_stride);                                \
  } while (0)
  if (out_dtype == DT_BF16) { if (vec) LLMLAB_RMSNORM(bf16_t, true); else LLMLAB_RMSNORM(bf16_t, false); }
  else                      { if (vec) LLMLAB_RMSNORM(float, true);  else LLMLAB_RMSNORM(float, false); }
#undef LLMLAB_RMSNORM
  LLMLAB_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// ------------------------------------------------- rotary + cache write
// One block per (row, head) of the packed projection output
//   qkv[r] = [q heads | k heads | v heads], each head `d` wide.
// q heads: rotated in place.  k heads: rotated, written in place and to the
// key page  K[page][kvh][off][d].  v heads: written to the value page, which is
// in the order of the attention kernels' fragments (kcache_index, vcache_index).  page = table[row_req[r]][pos / P],
// off = pos % P.  Angles, sine and cosine in float32; one rounding to T.
// Sine and cosine of a float32 angle.  float32 results: the library routine (exact
// range reduction).  bfloat16 results: the hardware instructions, which take
// revolutions; the reduction  r = frac(angle / 2 pi)  adds an error of the size the
// float32 angle itself has (position * frequency rounded to 24 bits).
template <typename T>
__device__ __forceinline__ void rope_sincos(float angle, float* s, float* c) {
  if constexpr (sizeof(T) == 4) {
    sincosf(angle, s, c);
  } else {
    float r = angle * 0.15915494309189535f;
    r -= floorf(r);
    *s = __builtin_amdgcn_sinf(r);
    *c = __builtin_amdgcn_cosf(r);
  }
}

// One block per row; a thread keeps its pair index over the heads it visits when
// the block size is a multiple of d/2, so its sine and cosine are computed once.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ qkv, int row_stride, int nq, int nkv, int d, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ row_req, const int* __restrict__ table,
    int table_stride, int page_size, T* __restrict__ kcache, T* __restrict__ vcache) {
  const int r = blockIdx.x;
  const int pos = positions[r];
  T* row = qkv + (size_t)r * row_stride;
  size_t page = 0;
  int off = 0;
  if (kcache) {
    page = (size_t)table[(size_t)row_req[r] * table_stride + pos / page_size];
    off = pos % page_size;
  }
  const int half = d >> 1;
  const int qk_heads = (kcache || inv_freq) ? nq + nkv : 0;     // heads rotated (k also written)
  const bool fixed_pair = (int)blockDim.x % half == 0;
  float s0 = 0.f, c0 = 1.f;
  if (inv_freq && fixed_pair) rope_sincos<T>((float)pos * inv_freq[threadIdx.x % half], &s0, &c0);
  for (int idx = threadIdx.x; idx < qk_heads * half; idx += blockDim.x) {
    const int head = idx / half, i = idx - head * half;
    T* base = row + (size_t)head * d;
    float lo = to_float(base[i]), hi = to_float(base[i + half]);
    if (inv_freq) {
      float s = s0, c = c0;
      if (!fixed_pair) rope_sincos<T>((float)pos * inv_freq[i], &s, &c);
      const float nlo = lo * c - hi * s, nhi = hi * c + lo * s;
      lo = nlo;
      hi = nhi;
      base[i] = from_float<T>(lo);
      base[i + half] = from_float<T>(hi);
    }
    if (head >= nq && kcache) {
      T* kdst = kcache + (page * nkv + (head - nq)) * (size_t)page_size * d;
      kdst[kcache_index(off, i, d)] = from_float<T>(lo);
      kdst[kcache_index(off, i + half, d)] = from_float<T>(hi);
    }
  }
  if (vcache) {
    const T* vsrc = row + (size_t)(nq + nkv) * d;
    for (int idx = threadIdx.x; idx < nkv * d; idx += blockDim.x) {
      const int head = idx / d, i = idx - head * d;
      vcache[(page * nkv + head) * (size_t)d * page_size + vcache_index(off, i, d)] = vsrc[idx];
    }
  }
}

extern "C" int llmlab_rope_kv_write(void* qkv, int dtype, int rows, int row_stride, int nq, int nkv,
                                    int d, const float* inv_freq, const int* positions,
                                    const int* row_req, const int* table, int table_stride,
                                    int page_size, void* kcache, void* vcache, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && nq > 0 && nkv >= 0 && d > 0 && d % 2 == 0,
                 "rope_kv_write: bad sizes rows=%d nq=%d nkv=%d d=%d", rows, nq, nkv, d);
  LLMLAB_REQUIRE(row_stride >= (nq + 2 * nkv) * d || (kcache == nullptr && row_stride >= nq * d),
                 "rope_kv_write: row stride %d is smaller than the heads it holds", row_stride);
  LLMLAB_REQUIRE((kcache == nullptr) == (vcache == nullptr), "rope_kv_write: need both caches or none");
  LLMLAB_REQUIRE(kcache == nullptr || (table != nullptr && row_req != nullptr && page_size > 0),
                 "rope_kv_write: a cache write needs a block table");
  if (rows == 0) return 0;
  // Without a cache only q and k heads are rotated (k in place) and v is left alone.
  if (!kcache && !inv_freq) return 0;
  dim3 grid(rows), block(256);
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(rope_kv_write_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)qkv, row_stride,
                       nq, nkv, d, inv_freq, positions, row_req, table, table_stride, page_size,
                       (bf16_t*)kcache, (bf16_t*)vcache);
  else
    hipLaunchKernelGGL(rope_kv_write_kernel<float>, grid, block, 0, stream, (float*)qkv, row_stride,
                       nq, nkv, d, inv_freq, positions, row_req, table, table_stride, page_size,
                       (float*)kcache, (float*)vcache);
  LLMLAB_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// The same from a q/k/v product that was left in pieces along its inner size
// (float32 parts[s][row][ld], s < splits): one block per (row, head) sums the pieces in
// their order, adds the bias, rotates q and k heads and writes q to q_out [rows, ldq] and
// k and v into their cache pages (skipped without a cache).  One rounding, as in the
// product kernels that have this epilogue.  For some rows of a large matrix: cut along
// K the product spreads over the chip, which a head per block does not.
__global__ __launch_bounds__(256) void qkv_from_pieces_kernel(
    const float* __restrict__ parts, int splits, size_t part_stride, int ld, const void* __restrict__ bias,
    int bias_bf16, int nq, int nkv, int d, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ row_req, const int* __restrict__ table,
    int table_stride, int page_size, bf16_t* __restrict__ kcache, bf16_t* __restrict__ vcache,
    bf16_t* __restrict__ q_out, int ldq) {
  const int r = blockIdx.x, head = blockIdx.y;
  if (head >= nq && !kcache) return;
  const int pos = positions[r];
  size_t page = 0;
  int off = 0;
  if (head >= nq) {
    page = (size_t)table[(size_t)row_req[r] * table_stride + pos / page_size];
    off = pos % page_size;
  }
  const int half = d >> 1;
  const float* src = parts + (size_t)r * ld + (size_t)head * d;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float lo = bias ? load_vec(bias, bias_bf16, head * d + i) : 0.f;
    float hi = bias ? load_vec(bias, bias_bf16, head * d + i + half) : 0.f;
    // four pieces at a time, loads unconditional (past the last piece: the last one again,
    // not added), so that they travel together
    for (int s0 = 0; s0 < splits; s0 += 4) {
      float pl[4], ph[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float* ps = src + (size_t)min(s0 + j, splits - 1) * part_stride;
        pl[j] = ps[i];
        ph[j] = ps[i + half];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (s0 + j < splits) {
          lo += pl[j];
          hi += ph[j];
        }
    }
    if (inv_freq && head < nq + nkv) {
      float sn, cs;
      rope_sincos<bf16_t>((float)pos * inv_freq[i], &sn, &cs);
      const float nlo = lo * cs - hi * sn, nhi = hi * cs + lo * sn;
      lo = nlo;
      hi = nhi;
    }
    if (head < nq) {
      bf16_t* dst = q_out + (size_t)r * ldq + (size_t)head * d;
      dst[i] = (bf16_t)lo;
      dst[i + half] = (bf16_t)hi;
    } else if (head < nq + nkv) {
      bf16_t* kdst = kcache + (page * nkv + (head - nq)) * (size_t)page_size * d;
      kdst[kcache_index(off, i, d)] = (bf16_t)lo;
      kdst[kcache_index(off, i + half, d)] = (bf16_t)hi;
    } else {
      bf16_t* vdst = vcache + (page * nkv + (head - nq - nkv)) * (size_t)d * page_size;
      vdst[vcache_index(off, i, d)] = (bf16_t)lo;
      vdst[vcache_index(off, i + half, d)] = (bf16_t)hi;
    }
  }
}

extern "C" int llmlab_qkv_from_pieces(const float* parts, int splits, size_t part_stride, int ld,
                                      const void* bias, int bias_dtype, int rows, int nq, int nkv, int d,
                                      const float* inv_freq, const int* positions, const int* row_req,
                                      const int* table, int table_stride, int page_size, void* kcache,
                                      void* vcache, void* q_out, int ldq, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && nq > 0 && nkv >= 0 && d > 0 && d % 2 == 0 && nq + 2 * nkv <= 65535,
                 "qkv_from_pieces: bad sizes rows=%d nq=%d nkv=%d d=%d", rows, nq, nkv, d);
  LLMLAB_REQUIRE(splits >= 1 && ld >= (nq + 2 * nkv) * d && part_stride >= (size_t)rows * ld && ldq >= nq * d,
                 "qkv_from_pieces: %d pieces, row strides %d and %d", splits, ld, ldq);
  LLMLAB_REQUIRE((kcache == nullptr) == (vcache == nullptr), "qkv_from_pieces: need both caches or none");
  LLMLAB_REQUIRE(positions != nullptr && (kcache == nullptr || (table != nullptr && row_req != nullptr && page_size > 0)),
                 "qkv_from_pieces: positions and, for a cache write, a block table are needed");
  if (rows == 0) return 0;
  const int half = d / 2;
  dim3 grid(rows, nq + 2 * nkv), block(half >= 256 ? 256 : (half + 63) / 64 * 64);
  hipLaunchKernelGGL(qkv_from_pieces_kernel, grid, block, 0, stream, parts, splits, part_stride, ld, bias,
                     bias_dtype == DT_BF16, nq, nkv, d, inv_freq, positions, row_req, table, table_stride,
                     page_size, (bf16_t*)kcache, (bf16_t*)vcache, (bf16_t*)q_out, ldq);
  LLMLAB_LAUNCH_CHECK("qkv_from_pieces");
  return 0;
}

// Rotation alone, of x[rows, heads, d] with arbitrary row and head strides.
template <typename T>
__global__ void rope_inplace_kernel(T* __restrict__ x, long row_stride, long head_stride, int d,
                                    const float* __restrict__ inv_freq,
                                    const int* __restrict__ positions) {
  const int r = blockIdx.x, head = blockIdx.y;
  const int pos = positions[r];
  T* base = x + (size_t)r * row_stride + (size_t)head * head_stride;
  const int half = d >> 1;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float lo = to_float(base[i]), hi = to_float(base[i + half]);
    float s, c;
    rope_sincos<T>((float)pos * inv_freq[i], &s, &c);
    base[i] = from_float<T>(lo * c - hi * s);
    base[i + half] = from_float<T>(hi * c + lo * s);
  }
}

extern "C" int llmlab_rope_inplace(void* x, int dtype, int rows, int heads, int d, long row_stride,
                                   long head_stride, const float* inv_freq, const int* positions,
                                   hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && heads > 0 && d > 0 && d % 2 == 0, "rope_inplace: bad sizes");
  if (rows == 0) return 0;
  dim3 grid(rows, heads), block(64);
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(rope_inplace_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)x, row_stride,
                       head_stride, d, inv_freq, positions);
  else
    hipLaunchKernelGGL(rope_inplace_kernel<float>, grid, block, 0, stream, (float*)x, row_stride,
                       head_stride, d, inv_freq, positions);
  LLMLAB_LAUNCH_CHECK("rope_inplace");
  return 0;
}

// ------------------------------------------------------------- token feedback
// dst[dst_index[i]] = src[src_index[i]]: tokens chosen by the previous step go
// straight into this step's input rows without a trip through the host.
__global__ void gather_tokens_kernel(int* __restrict__ dst, const int* __restrict__ dst_index,
                                     const int* __restrict__ src, const int* __restrict__ src_index,
                                     int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[dst_index[i]] = src[src_index[i]];
}

extern "C" int llmlab_gather_tokens(int* dst, const int* dst_index, const int* src, const int* src_index,
                                    int n, hipStream_t stream) {
  LLMLAB_REQUIRE(n >= 0, "gather_tokens: negative count");
  if (n == 0) return 0;
  hipLaunchKernelGGL(gather_tokens_kernel, dim3((n + 63) / 64), dim3(64), 0, stream, dst, dst_index, src,
                     src_index, n);
  LLMLAB_LAUNCH_CHECK("gather_tokens");
  return 0;
}

// ------------------------------------------------------------ weight packing
// A bfloat16 matrix W [N, K] in MFMA fragment order: strips of 16 rows, each strip
// a run of K/32 tiles (K padded to a multiple of 32, N to a multiple of 16, with
// zeros); a tile is the B operand of one v_mfma_f32_16x16x32_bf16, 1 KB, lane l
// (row l % 16 of the strip, columns 8 * (l / 16) .. + 7 of the tile) owning bytes
// 16 l .. 16 l + 15.  Every product kernel reads W in this order, one or two
// contiguous KB per wave instruction, instead of 16 rows of 64 bytes each.
__global__ __launch_bounds__(256) void pack_weight_kernel(const bf16_t* __restrict__ src,
                                                           bf16_t* __restrict__ dst, int N, int K,
                                                           int tiles_per_strip, long chunks) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= chunks) return;
  const long tile = idx >> 6;
  const int l = (int)(idx & 63), c = l & 15, g = l >> 4;
  const int n = (int)(tile / tiles_per_strip) * 16 + c;
  const int k = (int)(tile % tiles_per_strip) * 32 + g * 8;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  *(bf16x8*)(dst + idx * 8) = (n < N && k < K) ? *(const bf16x8*)(src + (size_t)n * K + k) : zero;
}

extern "C" long llmlab_packed_elements(int N, int K) {
  return (long)((N + 15) / 16) * ((K + 31) / 32) * 512;
}

extern "C" int llmlab_pack_weight(const void* src, void* dst, int N, int K, hipStream_t stream) {
  LLMLAB_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "pack_weight: bad sizes N=%d K=%d (K must be a multiple of 8)", N, K);
  LLMLAB_REQUIRE(((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0), "pack_weight: operands must be 16-byte aligned");
  const int tiles = (K + 31) / 32;
  const long chunks = (long)((N + 15) / 16) * tiles * 64;
  hipLaunchKernelGGL(pack_weight_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, stream,
                     (const bf16_t*)src, (bf16_t*)dst, N, K, tiles, chunks);
  LLMLAB_LAUNCH_CHECK("pack_weight");
  return 0;
}

// ------------------------------------------------------------ pending sums
// x[r, :] += sum_s pend[s][r, :], s in order: folds what a product left in pieces
// into the float32 residual stream (for consumers that cannot add it on the fly).
__global__ __launch_bounds__(256) void add_pending_kernel(float* __restrict__ x, const float* __restrict__ pend,
                                                           int splits, size_t stride, long count) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float v = x[i];
  for (int s = 0; s < splits; ++s) v += pend[s * stride + i];
  x[i] = v;
}

extern "C" int llmlab_add_pending(float* x, const float* pend, int splits, size_t stride, int rows,
                                  int width, hipStream_t stream) {
  LLMLAB_REQUIRE(rows >= 0 && width > 0 && splits >= 0 && stride >= (size_t)rows * width,
                 "add_pending: bad sizes rows=%d width=%d splits=%d", rows, width, splits);
  if (rows == 0 || splits == 0) return 0;
  const long count = (long)rows * width;
  hipLaunchKernelGGL(add_pending_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, x, pend,
                     splits, stride, count);
  LLMLAB_LAUNCH_CHECK("add_pending");
  return 0;
}
