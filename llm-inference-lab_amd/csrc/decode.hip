// Matrix products for few rows (M <= 64: decode steps and short portions),
// bfloat16, gfx950.  At this size a step is bound by launch count and by memory
// latency, not by arithmetic, so one kernel does what the general path does in
// three or four:
//
//   [RMSNorm of the float32 residual rows]  ->  x . W^T  ->  K-split reduction
//   ->  epilogue: bias / add into the residual / float32 logits / SwiGLU /
//                 rotary + write of q, and of k and v into their cache pages
//
// A block owns `nsb` strips of 16 weight rows (for the q/k/v projection: exactly one
// head) and splits K over `kw` waves per strip, so blockDim = 64 * nsb * kw.  Every
// wave streams its slice of W from HBM straight into MFMA B fragments with several
// 16-byte loads in flight per lane, multiplies with the A fragments of all rows, and
// leaves its partial sums in LDS; the block adds the partial sums in a fixed order
// (no atomics, results do not depend on timing) and applies the epilogue.
//
// The norm is folded in without a pass of its own:  norm(x) . W^T  =
// inv_rms[m] * ((x * w_norm) . W^T).  The waves read x (float32) anyway to build
// their A fragments, so each also sums the squares of its slice; the block adds
// those and scales the reduced sums by inv_rms[m] in the epilogue.
//
// Fragment layout of v_mfma_f32_16x16x32_bf16 (lane l): A row l%16, B column l%16,
// k = 8*(l/16)..+7; result element i: row 4*(l/16)+i, column l%16.
#include "common.h"

enum { SK_STORE = 0, SK_RESID = 1, SK_F32 = 2, SK_SWIGLU = 3, SK_QKV = 4 };

struct SkinnyArgs {
  const void* x;        // NORM: float32 rows of the residual stream; else bfloat16 [M, K]
  const int* x_rows;    // NORM only, optional: row of x for each m (final norm of wanted rows)
  const void* norm_w;   // NORM: [K]
  const bf16_t* W;      // [N, K]
  const void* bias;     // [N] or null
  void* out;            // STORE/SWIGLU: bf16 [M, ldo]; RESID/F32: float [M, ldo]; QKV: bf16 q [M, ldo]
  // QKV epilogue
  const float* inv_freq;   // [d/2] or null (no rotation)
  const int* positions;    // [M]
  const int* row_req;      // [M]
  const int* table;        // block table
  bf16_t* kcache;          // may be null: q only is produced, k and v heads are skipped
  bf16_t* vcache;
  int M, N, K, ldo, n_out;
  int norm_w_bf16, bias_bf16;
  int nsb, kw;
  int nq, nkv, d, table_stride, page_size;
  float eps;
};

__device__ __forceinline__ float sk_silu(float z) { return z / (1.f + __expf(-z)); }

template <int MB, int EPI, bool NORM>
__global__ __launch_bounds__(MB >= 4 ? 512 : 1024) void skinny_block_kernel(SkinnyArgs a) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr int U = (MB >= 2) ? 2 : 4;   // steps of 32 in flight
  const int nsb = a.nsb, kw = a.kw;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int strip = wave % nsb, ks = wave / nsb;
  const int c = lane & 15, g = lane >> 4;
  const int cols = 16 * nsb;
  const int n0 = blockIdx.x * cols;
  const int K = a.K, M = a.M;
  // LDS: partial sums, then sums of squares, inverse rms, and the output tile
  float* part = smem;                                   // [kw*nsb][MB][64][4]
  float* ss_part = part + (size_t)kw * nsb * MB * 256;  // [kw][MB*16]
  float* inv = ss_part + kw * MB * 16;                  // [MB*16]
  float* tile = inv + MB * 16;                          // [M][cols]   (SWIGLU, QKV)

  const int n = n0 + strip * 16 + c;
  const bool wok = n < a.N;
  const bf16_t* wrow = a.W + (size_t)(wok ? n : 0) * K;
  const int steps = (K + 31) >> 5;
  const int per = (steps + kw - 1) / kw;
  const int s_begin = ks * per;
  const int s_end = min(steps, s_begin + per);
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  floatx4 acc[MB];
  float ss[MB];
  const float* xf[MB];
  const bf16_t* xb[MB];
  bool aok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    ss[mb] = 0.f;
    const int m = mb * 16 + c;
    aok[mb] = m < M;
    const size_t row = aok[mb] ? (size_t)((NORM && a.x_rows) ? a.x_rows[m] : m) : 0;
    xf[mb] = (const float*)a.x + row * K;
    xb[mb] = (const bf16_t*)a.x + row * K;
  }

  for (int s0 = s_begin; s0 < s_end; s0 += U) {
    bf16x8 b[U];
    floatx4 x0[U][MB], x1[U][MB];
    bf16x8 ab[U][MB];
    floatx4 w0[U], w1[U];
    bf16x8 wb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = (s0 + u) * 32 + g * 8;
      const bool kok = (s0 + u) < s_end && kk < K;
      b[u] = (wok && kok) ? *(const bf16x8*)(wrow + kk) : zero;
      if constexpr (NORM) {
        if (a.norm_w_bf16) {
          wb[u] = kok ? *(const bf16x8*)((const bf16_t*)a.norm_w + kk) : zero;
        } else {
          w0[u] = kok ? *(const floatx4*)((const float*)a.norm_w + kk) : floatx4{0.f, 0.f, 0.f, 0.f};
          w1[u] = kok ? *(const floatx4*)((const float*)a.norm_w + kk + 4) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const bool ok = aok[mb] && kok;
          x0[u][mb] = ok ? *(const floatx4*)(xf[mb] + kk) : floatx4{0.f, 0.f, 0.f, 0.f};
          x1[u][mb] = ok ? *(const floatx4*)(xf[mb] + kk + 4) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
      } else {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          ab[u][mb] = (aok[mb] && kok) ? *(const bf16x8*)(xb[mb] + kk) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        bf16x8 av;
        if constexpr (NORM) {
          float wv[8];
          if (a.norm_w_bf16) {
#pragma unroll
            for (int j = 0; j < 8; ++j) wv[j] = (float)wb[u][j];
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              wv[j] = w0[u][j];
              wv[4 + j] = w1[u][j];
            }
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float p = x0[u][mb][j], q = x1[u][mb][j];
            ss[mb] += p * p + q * q;
            av[j] = (bf16_t)(p * wv[j]);
            av[4 + j] = (bf16_t)(q * wv[4 + j]);
          }
        } else {
          av = ab[u][mb];
        }
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, b[u], acc[mb], 0, 0, 0);
      }
    }
  }

  // partial sums to LDS
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
    *(floatx4*)(part + (((size_t)wave * MB + mb) * 64 + lane) * 4) = acc[mb];
  if constexpr (NORM) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      float v = ss[mb];
      v += __shfl_xor(v, 16, WAVE);
      v += __shfl_xor(v, 32, WAVE);
      if (strip == 0 && g == 0) ss_part[(ks * MB + mb) * 16 + c] = v;
    }
  }
  __syncthreads();
  if constexpr (NORM) {
    if ((int)threadIdx.x < MB * 16) {
      const int mb = threadIdx.x >> 4, cc = threadIdx.x & 15;
      float t = 0.f;
      for (int k2 = 0; k2 < kw; ++k2) t += ss_part[(k2 * MB + mb) * 16 + cc];
      inv[threadIdx.x] = rsqrtf(t / (float)K + a.eps);
    }
    __syncthreads();
  }

  // reduce over the K slices in a fixed order; epilogue
  for (int idx = threadIdx.x; idx < M * cols; idx += blockDim.x) {
    const int m = idx / cols, col = idx - m * cols;
    const int st = col >> 4, cc = col & 15;
    const int mb = m >> 4, gg = (m & 15) >> 2, xx = m & 3;
    float sum = 0.f;
    for (int k2 = 0; k2 < kw; ++k2)
      sum += part[((((size_t)k2 * nsb + st) * MB + mb) * 64 + gg * 16 + cc) * 4 + xx];
    if constexpr (NORM) sum *= inv[m];
    const int nn = n0 + col;
    if (nn < a.N && a.bias) sum += load_vec(a.bias, a.bias_bf16, nn);
    if constexpr (EPI == SK_SWIGLU || EPI == SK_QKV) {
      tile[idx] = sum;
    } else if (nn < a.N) {
      const size_t at = (size_t)m * a.ldo + nn;
      if (EPI == SK_STORE) ((bf16_t*)a.out)[at] = (bf16_t)sum;
      else if (EPI == SK_RESID) ((float*)a.out)[at] += sum;
      else ((float*)a.out)[at] = sum;
    }
  }
  if constexpr (EPI == SK_SWIGLU) {
    __syncthreads();
    const int half = cols >> 1;   // outputs of this block
    for (int idx = threadIdx.x; idx < M * half; idx += blockDim.x) {
      const int m = idx / half, j = idx - m * half;
      const int pr = j >> 4, cc = j & 15;
      const float gv = tile[m * cols + pr * 32 + cc], uv = tile[m * cols + pr * 32 + 16 + cc];
      const int o = ((n0 >> 5) + pr) * 16 + cc;
      if (o < a.n_out) ((bf16_t*)a.out)[(size_t)m * a.ldo + o] = (bf16_t)(sk_silu(gv) * uv);
    }
  }
  if constexpr (EPI == SK_QKV) {
    __syncthreads();
    // this block is head `blockIdx.x` of [q heads | k heads | v heads]
    const int head = blockIdx.x, d = a.d, half = d >> 1;
    const bool is_q = head < a.nq, is_k = !is_q && head < a.nq + a.nkv;
    for (int idx = threadIdx.x; idx < M * half; idx += blockDim.x) {
      const int m = idx / half, i = idx - m * half;
      float lo = tile[m * cols + i], hi = tile[m * cols + i + half];
      const int pos = a.positions[m];
      if ((is_q || is_k) && a.inv_freq) {
        float s, co;
        sincosf((float)pos * a.inv_freq[i], &s, &co);
        const float nlo = lo * co - hi * s, nhi = hi * co + lo * s;
        lo = nlo;
        hi = nhi;
      }
      if (is_q) {
        bf16_t* dst = (bf16_t*)a.out + (size_t)m * a.ldo + (size_t)head * d;
        dst[i] = (bf16_t)lo;
        dst[i + half] = (bf16_t)hi;
      } else if (a.kcache) {
        const size_t page = (size_t)a.table[(size_t)a.row_req[m] * a.table_stride + pos / a.page_size];
        const int off = pos % a.page_size;
        if (is_k) {
          bf16_t* dst = a.kcache + ((page * a.nkv + (head - a.nq)) * a.page_size + off) * (size_t)d;
          dst[i] = (bf16_t)lo;
          dst[i + half] = (bf16_t)hi;
        } else {
          bf16_t* dst = a.vcache + ((page * a.nkv + (head - a.nq - a.nkv)) * (size_t)d) * a.page_size + off;
          dst[(size_t)i * a.page_size] = (bf16_t)lo;
          dst[(size_t)(i + half) * a.page_size] = (bf16_t)hi;
        }
      }
    }
  }
}

// ---------------------------------------------------------------- dispatch
static size_t skinny_lds_bytes(int nsb, int kw, int mb, int M, int epi) {
  size_t floats = (size_t)kw * nsb * mb * 256 + (size_t)kw * mb * 16 + (size_t)mb * 16;
  if (epi == SK_SWIGLU || epi == SK_QKV) floats += (size_t)M * 16 * nsb;
  return floats * sizeof(float);
}

template <int MB, int EPI, bool NORM>
static void skinny_launch(const SkinnyArgs& a, int blocks, size_t lds, hipStream_t stream) {
  hipLaunchKernelGGL((skinny_block_kernel<MB, EPI, NORM>), dim3(blocks), dim3(64 * a.nsb * a.kw), lds,
                     stream, a);
}

template <int EPI, bool NORM>
static void skinny_launch_mb(const SkinnyArgs& a, int mb, int blocks, size_t lds, hipStream_t stream) {
  if (mb == 1) skinny_launch<1, EPI, NORM>(a, blocks, lds, stream);
  else if (mb == 2) skinny_launch<2, EPI, NORM>(a, blocks, lds, stream);
  else skinny_launch<4, EPI, NORM>(a, blocks, lds, stream);
}

// One entry point for the whole family.
//   norm != 0: x is the float32 residual stream (rows x_rows[m] or m), norm_w/eps its RMSNorm
//   epilogue SK_QKV: N = (nq + 2 nkv) * d, one block per head, `out` is q [M, ldo]
extern "C" int llmlab_skinny_linear(const void* x, int norm, const int* x_rows, const void* norm_w,
                                    int norm_w_dtype, float eps, const void* w, const void* bias,
                                    int bias_dtype, int epilogue, void* out, int M, int N, int K,
                                    int ldo, int n_out, const float* inv_freq, const int* positions,
                                    const int* row_req, const int* table, int table_stride,
                                    int page_size, void* kcache, void* vcache, int nq, int nkv, int d,
                                    int num_cus, hipStream_t stream) {
  LLMLAB_REQUIRE(M >= 0 && M <= 64, "skinny_linear: takes at most 64 rows, got %d", M);
  LLMLAB_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "skinny_linear: bad sizes N=%d K=%d (K must be a multiple of 8)", N, K);
  LLMLAB_REQUIRE(epilogue >= 0 && epilogue <= 4, "skinny_linear: unknown epilogue %d", epilogue);
  LLMLAB_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
                 (norm_w == nullptr || (uintptr_t)norm_w % 16 == 0),
                 "skinny_linear: operands must be 16-byte aligned");
  if (M == 0) return 0;
  if (num_cus <= 0) num_cus = 256;
  const int mb = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int steps = (K + 31) / 32;
  int nsb;
  if (epilogue == SK_QKV) {
    LLMLAB_REQUIRE(d >= 16 && d % 16 == 0 && d <= 256 && N == (nq + 2 * nkv) * d,
                   "skinny_linear(qkv): head size %d / %d rows do not fit", d, N);
    LLMLAB_REQUIRE((kcache == nullptr) == (vcache == nullptr), "skinny_linear(qkv): both caches or none");
    LLMLAB_REQUIRE(positions != nullptr && (kcache == nullptr || (table && row_req && page_size > 0)),
                   "skinny_linear(qkv): positions and block table are needed");
    nsb = d / 16;
  } else if (epilogue == SK_SWIGLU) {
    LLMLAB_REQUIRE(N % 32 == 0 && 2 * ((n_out + 15) / 16 * 16) == N && bias == nullptr,
                   "skinny_linear(swiglu): %d rows do not interleave %d outputs", N, n_out);
    nsb = 2;
  } else {
    LLMLAB_REQUIRE(n_out == N, "skinny_linear: n_out %d != N %d", n_out, N);
    nsb = (N >= 32 * 2 * num_cus) ? 2 : 1;
  }
  LLMLAB_REQUIRE(ldo >= (epilogue == SK_QKV ? nq * d : n_out), "skinny_linear: output stride too small");
  const int cols = 16 * nsb;
  const int blocks = (N + cols - 1) / cols;
  // enough waves to have the whole matrix in flight, within the block and LDS limits
  const long want_waves = 12L * num_cus;
  int kw = (int)((want_waves + (long)blocks * nsb - 1) / ((long)blocks * nsb));
  if (kw > 16 / nsb) kw = 16 / nsb;
  if (kw > steps) kw = steps;
  while (kw > 1 && nsb * kw * mb > 32) --kw;
  if (kw < 1) kw = 1;
  const size_t lds = skinny_lds_bytes(nsb, kw, mb, M, epilogue);
  LLMLAB_REQUIRE(lds <= 64 * 1024, "skinny_linear: %zu bytes of LDS needed", lds);
  SkinnyArgs a;
  a.x = x; a.x_rows = x_rows; a.norm_w = norm_w; a.W = (const bf16_t*)w; a.bias = bias; a.out = out;
  a.inv_freq = inv_freq; a.positions = positions; a.row_req = row_req; a.table = table;
  a.kcache = (bf16_t*)kcache; a.vcache = (bf16_t*)vcache;
  a.M = M; a.N = N; a.K = K; a.ldo = ldo; a.n_out = n_out;
  a.norm_w_bf16 = norm_w_dtype == DT_BF16; a.bias_bf16 = bias_dtype == DT_BF16;
  a.nsb = nsb; a.kw = kw; a.nq = nq; a.nkv = nkv; a.d = d; a.table_stride = table_stride;
  a.page_size = page_size; a.eps = eps;
#define SK_CASE(E)                                                          \
  case E:                                                                   \
    if (norm) skinny_launch_mb<E, true>(a, mb, blocks, lds, stream);        \
    else skinny_launch_mb<E, false>(a, mb, blocks, lds, stream);            \
    break;
  switch (epilogue) {
    SK_CASE(SK_STORE)
    SK_CASE(SK_RESID)
    SK_CASE(SK_F32)
    SK_CASE(SK_SWIGLU)
    SK_CASE(SK_QKV)
  }
#undef SK_CASE
  LLMLAB_LAUNCH_CHECK("skinny_linear");
  return 0;
}
