// Matrix products for few rows (decode steps and short portions; up to 1,024 rows of
// a small matrix, in tiles of 16 to 64 rows), bfloat16, gfx950.  At this size a step is bound by launch count and by memory
// latency, not by arithmetic, so one kernel does what the general path does in
// three or four:
//
//   [RMSNorm of the float32 residual rows]  ->  x . W^T  ->  K-split reduction
//   ->  epilogue: bias / add into the residual / float32 logits / SwiGLU /
//                 rotary + write of q, and of k and v into their cache pages
//
// W comes packed in MFMA fragment order (see llmlab_pack_weight): the 16 rows x 32
// columns a wave multiplies in one step are 1 KB of consecutive memory, lane l
// owning bytes 16 l .. 16 l + 15, and the steps of a strip follow each other.  A
// wave therefore streams one contiguous run of memory with full cache lines,
// which at these sizes is worth a factor of two over rows of 64 bytes each.
//
// A block owns `nsb` strips of 16 weight rows (for the q/k/v projection: one head,
// or two strips of one) and splits K over `kw` waves per strip, so blockDim =
// 64 * nsb * kw.  Every wave streams its slice of W from HBM straight into MFMA B
// fragments through a ring of registers, and leaves its partial sums in LDS; the
// block adds the partial sums in a fixed order (no atomics, results do not depend
// on timing) and applies the epilogue.
//
// The rows of x are staged once per block in LDS as bfloat16 (STAGE), so the strips
// of a block share them; or every wave reads its slice from global memory (plain
// products only).  The norm is folded in without a pass of its own:
//   norm(x) . W^T = inv_rms[m] * ((x * w_norm) . W^T)
// x * w_norm is what is staged (or built on the fly), the sum of squares falls out
// of the same read, and inv_rms[m] scales the reduced sums in the epilogue.
//
// What the epilogue needs from global memory (bias, positions, page numbers,
// rotary frequencies, the residual value it adds to) is fetched at the start of the
// kernel, so those latencies overlap the weight stream instead of following it.
//
// A compute unit draws only about 50 GB/s from HBM, so a product with a narrow
// output (few strips, hence few blocks) is bound by the units it uses, not by the
// chip.  Epilogue SK_PART cuts such a product along K over `ksplit` groups of blocks
// as well and leaves one piece of the result per group, unsummed: no second kernel
// and no atomics.  The pieces are owed to the float32 rows they would have been
// added to; the next kernel that reads those rows (under a fused norm) adds them on
// the fly in their order, and the next SK_RESID product into those rows folds them
// in for good (`pend` below).
//
// More than 16 rows are cut into tiles of 16 MB rows (MB = 1, 2 or 4) that separate
// blocks take: a block then stages, norms and multiplies its own rows only, and
// four times the blocks hide each other's latencies.  The tiles of one set of
// columns read the same part of W; their block numbers are equal modulo 8 and
// adjacent there, so that they run on one XCD at about the same time and all but
// the first find W in its L2.  Measured at 64 rows of the 0.5B shapes, tiles of 16
// rows against one tile of 64: q/k/v 5.2 against 9.8 us, output product 4.3
// against 7.7, down product 8.7 against 21.8.
//
// Fragment layout of v_mfma_f32_16x16x32_bf16 (lane l): A row l%16, B column l%16,
// k = 8*(l/16)..+7; result element i: row 4*(l/16)+i, column l%16.
#include <stdlib.h>

#include <type_traits>

#include "common.h"

enum { SK_STORE = 0, SK_RESID = 1, SK_F32 = 2, SK_SWIGLU = 3, SK_QKV = 4, SK_PART = 5 };

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
  int qsplit;   // QKV: blocks per head (1, or d/32: a block then owns the strips p and p + d/32)
  int nq, nkv, d, table_stride, page_size;
  float eps;
  // Sums that a former product left in pieces (SK_PART) and that still belong to the
  // float32 rows this kernel reads (NORM) or adds into (RESID): pend[s][row][pend_ld],
  // s < pend_splits, added in the order of s.
  const float* pend;
  int pend_splits, pend_ld;
  size_t pend_stride;
  // SK_PART: K is split over `ksplit` groups of blocks as well; group s leaves its sums
  // (no residual, bias in group 0) in out[s][M][ldo], part_stride numbers apart.
  int ksplit;
  size_t part_stride;
  int tiles;       // tiles of 16 MB rows
  int col_blocks;  // blocks that a tile of rows takes (sets of columns, times ksplit)
};

__device__ __forceinline__ float sk_silu(float z) { return z / (1.f + __expf(-z)); }

// Loads of W (and of x where it is not staged) run R steps ahead of the MFMAs in a
// ring of registers that is refilled slot by slot, so a wave always has R loads
// in flight and never waits for all of them at once.  Measured per decode step, staged
// ring 4 / 6 / 8 / 12 / 16 deep: one request of the 7B shape 3.21 / 3.13 / 3.07 / 3.34 /
// 3.76 ms, eight of the 32B shape 15.83 / 15.66 / 15.61 / 15.96 / 16.96, eight of the
// 0.5B shape 0.963 / 0.976 / 0.962 / 1.010 / 1.162 (a block of 16 waves has 128
// registers a lane; a wave with fewer steps than the ring is deep reads its last tile
// again for nothing); the ring of the unstaged products 4 / 6 / 8 deep: 15.61 / 15.52 /
// 15.51 and 0.965 / 0.959 / 0.971.
constexpr int SK_RING_STAGE = 8, SK_RING_DIRECT = 6;
__host__ __device__ constexpr int sk_ring(int mb, bool stage) {
  return stage ? SK_RING_STAGE : (mb >= 4 ? SK_RING_DIRECT / 2 : SK_RING_DIRECT);
}

constexpr int SK_STAGE_U_PIECES = 1;
constexpr int SK_APAD = 8;   // padding of a staged row, in elements: 16-byte reads of 8 lanes cover all banks

// floats of LDS before the staged rows (host and device must agree)
__host__ __device__ inline size_t sk_float_words(int nsb, int kw, int mb, int M, int epi) {
  size_t f = (size_t)kw * nsb * mb * 256;        // partial sums
  f += (size_t)mb * 16 + 16;                      // inverse rms; sums of squares of the parts of a row
  f += (size_t)16 * nsb;                          // bias
  f += (size_t)mb * 16 * 2 + 128;                 // positions, pages, frequencies
  if (epi == SK_SWIGLU || epi == SK_QKV) f += (size_t)M * 16 * nsb;
  return (f + 3) & ~(size_t)3;
}

template <int MB, int EPI, bool NORM, bool STAGE>
__global__ __launch_bounds__(MB >= 4 ? 512 : 1024) void skinny_block_kernel(SkinnyArgs a) {
  static_assert(STAGE || !NORM, "the fused norm needs the staged rows");
  extern __shared__ __attribute__((aligned(16))) float smem[];
  // Rows in tiles of 16 MB: a block sees its tile as if it were the whole product,
  // through pointers moved to the tile's first row.  The tiles of one set of columns
  // read the same part of W: they get block numbers that are equal modulo 8 (the
  // same XCD, hence the same L2) and follow each other there.
  int col_block = (int)blockIdx.x;
  if (a.tiles > 1) {
    const int xcd = (int)blockIdx.x & 7, j = (int)blockIdx.x >> 3;
    const int tile = j % a.tiles;
    col_block = (j / a.tiles) * 8 + xcd;
    if (col_block >= a.col_blocks) return;      // (the grid is rounded up to whole eights)
    const int m0 = tile * (MB * 16);
    a.M = min(MB * 16, a.M - m0);
    if (NORM && a.x_rows) a.x_rows += m0;       // (the pieces owed are then found by these numbers too)
    else {
      a.x = NORM ? (const void*)((const float*)a.x + (size_t)m0 * a.K)
                 : (const void*)((const bf16_t*)a.x + (size_t)m0 * a.K);
      a.pend += (size_t)m0 * a.pend_ld;
    }
    constexpr bool OUT32 = EPI == SK_RESID || EPI == SK_F32 || EPI == SK_PART;
    a.out = OUT32 ? (void*)((float*)a.out + (size_t)m0 * a.ldo) : (void*)((bf16_t*)a.out + (size_t)m0 * a.ldo);
    if constexpr (EPI == SK_QKV) {
      a.positions += m0;
      if (a.row_req) a.row_req += m0;
    }
  }
  constexpr int R = sk_ring(MB, STAGE);   // K steps whose loads a wave keeps in flight
  const int nsb = a.nsb, kw = a.kw;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int strip = wave % nsb, ks = wave / nsb;
  const int c = lane & 15, g = lane >> 4;
  const int cols = 16 * nsb;
  // SK_PART: the blocks of one K group follow each other
  const int nblk = (EPI == SK_PART) ? a.col_blocks / a.ksplit : a.col_blocks;
  const int ksp = (EPI == SK_PART) ? col_block / nblk : 0;
  const int bidx = (EPI == SK_PART) ? col_block - ksp * nblk : col_block;
  const int n0 = bidx * cols;
  const int K = a.K, M = a.M;
  const int steps = (K + 31) >> 5;      // K steps of 32; W is packed and zero-padded to this

  float* part = smem;                                   // [kw*nsb][MB][64][4]
  float* inv = part + (size_t)kw * nsb * MB * 256;      // [MB*16]
  float* s_ssq = inv + MB * 16;                         // [16]: a row's sum of squares, by the waves that share it
  float* s_bias = s_ssq + 16;                           // [cols]
  int* s_pos = (int*)(s_bias + cols);                   // [MB*16]
  int* s_page = s_pos + MB * 16;                        // [MB*16]
  float* s_freq = (float*)(s_page + MB * 16);           // [128]
  float* tile = s_freq + 128;                           // [M][cols]   (SWIGLU, QKV)
  bf16_t* As = (bf16_t*)(smem + sk_float_words(nsb, kw, MB, M, EPI));   // [M][steps*32 + SK_APAD]
  const int lda = steps * 32 + SK_APAD;

  // QKV with qsplit > 1: block = (head, p); its two strips are columns p*16.. and
  // d/2 + p*16.. of the head, i.e. both halves of the rotary pairs
  int qhead = 0, qp = 0;
  if constexpr (EPI == SK_QKV) {
    qhead = bidx / a.qsplit;
    qp = bidx - qhead * a.qsplit;
  }
  auto head_col = [&](int col) {   // column of the block -> column of the head
    if (a.qsplit == 1) return col;
    return col < 16 ? qp * 16 + col : (a.d >> 1) + qp * 16 + (col - 16);
  };
  // the strip of 16 weight rows this wave multiplies (past the last one: the last
  // one again, and what comes of it is dropped by the epilogue)
  int wstrip = (EPI == SK_QKV) ? (qhead * a.d + head_col(strip * 16)) >> 4 : bidx * nsb + strip;
  wstrip = min(wstrip, ((a.N + 15) >> 4) - 1);
  const bf16_t* wp = a.W + (size_t)wstrip * steps * 512 + lane * 8;
  // this block's K steps (all of them, or its group's share), split over its waves
  const int gsteps = (EPI == SK_PART) ? (steps + a.ksplit - 1) / a.ksplit : steps;
  const int g_begin = ksp * gsteps, g_end = min(steps, g_begin + gsteps);
  const int per = (max(g_end - g_begin, 0) + kw - 1) / kw;
  const int s_begin = g_begin + ks * per;
  const int s_end = min(g_end, s_begin + per);
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const floatx4 fzero = {0.f, 0.f, 0.f, 0.f};

  // ---- what the epilogue needs from global memory, fetched now
  for (int i = threadIdx.x; i < cols; i += blockDim.x) {
    const int nn = (EPI == SK_QKV) ? qhead * a.d + head_col(i) : n0 + i;
    s_bias[i] = (a.bias && nn < a.N && ksp == 0) ? load_vec(a.bias, a.bias_bf16, nn) : 0.f;
  }
  if constexpr (EPI == SK_QKV) {
    const int head = qhead;
    for (int m = threadIdx.x; m < M; m += blockDim.x) {
      const int pos = a.positions[m];
      s_pos[m] = pos;
      s_page[m] = (a.kcache && head >= a.nq)
                      ? a.table[(size_t)a.row_req[m] * a.table_stride + pos / a.page_size] : 0;
    }
    for (int i = threadIdx.x; i < (a.d >> 1); i += blockDim.x)
      s_freq[i] = a.inv_freq ? a.inv_freq[i] : 0.f;
  }

  // the residual value this thread will add to (its first one): on its way now, not
  // after the reduction
  float resid_old = 0.f;
  if constexpr (EPI == SK_RESID) {
    const int idx = threadIdx.x;
    const int m = idx / cols, nn = n0 + idx - m * cols;
    if (idx < M * cols && nn < a.N) {
      resid_old = ((const float*)a.out)[(size_t)m * a.ldo + nn];
      for (int sp0 = 0; sp0 < a.pend_splits; sp0 += 4) {      // four pieces at a time, as above
        float pp[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
          pp[j] = a.pend[min(sp0 + j, a.pend_splits - 1) * a.pend_stride + (size_t)m * a.pend_ld + nn];
#pragma unroll
        for (int j = 0; j < 4; ++j) resid_old += sp0 + j < a.pend_splits ? pp[j] : 0.f;
      }
    }
  }

  floatx4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = fzero;

  // Loads in the ring are unconditional (a step past the end reads the last tile
  // again and is multiplied by zeros): a load under a branch makes the compiler wait
  // for every load in flight at the join, and the stream stalls once per round.
  auto wload = [&](int st) { return *(const bf16x8*)(wp + (size_t)max(0, min(st, steps - 1)) * 512); };
  bf16x8 b[R];

  if constexpr (STAGE) {
#pragma unroll
    for (int u = 0; u < R; ++u) b[u] = wload(min(s_begin + u, s_end - 1));
    // ---- the first weight tiles are on their way; stage the rows of x
    // Fewer rows than waves: `wpr` waves share a row, each taking every wpr-th run of 64
    // chunks (one wave alone would walk a long row in many trips while the others wait)
    const int chunks = K >> 3, chunks_pad = steps * 4;
    int wpr = 1;
    while (2 * wpr * M <= nwaves) wpr *= 2;
    // A wave walks its part of a row U chunks at a time: the loads of all U (the row, the
    // norm's weight, the pieces owed) are on their way before the first is used, so a part
    // costs one trip to memory per U chunks and not one per chunk.  Loads are unconditional
    // (a chunk past the end reads the last one again and is not stored).
    auto stage_rows = [&](auto u_tag, auto w_tag) {
      constexpr int U = decltype(u_tag)::value;
      constexpr bool W_BF16 = decltype(w_tag)::value;     // (the norm's weight: no branch among the loads)
      const int stride = 64 * wpr;
      for (int unit = wave; unit < M * wpr; unit += nwaves) {
        const int r = unit / wpr, sub = unit - r * wpr;
        bf16_t* dst = As + (size_t)r * lda;
        if constexpr (NORM) {
          const float* src = (const float*)a.x + (size_t)(a.x_rows ? a.x_rows[r] : r) * K;
          float ssq = 0.f;
          const size_t prow = (size_t)(a.x_rows ? a.x_rows[r] : r) * a.pend_ld;
          for (int ch0 = sub * 64 + lane; ch0 < chunks; ch0 += U * stride) {
            floatx4 p[U], q[U], w0[U], w1[U];
            bf16x8 w8[U];
            int chs[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
              chs[u] = min(ch0 + u * stride, chunks - 1);
              p[u] = *(const floatx4*)(src + chs[u] * 8);
              q[u] = *(const floatx4*)(src + chs[u] * 8 + 4);
              if constexpr (W_BF16) {
                w8[u] = *(const bf16x8*)((const bf16_t*)a.norm_w + chs[u] * 8);
              } else {
                w0[u] = *(const floatx4*)((const float*)a.norm_w + chs[u] * 8);
                w1[u] = *(const floatx4*)((const float*)a.norm_w + chs[u] * 8 + 4);
              }
            }
            // sums still owed to these rows: four pieces at a time for every chunk, loads
            // unconditional (past the last piece: the last one again, not added)
            for (int sp0 = 0; sp0 < a.pend_splits; sp0 += 4) {
              floatx4 pp[U][4], qq[U][4];
#pragma unroll
              for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  const float* src2 = a.pend + min(sp0 + j, a.pend_splits - 1) * a.pend_stride + prow + chs[u] * 8;
                  pp[u][j] = *(const floatx4*)src2;
                  qq[u][j] = *(const floatx4*)(src2 + 4);
                }
#pragma unroll
              for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  const float on = sp0 + j < a.pend_splits ? 1.f : 0.f;
                  p[u] += pp[u][j] * on;
                  q[u] += qq[u][j] * on;
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
              if (ch0 + u * stride >= chunks) break;
              float wv[8];
              if constexpr (W_BF16) {
#pragma unroll
                for (int j = 0; j < 8; ++j) wv[j] = (float)w8[u][j];
              } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  wv[j] = w0[u][j];
                  wv[4 + j] = w1[u][j];
                }
              }
              bf16x8 av;
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                ssq += p[u][j] * p[u][j] + q[u][j] * q[u][j];
                av[j] = (bf16_t)(p[u][j] * wv[j]);
                av[4 + j] = (bf16_t)(q[u][j] * wv[4 + j]);
              }
              *(bf16x8*)(dst + chs[u] * 8) = av;
            }
          }
          ssq = wave_sum(ssq);
          if (lane == 0) {
            if (wpr == 1) inv[r] = rsqrtf(ssq / (float)K + a.eps);
            else s_ssq[unit] = ssq;       // (M * wpr <= 16 waves)
          }
        } else {
          const bf16_t* src = (const bf16_t*)a.x + (size_t)r * K;
          for (int ch0 = sub * 64 + lane; ch0 < chunks; ch0 += U * stride) {
            bf16x8 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = *(const bf16x8*)(src + min(ch0 + u * stride, chunks - 1) * 8);
#pragma unroll
            for (int u = 0; u < U; ++u)
              if (ch0 + u * stride < chunks) *(bf16x8*)(dst + (ch0 + u * stride) * 8) = v[u];
          }
        }
        if (sub == 0)
          for (int ch = chunks + lane; ch < chunks_pad; ch += 64) *(bf16x8*)(dst + ch * 8) = zero;
      }
    };
    // (with pieces owed, two chunks' loads are as many registers as four without)
    using two = std::integral_constant<int, SK_STAGE_U_PIECES>;
    using four = std::integral_constant<int, 4>;
    if (NORM && a.pend_splits > 0) {
      if (a.norm_w_bf16) stage_rows(two{}, std::true_type{});
      else stage_rows(two{}, std::false_type{});
    } else if (NORM && !a.norm_w_bf16) {
      stage_rows(four{}, std::false_type{});
    } else {
      stage_rows(four{}, std::true_type{});
    }
    __syncthreads();
    if constexpr (NORM) {
      // the parts of a row in their order (read by the epilogue, behind the next barrier)
      if (wpr > 1 && (int)threadIdx.x < M) {
        float total = 0.f;
        for (int sub = 0; sub < wpr; ++sub) total += s_ssq[threadIdx.x * wpr + sub];
        inv[threadIdx.x] = rsqrtf(total / (float)K + a.eps);
      }
    }
    // rows past M are not staged: their lanes read the last row, and what they
    // compute lands in rows of the result that nobody reads
    const bf16_t* arow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) arow[mb] = As + (size_t)min(mb * 16 + c, M - 1) * lda + g * 8;
    int s0 = s_begin;
    for (; s0 + R < s_end; s0 += R) {       // rounds that refill the ring
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const int st = s0 + u;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const bf16x8 av = *(const bf16x8*)(arow[mb] + st * 32);
          acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, b[u], acc[mb], 0, 0, 0);
        }
        b[u] = wload(min(st + R, s_end - 1));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {           // the last round drains it
      const int st = s0 + u;
      const bf16x8 bu = st < s_end ? b[u] : zero;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const bf16x8 av = *(const bf16x8*)(arow[mb] + min(st, steps - 1) * 32);
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bu, acc[mb], 0, 0, 0);
      }
    }
  } else {
    // ---- rows of x (bfloat16) straight from global memory, in the same ring; a
    // piece past K or a row past M reads a valid piece instead: it meets zeros of
    // the padded W, or lands in a row of the result that nobody reads
    const bf16_t* xb[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xb[mb] = (const bf16_t*)a.x + (size_t)min(mb * 16 + c, M - 1) * K;
    auto xload = [&](int st, int mb) {
      return *(const bf16x8*)(xb[mb] + min(max(0, min(st, steps - 1)) * 32 + g * 8, K - 8));
    };
    bf16x8 ab[R][MB];
#pragma unroll
    for (int u = 0; u < R; ++u) {     // in the order in which the loop below refills the ring
      const int st = min(s_begin + u, s_end - 1);
      b[u] = wload(st);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) ab[u][mb] = xload(st, mb);
      __builtin_amdgcn_sched_barrier(0);
    }
    int s0 = s_begin;
    for (; s0 + R < s_end; s0 += R) {       // rounds that refill the ring
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const int st = s0 + u;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ab[u][mb], b[u], acc[mb], 0, 0, 0);
        const int nx = min(st + R, s_end - 1);
        b[u] = wload(nx);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) ab[u][mb] = xload(nx, mb);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {           // the last round drains it
      const bf16x8 bu = s0 + u < s_end ? b[u] : zero;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ab[u][mb], bu, acc[mb], 0, 0, 0);
    }
  }

  // ---- partial sums to LDS
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
    *(floatx4*)(part + (((size_t)wave * MB + mb) * 64 + lane) * 4) = acc[mb];
  __syncthreads();
  // ---- reduce over the K slices in a fixed order; epilogue
  for (int idx = threadIdx.x; idx < M * cols; idx += blockDim.x) {
    const int m = idx / cols, col = idx - m * cols;
    const int st = col >> 4, cc = col & 15;
    const int mb = m >> 4, gg = (m & 15) >> 2, xx = m & 3;
    float sum = 0.f;
    for (int k2 = 0; k2 < kw; ++k2)
      sum += part[((((size_t)k2 * nsb + st) * MB + mb) * 64 + gg * 16 + cc) * 4 + xx];
    if constexpr (NORM) sum *= inv[m];
    sum += s_bias[col];
    const int nn = n0 + col;
    if constexpr (EPI == SK_SWIGLU || EPI == SK_QKV) {
      tile[idx] = sum;
    } else if (nn < a.N) {
      const size_t at = (size_t)m * a.ldo + nn;
      if (EPI == SK_STORE) ((bf16_t*)a.out)[at] = (bf16_t)sum;
      else if (EPI == SK_RESID) {
        float old = resid_old;
        if (idx != (int)threadIdx.x) {
          old = ((float*)a.out)[at];
          for (int sp = 0; sp < a.pend_splits; ++sp) old += a.pend[sp * a.pend_stride + (size_t)m * a.pend_ld + nn];
        }
        ((float*)a.out)[at] = old + sum;
      } else if (EPI == SK_PART) {
        ((float*)a.out)[ksp * a.part_stride + at] = sum;
      } else {
        ((float*)a.out)[at] = sum;
      }
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
    // this block is (part of) head `qhead` of [q heads | k heads | v heads]; its tile
    // holds the low halves of its rotary pairs in the first half of its columns
    const int head = qhead, d = a.d, dhalf = d >> 1, half = cols >> 1;
    const int i0 = a.qsplit == 1 ? 0 : qp * 16;
    const bool is_q = head < a.nq, is_k = !is_q && head < a.nq + a.nkv;
    for (int idx = threadIdx.x; idx < M * half; idx += blockDim.x) {
      const int m = idx / half, il = idx - m * half;
      const int i = i0 + il;                      // pair index within the head
      float lo = tile[m * cols + il], hi = tile[m * cols + il + half];
      const int pos = s_pos[m];
      if ((is_q || is_k) && a.inv_freq) {
        // bfloat16 results: the hardware sine and cosine of r = frac(angle / 2 pi)
        float r = (float)pos * s_freq[i] * 0.15915494309189535f;
        r -= floorf(r);
        const float s = __builtin_amdgcn_sinf(r), co = __builtin_amdgcn_cosf(r);
        const float nlo = lo * co - hi * s, nhi = hi * co + lo * s;
        lo = nlo;
        hi = nhi;
      }
      if (is_q) {
        bf16_t* dst = (bf16_t*)a.out + (size_t)m * a.ldo + (size_t)head * d;
        dst[i] = (bf16_t)lo;
        dst[i + dhalf] = (bf16_t)hi;
      } else if (a.kcache) {
        const size_t page = (size_t)s_page[m];
        const int off = pos % a.page_size;
        if (is_k) {
          bf16_t* dst = a.kcache + (page * a.nkv + (head - a.nq)) * (size_t)a.page_size * d;
          dst[kcache_index(off, i, d)] = (bf16_t)lo;
          dst[kcache_index(off, i + dhalf, d)] = (bf16_t)hi;
        } else {
          bf16_t* dst = a.vcache + (page * a.nkv + (head - a.nq - a.nkv)) * (size_t)a.page_size * d;
          dst[vcache_index(off, i, d)] = (bf16_t)lo;
          dst[vcache_index(off, i + dhalf, d)] = (bf16_t)hi;
        }
      }
    }
  }
}

// ---------------------------------------------------------------- dispatch
static size_t skinny_lds_bytes(int nsb, int kw, int mb, int M, int K, int epi, bool stage) {
  size_t bytes = sk_float_words(nsb, kw, mb, M, epi) * sizeof(float);
  if (stage) bytes += (size_t)M * ((K + 31) / 32 * 32 + SK_APAD) * sizeof(bf16_t);
  return bytes;
}

// Most LDS a block may take (a compute unit of gfx950 has 160 KB).
static const size_t SK_LDS_LIMIT = 152 * 1024;
// Most rows of a call (tiles of at most 64 rows, a block each per set of columns).
constexpr int SK_MAX_ROWS = 1024;

template <int MB, int EPI, bool NORM, bool STAGE>
static int skinny_launch(const SkinnyArgs& a, int blocks, size_t lds, hipStream_t stream) {
  auto kernel = skinny_block_kernel<MB, EPI, NORM, STAGE>;
  if (lds > 48 * 1024) {
    static size_t raised = 0;     // per instantiation
    if (lds > raised) {
      if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)SK_LDS_LIMIT) != hipSuccess) {
        llmlab_set_error("skinny_linear: cannot raise the LDS limit to %zu bytes", SK_LDS_LIMIT);
        return 3;
      }
      raised = SK_LDS_LIMIT;
    }
  }
  const int grid = a.tiles > 1 ? (blocks + 7) / 8 * 8 * a.tiles : blocks;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * a.nsb * a.kw), lds, stream, a);
  return 0;
}

template <int EPI, bool NORM, bool STAGE>
static int skinny_launch_mb(const SkinnyArgs& a, int mb, int blocks, size_t lds, hipStream_t stream) {
  if (mb == 1) return skinny_launch<1, EPI, NORM, STAGE>(a, blocks, lds, stream);
  if (mb == 2) return skinny_launch<2, EPI, NORM, STAGE>(a, blocks, lds, stream);
  return skinny_launch<4, EPI, NORM, STAGE>(a, blocks, lds, stream);
}

template <int EPI, bool NORM>
static int skinny_launch_stage(const SkinnyArgs& a, bool stage, int mb, int blocks, size_t lds,
                               hipStream_t stream) {
  if constexpr (NORM) {
    return skinny_launch_mb<EPI, true, true>(a, mb, blocks, lds, stream);   // the norm is staged always
  } else {
    if (stage) return skinny_launch_mb<EPI, false, true>(a, mb, blocks, lds, stream);
    return skinny_launch_mb<EPI, false, false>(a, mb, blocks, lds, stream);
  }
}

// Debug interface (kernels/debug.py): a block shape can be forced, for tests and
// measurements (0 = choose).
static int g_force_nsb = 0, g_force_kw = 0, g_force_stage = -1, g_force_mb = 0, g_force_epi = -1;
extern "C" void llmlab_debug_skinny_shape(int nsb, int kw, int stage, int mb) {
  g_force_nsb = nsb;
  g_force_kw = kw;
  g_force_stage = stage;
  g_force_mb = mb;
}
// ... for one epilogue only (-1: for all)
extern "C" void llmlab_debug_skinny_epilogue(int epilogue) { g_force_epi = epilogue; }

struct SkinnyShape {
  int nsb, kw;
  bool stage;
  int qsplit;
  int mb;       // row blocks of 16 per tile of rows (1, 2 or 4); tiles = ceil(M / 16 mb)
};

static inline int sk_tiles(int M, int mb) { return (M + 16 * mb - 1) / (16 * mb); }

// Pick strips per block, K slices per strip and staging by an estimate of the
// kernel's time: a fixed part, plus what the busiest compute unit needs to stream
// its share of W and of x (a unit sustains far less than 1/256 of the chip's
// bandwidth would suggest, so spreading the matrix over all units matters most),
// or the memory round trips of a wave if those take longer.
static SkinnyShape skinny_choose_tile(int epilogue, bool norm, int mb, int M, int tiles, int N, int K, int d,
                                      int num_cus, int ksplit, double* cost_out) {
  const int steps = ((K + 31) / 32 + ksplit - 1) / ksplit;     // per K group of blocks
  const int strips = (N + 15) / 16;
  const int max_waves = mb >= 4 ? 8 : 16;
  SkinnyShape best{0, 0, false, 1, mb};
  double best_cost = 1e30;
  int cand[5], ncand = 0;
  if (epilogue == SK_QKV) {
    cand[ncand++] = d / 16;                   // a block per head
    if (d % 32 == 0 && d > 32) cand[ncand++] = 2;   // or d/32 blocks per head, two strips each
  } else {
    for (int nsb = (epilogue == SK_SWIGLU ? 2 : 1); nsb <= 16; nsb *= 2) cand[ncand++] = nsb;
  }
  for (int ci = 0; ci < ncand; ++ci) {
    const int nsb = cand[ci];
    if (nsb > max_waves) continue;
    for (int kw = 1; kw * nsb <= max_waves && kw <= steps; ++kw) {
      for (int st = norm ? 1 : 0; st < (epilogue == SK_PART ? 1 : 2); ++st) {     // pieces of K: no staging
        const bool stage = st == 1;
        const size_t lds = skinny_lds_bytes(nsb, kw, mb, M, K, epilogue, stage);
        if (lds > SK_LDS_LIMIT) continue;
        const int blocks = (strips + nsb - 1) / nsb * ksplit * tiles;     // (for QKV: heads, or heads * d/32)
        const int per_cu = (blocks + num_cus - 1) / num_cus;       // blocks the busiest unit runs
        int resident = 16 / (nsb * kw);                             // of which so many at a time
        if (resident > per_cu) resident = per_cu;
        const int by_lds = (int)((160 * 1024) / (lds > 1024 ? lds : 1024));
        if (resident > by_lds) resident = by_lds;
        if (resident < 1) resident = 1;
        const int rounds = (per_cu + resident - 1) / resident;
        // a compute unit streams about 50 GB/s from HBM (a good 3 GB/s per resident wave
        // until that limit) and more from the caches; rows of x read by every wave on its own
        // (not staged) come in short strided pieces and cost about twice that
        // (fitted twice: a large matrix is bound by what the waves of a unit keep in
        // flight, up to about 50 GB/s; a small one by latencies, which the lower figures
        // stand for)
        const bool large = (double)N * K * 2.0 >= 64e6;
        double rate = (large ? 3.2e3 : 3.5e3) * resident * nsb * kw;
        // (more than one tile of rows of a wide output: all but the first tile of a set of
        // columns find W in the L2 of their die, and sixteen waves a block draw what eight
        // cannot: gate/up of the 0.5B shape at 48 rows, 10.5 us with 8 strips x 2 slices, 14.3
        // with 4 x 2; a narrow output gains nothing from more slices)
        const double cap = (large || (tiles > 1 && strips >= num_cus)) ? 50.0e3 : 25.0e3;
        if (rate > cap) rate = cap;
        const double t_stream = per_cu * (16.0 * nsb * K * 2.0) / rate;
        const double x_bytes = (double)(stage ? 1 : 2 * nsb) * M * K * (norm ? 4.0 : 2.0);
        const double t_x = per_cu * x_bytes / 50.0e3;
        const int per = (steps + kw - 1) / kw;
        const int u = sk_ring(mb, stage);
        const double trips = stage ? 1.0 + 0.3 * ((per + u - 1) / u - 1) : (double)((per + u - 1) / u);
        const double busy = t_stream + t_x > 0.8 * trips ? t_stream + t_x : 0.8 * trips;
        // a fixed part per kernel, and again (in part hidden by the neighbours) for every
        // further round of blocks on the busiest unit
        const double cost = 3.3 + (stage ? 0.3 : 0.0) + busy + (rounds - 1) * 2.4 / resident +
                            0.03 * kw * nsb;
        if (cost < best_cost) {
          best_cost = cost;
          best = SkinnyShape{nsb, kw, stage, (epilogue == SK_QKV && nsb != d / 16) ? d / 32 : 1, mb};
        }
      }
    }
  }
  *cost_out = best_cost;
  return best;
}

// The rows may be cut into tiles of 16, 32 or 64 as well: smaller tiles give more
// blocks, each of which stages (and norms) fewer rows, and W is read once per tile
// (from the cache after the first).
static SkinnyShape skinny_choose(int epilogue, bool norm, int M, int N, int K, int d, int num_cus,
                                 int ksplit = 1) {
  SkinnyShape best{0, 0, false, 1, 1};
  double best_cost = 1e30;
  // (q/k/v of more than 64 rows: tiles of 16 rows, measured; 576 rows of 1152 x 896 take
  // 13.4 us so, 16.4 in tiles of 32 and 26 in tiles of 64)
  const int mb_max = M <= 16 || (epilogue == SK_QKV && M > 64) ? 1 : (M <= 32 ? 2 : 4);
  for (int mb = mb_max; mb >= 1; mb >>= 1) {
    if (g_force_mb > 0 && (g_force_epi < 0 || g_force_epi == epilogue) && mb != g_force_mb &&
        !(g_force_mb > mb_max && mb == mb_max))
      continue;
    const int tiles = sk_tiles(M, mb);
    double cost;
    const SkinnyShape s = skinny_choose_tile(epilogue, norm, mb, M < 16 * mb ? M : 16 * mb, tiles, N, K, d,
                                             num_cus, ksplit, &cost);
    if (s.nsb > 0 && cost < best_cost) {
      best_cost = cost;
      best = s;
    }
  }
  return best;
}

// The shape the chooser takes for a product (for tests and tuning): out = {nsb, kw, stage, qsplit, mb}.
extern "C" void llmlab_skinny_shape(int epilogue, int norm, int M, int N, int K, int d, int num_cus, int ksplit,
                                    int* out) {
  const SkinnyShape s = skinny_choose(epilogue, norm != 0, M, N, K, d, num_cus, ksplit < 1 ? 1 : ksplit);
  out[0] = s.nsb; out[1] = s.kw; out[2] = s.stage; out[3] = s.qsplit; out[4] = s.mb;
}

// One entry point for the whole family.
//   norm != 0: x is the float32 residual stream (rows x_rows[m] or m), norm_w/eps its RMSNorm
//   epilogue SK_QKV: N = (nq + 2 nkv) * d, one block per head, `out` is q [M, ldo]
//   epilogue SK_PART: K is split over `ksplit` groups of blocks, `out` is float32
//     [ksplit][M][ldo] (part_stride numbers from one piece to the next); nothing is added up
//   pend / pend_splits / pend_ld / pend_stride: pieces that a former SK_PART call left and
//     that belong to the rows of x (norm != 0: added while the rows are read) or to the
//     rows of out (SK_RESID: added with the product, which folds them into the stream)
extern "C" int llmlab_skinny_linear(const void* x, int norm, const int* x_rows, const void* norm_w,
                                    int norm_w_dtype, float eps, const void* w, const void* bias,
                                    int bias_dtype, int epilogue, void* out, int M, int N, int K,
                                    int ldo, int n_out, const float* inv_freq, const int* positions,
                                    const int* row_req, const int* table, int table_stride,
                                    int page_size, void* kcache, void* vcache, int nq, int nkv, int d,
                                    int num_cus, const float* pend, int pend_splits, int pend_ld,
                                    size_t pend_stride, int ksplit, size_t part_stride,
                                    hipStream_t stream) {
  LLMLAB_REQUIRE(M >= 0 && M <= SK_MAX_ROWS, "skinny_linear: takes at most %d rows, got %d", SK_MAX_ROWS, M);
  LLMLAB_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "skinny_linear: bad sizes N=%d K=%d (K must be a multiple of 8)", N, K);
  LLMLAB_REQUIRE(epilogue >= 0 && epilogue <= 5, "skinny_linear: unknown epilogue %d", epilogue);
  LLMLAB_REQUIRE(pend_splits >= 0 && (pend_splits == 0 || (pend != nullptr && (norm || epilogue == SK_RESID))),
                 "skinny_linear: pending sums go with a norm or into the residual");
  LLMLAB_REQUIRE(pend_splits == 0 || !norm ||
                 (pend_ld % 4 == 0 && (uintptr_t)pend % 16 == 0 && pend_stride % 4 == 0),
                 "skinny_linear: pending sums under a norm are read 16 bytes at a time: not aligned");
  if (epilogue != SK_PART) ksplit = 1;
  LLMLAB_REQUIRE(ksplit >= 1 && ksplit <= 16 && (epilogue != SK_PART || (!norm && part_stride >= (size_t)M * ldo)),
                 "skinny_linear(pieces): bad split %d", ksplit);
  LLMLAB_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
                 (norm_w == nullptr || (uintptr_t)norm_w % 16 == 0),
                 "skinny_linear: operands must be 16-byte aligned");
  LLMLAB_REQUIRE(!norm || norm_w != nullptr, "skinny_linear: a norm needs its weight");
  if (M == 0) return 0;
  if (num_cus <= 0) num_cus = 256;
  if (epilogue == SK_QKV) {
    LLMLAB_REQUIRE(d >= 16 && d % 16 == 0 && d <= 256 && N == (nq + 2 * nkv) * d,
                   "skinny_linear(qkv): head size %d / %d rows do not fit", d, N);
    LLMLAB_REQUIRE((kcache == nullptr) == (vcache == nullptr), "skinny_linear(qkv): both caches or none");
    LLMLAB_REQUIRE(positions != nullptr && (kcache == nullptr || (table && row_req && page_size > 0)),
                   "skinny_linear(qkv): positions and block table are needed");
  } else if (epilogue == SK_SWIGLU) {
    LLMLAB_REQUIRE(N % 32 == 0 && 2 * ((n_out + 15) / 16 * 16) == N && bias == nullptr,
                   "skinny_linear(swiglu): %d rows do not interleave %d outputs", N, n_out);
  } else {
    LLMLAB_REQUIRE(n_out == N, "skinny_linear: n_out %d != N %d", n_out, N);
  }
  LLMLAB_REQUIRE(ldo >= (epilogue == SK_QKV ? nq * d : n_out), "skinny_linear: output stride too small");
  SkinnyShape shape = skinny_choose(epilogue, norm != 0, M, N, K, d, num_cus, ksplit);
  const int mb = shape.mb, tiles = sk_tiles(M, mb), tile_rows = M < 16 * mb ? M : 16 * mb;
  const bool forced = g_force_epi < 0 || g_force_epi == epilogue;
  if (forced && g_force_nsb > 0 && epilogue != SK_QKV) shape.nsb = g_force_nsb;
  if (forced && g_force_nsb > 0 && epilogue == SK_QKV && d % 32 == 0 && d > 32) {
    shape.nsb = g_force_nsb == 2 ? 2 : d / 16;
    shape.qsplit = g_force_nsb == 2 ? d / 32 : 1;
  }
  if (forced && g_force_kw > 0) shape.kw = g_force_kw;
  if (forced && g_force_stage >= 0) shape.stage = norm || (g_force_stage != 0 && epilogue != SK_PART);
  LLMLAB_REQUIRE(shape.nsb > 0 && shape.kw > 0,
                 "skinny_linear: no block shape fits N=%d K=%d M=%d (16 rows of x to stage: %zu bytes of LDS)",
                 N, K, M, (size_t)(M < 16 ? M : 16) * ((K + 31) / 32 * 32 + SK_APAD) * sizeof(bf16_t));
  const size_t lds = skinny_lds_bytes(shape.nsb, shape.kw, mb, tile_rows, K, epilogue, shape.stage);
  LLMLAB_REQUIRE(lds <= SK_LDS_LIMIT && shape.nsb * shape.kw <= (mb >= 4 ? 8 : 16),
                 "skinny_linear: block shape %dx%d does not fit", shape.nsb, shape.kw);
  // (only a forced shape can fail these: a gate strip and its up strip share a block, and
  // every K slice has a step)
  LLMLAB_REQUIRE(!(epilogue == SK_SWIGLU && shape.nsb % 2 != 0) &&
                     shape.kw <= ((K + 31) / 32 + ksplit - 1) / ksplit,
                 "skinny_linear: block shape %dx%d does not fit this product", shape.nsb, shape.kw);
  const int blocks = (N + 16 * shape.nsb - 1) / (16 * shape.nsb) * ksplit;
  SkinnyArgs a;
  a.pend = pend; a.pend_splits = pend_splits; a.pend_ld = pend_ld; a.pend_stride = pend_stride;
  a.ksplit = ksplit; a.part_stride = part_stride; a.tiles = tiles; a.col_blocks = blocks;
  a.qsplit = shape.qsplit;
  a.x = x; a.x_rows = x_rows; a.norm_w = norm_w; a.W = (const bf16_t*)w; a.bias = bias; a.out = out;
  a.inv_freq = inv_freq; a.positions = positions; a.row_req = row_req; a.table = table;
  a.kcache = (bf16_t*)kcache; a.vcache = (bf16_t*)vcache;
  a.M = M; a.N = N; a.K = K; a.ldo = ldo; a.n_out = n_out;
  a.norm_w_bf16 = norm_w_dtype == DT_BF16; a.bias_bf16 = bias_dtype == DT_BF16;
  a.nsb = shape.nsb; a.kw = shape.kw; a.nq = nq; a.nkv = nkv; a.d = d; a.table_stride = table_stride;
  a.page_size = page_size; a.eps = eps;
  int rc = 0;
  if (norm) {
    switch (epilogue) {
      case SK_F32: rc = skinny_launch_stage<SK_F32, true>(a, shape.stage, mb, blocks, lds, stream); break;
      case SK_SWIGLU: rc = skinny_launch_stage<SK_SWIGLU, true>(a, shape.stage, mb, blocks, lds, stream); break;
      case SK_QKV: rc = skinny_launch_stage<SK_QKV, true>(a, shape.stage, mb, blocks, lds, stream); break;
      default: LLMLAB_REQUIRE(false, "skinny_linear: epilogue %d has no fused norm", epilogue);
    }
  } else {
    switch (epilogue) {
      case SK_STORE: rc = skinny_launch_stage<SK_STORE, false>(a, shape.stage, mb, blocks, lds, stream); break;
      case SK_RESID: rc = skinny_launch_stage<SK_RESID, false>(a, shape.stage, mb, blocks, lds, stream); break;
      case SK_F32: rc = skinny_launch_stage<SK_F32, false>(a, shape.stage, mb, blocks, lds, stream); break;
      case SK_SWIGLU: rc = skinny_launch_stage<SK_SWIGLU, false>(a, shape.stage, mb, blocks, lds, stream); break;
      case SK_QKV: rc = skinny_launch_stage<SK_QKV, false>(a, shape.stage, mb, blocks, lds, stream); break;
      case SK_PART: rc = skinny_launch_stage<SK_PART, false>(a, false, mb, blocks, lds, stream); break;
      default: LLMLAB_REQUIRE(false, "skinny_linear: epilogue %d needs the norm", epilogue);
    }
  }
  if (rc) return rc;
  LLMLAB_LAUNCH_CHECK("skinny_linear");
  return 0;
}
