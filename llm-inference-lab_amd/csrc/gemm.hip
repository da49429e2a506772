// Matrix products  out = x . W^T  (x [M, K] K-contiguous; W [N, K], in bfloat16
// packed in MFMA fragment order by llmlab_pack_weight, in float32 K-contiguous)
// for gfx950, with the epilogues the model needs fused in.
//
//   bfloat16:  v_mfma_f32_16x16x32_bf16 everywhere.
//     * tiled kernel: 256 threads = 4 waves, block tile 64x64 (waves 2x2), 64x128 or
//       128x128 (waves 1x4, side by side along the columns), or 512 threads = 8 waves on
//       128x256 (1x8), K step 64; x staged through
//       three stages of LDS (rows padded to 80 elements: a wave's 16-byte fragment reads
//       then take 8.4 clocks, as lane-contiguous ones do; 9.5 with 72, 16 unpadded), its
//       fragments read into registers half a tile ahead of their products, the fragments
//       of W read straight from the packed matrix into registers; three or four tiles
//       are on their way from memory in a ring of register buffers while one is
//       multiplied.  With the waves 1x4 every
//       fragment of W is read by one wave only and all four share the rows of x in LDS:
//       5 to 35 % faster than 2x2 waves with W staged through LDS too (which was the
//       large tile before).  Also measured and not adopted: 256x128 tiles with eight
//       64x64 or four 128x64 wave tiles, K steps of 128, 128x256, 64x256, 128x64 and
//       32x128 tiles with 1x4 waves (the second as good as 128x128, no better), eight
//       waves 2x4 on 128x128 and 64x128, a 64x256 tile with eight waves 1x8 for few rows of a wide
//       matrix (as fast as 64x128, no faster), and 256x256 tiles with four 128x128 wave tiles (half the LDS traffic
//       per product, one wave per SIMD: 833 against 793 TF/s on the largest product
//       tried, slower on the rest).  Counters of the 128x128 tile on a product of
//       2048 x 37888 x 3584 (900 TF/s; two blocks share a compute unit, the clock is at
//       2.0 GHz under this load): matrix pipes busy 40 % of the time, LDS 52 % (and
//       counted in bank conflicts for another 21 %), the texture address units 56 %: no
//       unit is the limit alone, the waves wait for one another's turns at three of them.
//     * the largest products (from 1024 rows on, where its blocks fill the chip): a 256x256
//       tile whose eight waves form two groups that alternate between reading LDS and
//       issuing MFMAs, both operands loaded from global memory straight into LDS
//       (gemm_bf16_pingpong): 1.1 to 1.17 PF/s where the tiles above reach 0.9 to 0.97.
//     (products of few rows, as in decode steps, have kernels of their own in decode.hip)
//   float32: a plain FMA kernel (tiles of 64x64 to 128x128, 4x4 to 8x8 outputs per thread) and, for up to 64
//     rows, one in which a wave owns four rows of W and its lanes split the inner size:
//     true 32-bit products and sums, no matrix-core shortcut.
//
// Fragment layout of the 16x16x32 MFMA (wave of 64 lanes, lane l):
//   A operand: row l%16, k = 8*(l/16) .. +7      B operand: column l%16, same k
//   result element i (0..3): row 4*(l/16)+i, column l%16
//
// Epilogues: STORE  out[M,N] (T) = acc (+bias)            RESID  out[M,N] (f32) += acc (+bias)
//            F32    out[M,N] (f32) = acc                   SWIGLU out[M,N/2] (T) = silu(g)*u
//            PART   out[z][M,N] (f32) = acc over the K range of group z
//            QKV    q (T) = rotate(acc + bias); rotated k and v of the rows go to their cache pages
// For SWIGLU the rows of W alternate in runs of 16: gate rows of 16 outputs, then
// the up rows of the same 16 outputs, so fragments j and j+1 hold gate and up of
// the same outputs in the same lanes.
#include "common.h"

enum { EPI_STORE = 0, EPI_RESID = 1, EPI_F32 = 2, EPI_SWIGLU = 3, EPI_QKV = 4, EPI_PART = 5 };

struct EpiArgs {
  void* out;         // T or float, see above
  const void* bias;  // may be null
  int bias_bf16;
  int ldo;    // row stride of out in elements
  int n_out;  // logical output columns (SWIGLU: intermediate size; else N)
  // PART: the inner size is cut over the blocks of grid z, kt_per_split K tiles each; group z
  // leaves its sums (float32, bias in group 0) in out + z * part_stride: the product without
  // the final sum, which the next reader of those rows does
  int kt_per_split;
  size_t part_stride;
  // QKV: the columns are [q heads | k heads | v heads] of size d; q and k are rotated by
  // their row's position, q goes to out [M, ldo], k and v into the cache pages of the row's
  // request (skipped when no cache is given).  A head must lie within one tile (BN % d == 0).
  const float* inv_freq;   // [d/2] or null (no rotation)
  const int* positions;    // [M]
  const int* row_req;      // [M]
  const int* table;        // block table
  bf16_t* kcache;
  bf16_t* vcache;
  int table_stride, page_size, nq, nkv, d;
};

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + __expf(-z)); }

// One output element (non-SWIGLU).
template <typename T, int EPI>
__device__ __forceinline__ void epi_store(const EpiArgs& e, int m, int n, float acc) {
  if (e.bias) acc += load_vec(e.bias, e.bias_bf16, n);
  const size_t at = (size_t)m * e.ldo + n;
  if (EPI == EPI_STORE)
    ((T*)e.out)[at] = from_float<T>(acc);
  else if (EPI == EPI_RESID)
    ((float*)e.out)[at] += acc;
  else
    ((float*)e.out)[at] = acc;
}

// The epilogue of a tile of BM x BN sums that lies in LDS (rows of BN + 4 floats), by the NT
// threads of the block: global memory is written (and the residual read) in pieces of 16 bytes,
// consecutive lanes next to each other.  s_pos, s_page, s_freq and s_bias are what the QKV
// epilogue fetched per row and per column of the tile before the product.
template <int BM, int BN, int NT, int EPI>
__device__ __forceinline__ void tile_epilogue(const float* Cs, const EpiArgs& e, int m0, int n0, int M, int N,
                                              int tid, const int* s_pos, const int* s_page, const float* s_freq,
                                              const float* s_bias) {
  constexpr int C_STRIDE = BN + 4;
  if constexpr (EPI == EPI_QKV) {
    // q and k heads.  A unit of work: eight pairs (i .. i+7, and those + d/2) of one head of
    // one row, rotated and stored 16 bytes at a time (eight neighbours of one octet of d lie
    // next to each other in the key order too).
    const int d = e.d, dh = d >> 1, heads = BN / d, cpl = dh >> 3, head0 = n0 / d;
    const int units = BM * heads * cpl;
    const bool vec = (e.ldo & 7) == 0 && ((uintptr_t)e.out & 15) == 0;
    for (int u = tid; u < units; u += NT) {
      const int jc = u % cpl, t = u / cpl, hh = t % heads, row = t / heads;
      const int m = m0 + row, head = head0 + hh, i = jc * 8;
      if (m >= M || head >= e.nq + e.nkv) continue;          // (values: below)
      const bool is_q = head < e.nq;
      if (!is_q && !e.kcache) continue;
      const float* src = Cs + row * C_STRIDE + hh * d + i;
      float lo[8], hi[8];
#pragma unroll
      for (int q = 0; q < 8; q += 4) {
        const floatx4 l4 = *(const floatx4*)(src + q), h4 = *(const floatx4*)(src + dh + q);
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          lo[q + x] = l4[x] + s_bias[hh * d + i + q + x];
          hi[q + x] = h4[x] + s_bias[hh * d + dh + i + q + x];
        }
      }
      const int pos = s_pos[row];
      if (e.inv_freq) {
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          // the hardware sine and cosine of r = frac(angle / 2 pi)
          float r = (float)pos * s_freq[i + q] * 0.15915494309189535f;
          r -= floorf(r);
          const float sn = __builtin_amdgcn_sinf(r), cs = __builtin_amdgcn_cosf(r);
          const float nlo = lo[q] * cs - hi[q] * sn, nhi = hi[q] * cs + lo[q] * sn;
          lo[q] = nlo;
          hi[q] = nhi;
        }
      }
      bf16x8 blo, bhi;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        blo[q] = (bf16_t)lo[q];
        bhi[q] = (bf16_t)hi[q];
      }
      if (is_q) {
        bf16_t* dst = (bf16_t*)e.out + (size_t)m * e.ldo + (size_t)head * d + i;
        if (vec) {
          *(bf16x8*)dst = blo;
          *(bf16x8*)(dst + dh) = bhi;
        } else {
          for (int q = 0; q < 8; ++q) {
            dst[q] = blo[q];
            dst[dh + q] = bhi[q];
          }
        }
      } else {
        bf16_t* dst = e.kcache + ((size_t)s_page[row] * e.nkv + (head - e.nq)) * (size_t)e.page_size * d;
        const int off = pos % e.page_size;
        *(bf16x8*)(dst + kcache_index(off, i, d)) = blo;
        *(bf16x8*)(dst + kcache_index(off, i + dh, d)) = bhi;
      }
    }
    // v heads.  In the value order four consecutive keys of one number of d lie next to each
    // other, and the numbers of a 16-wide block of d after one another: four rows that are
    // four consecutive positions of one request, the first a multiple of four, put four
    // numbers of a head into 32 consecutive bytes of the page.  The rows of the tile are
    // taken in fours from the first row on whose position is a multiple of four if the tile
    // continues as its first row begins (a prompt from its start does; so does a portion
    // that follows the rows of decoding requests, from its second tile on); a unit of work
    // is such a group of rows by four numbers.  Groups that are not four positions in a row
    // of one request (and the rows before the first group and after the last) store number
    // by number: 2 bytes each, which memory has to merge into what it holds; a tile of
    // value heads stored so finished long after the others.
    const int hv0 = max(0, e.nq + e.nkv - head0), hv1 = min(heads, e.nq + 2 * e.nkv - head0);
    if (e.vcache && hv1 > hv0) {
      const int nv = hv1 - hv0, chunks = d >> 2;
      const int shift = (4 - (s_pos[0] & 3)) & 3;
      const size_t per_page = (size_t)e.page_size * d;
      for (int u = tid; u < (BM / 4 + 1) * nv * chunks; u += NT) {
        const int jc = u % chunks, t = u / chunks, hh = hv0 + t % nv, r0 = shift - 4 + 4 * (t / nv);
        const int dd0 = jc * 4, head = head0 + hh;
        const float* bias = s_bias + hh * d + dd0;
        bool together = r0 >= 0 && r0 + 3 < BM && m0 + r0 + 3 < M;
        if (together) {
          const int pos0 = s_pos[r0];
          together = (pos0 & 3) == 0;
#pragma unroll
          for (int k = 1; k < 4; ++k) together = together && s_pos[r0 + k] == pos0 + k && s_page[r0 + k] == s_page[r0];
        }
        if (together) {
          bf16x8 w0, w1;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const floatx4 v4 = *(const floatx4*)(Cs + (r0 + k) * C_STRIDE + hh * d + dd0);
            w0[k] = (bf16_t)(v4[0] + bias[0]);
            w0[4 + k] = (bf16_t)(v4[1] + bias[1]);
            w1[k] = (bf16_t)(v4[2] + bias[2]);
            w1[4 + k] = (bf16_t)(v4[3] + bias[3]);
          }
          bf16_t* dst = e.vcache + ((size_t)s_page[r0] * e.nkv + (head - e.nq - e.nkv)) * per_page +
                        vcache_index(s_pos[r0] % e.page_size, dd0, d);
          *(bf16x8*)dst = w0;
          *(bf16x8*)(dst + 8) = w1;
        } else {
          for (int k = 0; k < 4; ++k) {
            const int row = r0 + k;
            if (row < 0 || row >= BM || m0 + row >= M) continue;
            const floatx4 v4 = *(const floatx4*)(Cs + row * C_STRIDE + hh * d + dd0);
            bf16_t* dst = e.vcache + ((size_t)s_page[row] * e.nkv + (head - e.nq - e.nkv)) * per_page;
            const int off = s_pos[row] % e.page_size;
#pragma unroll
            for (int x = 0; x < 4; ++x) dst[vcache_index(off, dd0 + x, d)] = (bf16_t)(v4[x] + bias[x]);
          }
        }
      }
    }
  } else if constexpr (EPI == EPI_SWIGLU) {
    // columns of the tile alternate in runs of 16: gate, up of the same 16 outputs
    constexpr int OUTS = BN / 2, CH = OUTS / 8;      // outputs per row of the tile, chunks of 8 of them
    bf16_t* out = (bf16_t*)e.out;
    const int o0 = n0 >> 1;
    const bool vec = (e.ldo & 7) == 0 && ((uintptr_t)out & 15) == 0;
    for (int ch = tid; ch < BM * CH; ch += NT) {
      const int row = ch / CH, oc = (ch % CH) * 8;      // 8 outputs within one run of 16
      const int m = m0 + row;
      if (m >= M) continue;
      const float* gp = Cs + row * C_STRIDE + (oc >> 4) * 32 + (oc & 15);
      const floatx4 g0 = *(const floatx4*)gp, g1 = *(const floatx4*)(gp + 4);
      const floatx4 u0 = *(const floatx4*)(gp + 16), u1 = *(const floatx4*)(gp + 20);
      bf16x8 v;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v[q] = (bf16_t)(silu_f(g0[q]) * u0[q]);
        v[4 + q] = (bf16_t)(silu_f(g1[q]) * u1[q]);
      }
      bf16_t* dst = out + (size_t)m * e.ldo + o0 + oc;
      if (vec && o0 + oc + 8 <= e.n_out) *(bf16x8*)dst = v;
      else
        for (int q = 0; q < 8; ++q)
          if (o0 + oc + q < e.n_out) dst[q] = v[q];
    }
  } else {
    constexpr int CH = BN / 4;                         // chunks of 4 columns per row of the tile
    constexpr bool OUT32 = EPI != EPI_STORE;
    const bool vec = (e.ldo & 3) == 0 && ((uintptr_t)e.out & 15) == 0 && (OUT32 || (e.ldo & 7) == 0);
    for (int ch = tid; ch < BM * CH; ch += NT) {
      const int row = ch / CH, col = (ch % CH) * 4;
      const int m = m0 + row, n = n0 + col;
      if (m >= M || n >= N) continue;
      floatx4 v = *(const floatx4*)(Cs + row * C_STRIDE + col);
      if (e.bias)
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] += load_vec(e.bias, e.bias_bf16, min(n + q, N - 1));
      const size_t at = (size_t)m * e.ldo + n;
      const bool whole = vec && n + 4 <= N;
      if constexpr (EPI == EPI_STORE) {
        bf16_t* dst = (bf16_t*)e.out + at;
        if (whole) {
          bf16x4 o;
#pragma unroll
          for (int q = 0; q < 4; ++q) o[q] = (bf16_t)v[q];
          *(bf16x4*)dst = o;
        } else {
          for (int q = 0; q < 4; ++q)
            if (n + q < N) dst[q] = (bf16_t)v[q];
        }
      } else {
        float* dst = (float*)e.out + at;
        if (whole) {
          if constexpr (EPI == EPI_RESID) v += *(const floatx4*)dst;
          *(floatx4*)dst = v;
        } else {
          for (int q = 0; q < 4; ++q)
            if (n + q < N) dst[q] = (EPI == EPI_RESID ? dst[q] : 0.f) + v[q];
        }
      }
    }
  }
}

// ============================================================ bf16, tiled
template <int BM, int BN, int BK, int WM, int WN, int EPI>
__global__ __launch_bounds__(64 * WM * WN) void gemm_bf16_tiled(const bf16_t* __restrict__ A,
                                                        const bf16_t* __restrict__ W, EpiArgs e, int M,
                                                        int N, int K) {
  constexpr int LDS_STRIDE = BK + 16;        // padded rows: the fragment reads of a wave spread evenly over the banks
  constexpr int NT = 64 * WM * WN;           // threads: WM x WN waves
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
  constexpr int TM = WTM / 16, TN = WTN / 16;
  constexpr int KCH = BK / 8;                // 16-byte chunks in a row of a tile
  constexpr int A_CHUNKS = BM * KCH / NT;    // chunks of x per thread
  static_assert(A_CHUNKS >= 1 && BM * KCH % NT == 0, "tile too small");
  // three stages of LDS for x: the tile after the next is put in while this one is
  // multiplied and the next one's fragments are read, one barrier per tile
  constexpr int A_STAGE = BM * LDS_STRIDE;
  // (one array: after the last tile it holds the block's results for the epilogue)
  constexpr int C_STRIDE = BN + 4;           // floats per row of the result tile in LDS
  constexpr size_t STAGE_BYTES = (size_t)(3 * A_STAGE) * sizeof(bf16_t);
  constexpr size_t C_BYTES = (size_t)BM * C_STRIDE * sizeof(float);
  __shared__ __attribute__((aligned(16))) char smem[STAGE_BYTES > C_BYTES ? STAGE_BYTES : C_BYTES];
  bf16_t* As2 = (bf16_t*)smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // Blocks are handed to the 8 dies (each with an L2 of its own) in turn.  Give
  // every die a band of neighbouring column tiles, rows running fastest, so that
  // what its blocks read at one time is a few column tiles of W and the rows of x.
  int bx = blockIdx.x, by = blockIdx.y;
  {
    const int gx = gridDim.x, gy = gridDim.y, total = gx * gy;
    const int lin = by * gx + bx;
    const int whole = total & ~7;            // the last few blocks (total % 8) keep their place
    const int mapped = lin < whole ? (lin & 7) * (whole >> 3) + (lin >> 3) : lin;
    bx = mapped / gy;
    by = mapped - bx * gy;
  }
  const int m0 = by * BM, n0 = bx * BN;
  const int c = lane & 15, g = lane >> 4;

  // QKV: what the epilogue needs from global memory per row of the tile (position, and the
  // page of that position for the tiles that hold k or v heads) and per column (bias,
  // rotary frequencies) is fetched now, so that those round trips (the page follows the
  // position follows the request) pass behind the product instead of after it.
  constexpr bool QKV = EPI == EPI_QKV;
  __shared__ int s_pos[QKV ? BM : 1], s_page[QKV ? BM : 1];
  __shared__ float s_freq[QKV ? 128 : 1], s_bias[QKV ? BN : 1];
  if constexpr (QKV) {
    if (tid < BM) {
      const int m = min(m0 + tid, M - 1);
      const int pos = e.positions[m];
      s_pos[tid] = pos;
      s_page[tid] = (e.kcache && n0 + BN > e.nq * e.d)
                        ? e.table[(size_t)e.row_req[m] * e.table_stride + pos / e.page_size] : 0;
    }
    for (int i = tid; i < (e.d >> 1); i += NT) s_freq[i] = e.inv_freq ? e.inv_freq[i] : 0.f;
    for (int i = tid; i < BN; i += NT)
      s_bias[i] = (e.bias && n0 + i < N) ? load_vec(e.bias, e.bias_bf16, n0 + i) : 0.f;
  }

  floatx4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Memory latency is several times the time a tile takes to multiply, so PD tiles
  // are on their way at any time: a ring of register buffers, refilled as soon as a
  // buffer has been put into LDS.
  constexpr int PD = (A_CHUNKS + BN * KCH / NT) <= 4 ? 4 : 3;
  bf16x8 ra[PD][A_CHUNKS];
  // every wave reads the B fragments of its columns straight from the packed W into
  // registers; only x goes through LDS
  bf16x8 rbd[PD][BK / 32][TN];
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // Loads are unconditional (a load under a branch makes the compiler wait for every
  // load in flight where the branch ends).  Rows of x past M and pieces past K read
  // a valid piece instead: they meet zeros of the padded W or land in rows nobody
  // stores.  W is packed in fragment order: the 64 columns of a strip of 16 rows
  // are consecutive memory (1 KB per 32 columns), a thread reading 16 bytes of it.
  const int T = (K + 31) >> 5, nstrips = (N + 15) >> 4;
  auto fetch = [&](int slot, int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int ch = tid + i * NT, row = ch / KCH, kc = (ch % KCH) * 8;
      const int m = min(m0 + row, M - 1), k = min(k0 + kc, K - 8);
      ra[slot][i] = *(const bf16x8*)(A + (size_t)m * K + k);
    }
  };
  auto fetch_b = [&](int slot, int k0) {
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int step = (k0 >> 5) + ks;
        const int strip = min(((n0 + wn * WTN) >> 4) + j, nstrips - 1);
        const bf16x8 v = *(const bf16x8*)(W + ((size_t)strip * T + min(step, T - 1)) * 512 + lane * 8);
        rbd[slot][ks][j] = step < T ? v : zero;
      }
  };
  auto stash = [&](int slot, int stage) {
    bf16_t* As = As2 + stage * A_STAGE;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int ch = tid + i * NT, row = ch / KCH, kc = (ch % KCH) * 8;
      *(bf16x8*)(As + row * LDS_STRIDE + kc) = ra[slot][i];
    }
  };

  // this block's K tiles: all of them, or (PART) its group's share starting at tile kt0
  // (tiles past the share are fetched like any other and never multiplied)
  int nk = (K + BK - 1) / BK, kt0 = 0;
  if constexpr (EPI == EPI_PART) {
    kt0 = (int)blockIdx.z * e.kt_per_split;
    nk = max(0, min(nk - kt0, e.kt_per_split));
    e.out = (float*)e.out + (size_t)blockIdx.z * e.part_stride;
    if (blockIdx.z > 0) e.bias = nullptr;
  }
  const int kbase = kt0 * BK;
#pragma unroll
  for (int p = 0; p < PD; ++p) {      // past K: zeros for W
    fetch(p, kbase + p * BK);
    fetch_b(p, kbase + p * BK);
  }
  // Tile t lies in stage t % 3.  It is put there during tile t - 2, and its fragments are
  // read into registers half a tile ahead of their products (those of its first 32
  // columns of K during the second half of tile t - 1), so that the reads of LDS pass
  // behind the matrix instructions of the half before: with one wave on a SIMD nothing
  // else would hide them.  One barrier per tile: what is overwritten during tile t (stage
  // (t + 2) % 3) was last read during tile t - 1.
  auto frags = [&](bf16x8 (&a)[TM], int stage, int ks) {
    const bf16_t* As = As2 + stage * A_STAGE;
#pragma unroll
    for (int i = 0; i < TM; ++i)
      a[i] = *(const bf16x8*)(As + (wm * WTM + i * 16 + c) * LDS_STRIDE + ks * 32 + g * 8);
  };
  static_assert(BK == 64, "two half tiles");
  bf16x8 a0[TM], a1[TM];
  stash(0, 0);
  fetch(0, kbase + PD * BK);
  if (nk > 1) stash(1 % PD, 1);
  fetch(1 % PD, kbase + (PD + 1) * BK);
  __syncthreads();
  frags(a0, 0, 0);
  int stage = 0;                                 // t % 3
  for (int kt = 0; kt < nk; kt += PD) {
#pragma unroll
    for (int p = 0; p < PD; ++p) {
      const int t = kt + p;
      const bool live = t < nk;
      const int p2 = (p + 2) % PD;              // ring slot of tile t + 2 (a constant once unrolled)
      const int stage1 = stage == 2 ? 0 : stage + 1, stage2 = stage1 == 2 ? 0 : stage1 + 1;
      if (live) {
        frags(a1, stage, 1);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[i], rbd[p][0][j], acc[i][j], 0, 0, 0);
        frags(a0, stage1, 0);
        if (t + 2 < nk) stash(p2, stage2);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[i], rbd[p][1][j], acc[i][j], 0, 0, 0);
        __syncthreads();
      }
      // (outside the branch, like every load of the loop: see above)
      fetch(p2, kbase + (t + 2 + PD) * BK);
      fetch_b(p, kbase + (t + PD) * BK);
      stage = stage1;
    }
  }

  // ---- epilogue.  The results go through LDS so that global memory is written (and the
  // residual read) in pieces of 16 bytes, consecutive lanes next to each other: straight
  // from the MFMA layout a wave instruction would touch 32 bytes in each of four rows.
  // (Every live tile ended with a barrier, so the stages are free.)
  float* Cs = (float*)smem;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int x = 0; x < 4; ++x)
        Cs[(wm * WTM + i * 16 + g * 4 + x) * C_STRIDE + wn * WTN + j * 16 + c] = acc[i][j][x];
  __syncthreads();
  tile_epilogue<BM, BN, NT, EPI>(Cs, e, m0, n0, M, N, tid, s_pos, s_page, s_freq, s_bias);
}

// ============================================================ bf16, 256 x 256 by two groups of waves
// The largest products.  Eight waves, each with a 128 x 64 part of a 256 x 256 tile; both
// operands come by direct loads from global memory into LDS (no registers in between), in
// steps of 32 of the inner size, four stages of 32 KB.  The lanes of a load address the
// 16-byte pieces of one MFMA fragment (16 rows of x, or one 1 KB tile of the packed W), which
// the hardware lays down lane after lane: LDS holds fragments, and a fragment read is 1 KB
// of consecutive bytes.  The waves form two groups with a wave on every SIMD each, half a
// step apart: between two barriers one group reads its twelve fragments and issues its
// loads while the other issues its 32 MFMAs, then they change roles, so that the reads of
// LDS and the matrix instructions of a compute unit overlap by construction and not by
// the luck of the scheduler (all eight waves in step: 975 TF/s on 8192 x 37888 x 3584,
// the groups apart: 1065; the 128 x 256 tile of the kernel above: 966).  Under this load
// the chip holds 1.45 to 1.85 GHz, and a step takes 1340 clocks where the MFMAs alone
// need 1024.  A block fills a compute unit; the epilogue takes the two halves of the rows
// through LDS one after the other.
//
// The direct loads are written in assembly: the compiler then knows nothing of them, the
// waits (vmcnt) are placed by hand, and the loop holds no other load that it would count.
//
// BM = 192 is the same with 96 x 64 a wave, for steps whose rows fill tiles of 192 better
// than tiles of 256 (576 rows: three tiles instead of three of which one is a quarter full).
template <int BM, int EPI>
__global__ __launch_bounds__(512) void gemm_bf16_pingpong(const bf16_t* __restrict__ A,
                                                          const bf16_t* __restrict__ W, EpiArgs e, int M,
                                                          int N, int K) {
  static_assert(BM == 256 || BM == 192, "a wave has 128 or 96 rows");
  constexpr int BN = 256, NT = 512, HALF = 128;
  constexpr int TM = BM / 32;                           // blocks of 16 rows of a wave
  constexpr int XF = BM / 16;                           // fragments of x in a step
  constexpr int STAGE = (XF + BN / 16) * 1024;          // bytes: the fragments of x, then 16 of W
  constexpr int C_STRIDE = BN + 4;
  constexpr size_t C_BYTES = (size_t)HALF * C_STRIDE * sizeof(float);
  __shared__ __attribute__((aligned(1024))) char smem[C_BYTES > 4 * STAGE ? C_BYTES : 4 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;                             // waves 0-3 and 4-7: one of each on every SIMD
  const int wm = wave & 1, wn = ((wave >> 1) & 1) | (grp << 1);   // rows wm * BM / 2, columns wn * 64
  int bx = blockIdx.x, by = blockIdx.y;
  {                                                      // a band of column tiles per die, as above
    const int gx = gridDim.x, gy = gridDim.y, total = gx * gy;
    const int lin = by * gx + bx;
    const int whole = total & ~7;
    const int mapped = lin < whole ? (lin & 7) * (whole >> 3) + (lin >> 3) : lin;
    bx = mapped / gy;
    by = mapped - bx * gy;
  }
  const int m0 = by * BM, n0 = bx * BN;
  const int c = lane & 15, g = lane >> 4;

  constexpr bool QKV = EPI == EPI_QKV;
  __shared__ int s_pos[QKV ? BM : 1], s_page[QKV ? BM : 1];
  __shared__ float s_freq[QKV ? 128 : 1], s_bias[QKV ? BN : 1];
  if constexpr (QKV) {
    if (tid < BM) {
      const int m = min(m0 + tid, M - 1);
      const int pos = e.positions[m];
      s_pos[tid] = pos;
      s_page[tid] = (e.kcache && n0 + BN > e.nq * e.d)
                        ? e.table[(size_t)e.row_req[m] * e.table_stride + pos / e.page_size] : 0;
    }
    for (int i = tid; i < (e.d >> 1); i += NT) s_freq[i] = e.inv_freq ? e.inv_freq[i] : 0.f;
    for (int i = tid; i < BN; i += NT)
      s_bias[i] = (e.bias && n0 + i < N) ? load_vec(e.bias, e.bias_bf16, n0 + i) : 0.f;
  }

  // Per step a wave fetches four fragments (three of x with BM = 192): the even waves of x,
  // the odd ones of W (so that both groups fetch both).  Rows past M, strips past N and pieces past K read a
  // valid piece instead: they land in rows and columns that nobody stores, or meet the
  // zeros of the padded W.
  const int T = (K + 31) >> 5, nstrips = (N + 15) >> 4;
  const bool fetches_x = (wave & 1) == 0;
  const int quarter = wave >> 1;
  constexpr int NFX = XF / 4;                           // fragments of x that one of its four waves fetches
  const bf16_t* src[4];
  unsigned dst[4];
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (fetches_x) {
      const int f = min(quarter * NFX + i, XF - 1);
      src[i] = A + (size_t)min(m0 + f * 16 + c, M - 1) * K;
      dst[i] = lds0 + f * 1024;
    } else {
      const int f = quarter * 4 + i;
      src[i] = W + (size_t)min((n0 >> 4) + f, nstrips - 1) * T * 512 + lane * 8;
      dst[i] = lds0 + (XF + f) * 1024;
    }
  }
  auto load_to_lds = [&](const bf16_t* from, unsigned to) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(from), "s"(to)
                 : "memory", "m0");
  };
  // this block's steps: all of them, or (PART) its group's share of the inner size from
  // step `first` on, whose sums go to the group's own piece of the output
  int first = 0, nk = T;
  if constexpr (EPI == EPI_PART) {
    first = (int)blockIdx.z * e.kt_per_split * 2;
    nk = max(0, min(T - first, e.kt_per_split * 2));
    e.out = (float*)e.out + (size_t)blockIdx.z * e.part_stride;
    if (blockIdx.z > 0) e.bias = nullptr;
  }
  auto fetch = [&](int stage, int step) {
    const int t = min(first + step, T - 1);
    if (fetches_x) {
      const size_t off = (size_t)min(t * 32 + g * 8, K - 8);
#pragma unroll
      for (int i = 0; i < NFX; ++i) load_to_lds(src[i] + off, dst[i] + stage * STAGE);
    } else {
      const size_t off = (size_t)t * 512;
#pragma unroll
      for (int i = 0; i < 4; ++i) load_to_lds(src[i] + off, dst[i] + stage * STAGE);
    }
  };
  // lgkmcnt(0) and vmcnt(the loads of two steps): what a wave waits for before a barrier
  auto wait_all_but_two_steps = [&]() {
    if (NFX == 4 || !fetches_x) __builtin_amdgcn_s_waitcnt(0x0070 | 8);
    else __builtin_amdgcn_s_waitcnt(0x0070 | (2 * NFX));
  };

  floatx4 acc[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 a[TM], b[4];

  // every wave passes the same barriers; nothing may move across one
  auto barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
  };
  // Step t lies in stage t % 4.  A wave's memory phase of step t reads its fragments,
  // issues its loads of step t + 3 (into the stage that both groups read last in step
  // t - 1, at least one barrier ago) and waits for its own loads of step t + 1; the
  // barrier after the other group's same phase then says that step t + 1 is whole.
  fetch(0, 0);
  fetch(1, 1);
  fetch(2, 2);
  wait_all_but_two_steps();
  barrier();
  if (grp == 1) barrier();                               // the second group runs half a step behind
  for (int t0 = 0; t0 < nk; t0 += 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = t0 + u;
      if (t < nk) {                                      // (the same for every wave of the block)
        const char* stage = smem + u * STAGE;
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = *(const bf16x8*)(stage + (XF + wn * 4 + j) * 1024 + lane * 16);
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = *(const bf16x8*)(stage + (wm * TM + i) * 1024 + lane * 16);
        fetch((u + 3) & 3, t + 3);
        wait_all_but_two_steps();
        barrier();
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        barrier();
      }
    }
  }
  if (grp == 0) barrier();
  __builtin_amdgcn_s_waitcnt(0x0070);                    // the last loads (past K, never read) are in
  barrier();

  // ---- epilogue: the rows 0-127 of the tile through LDS, then the rest
  float* Cs = (float*)smem;
  auto to_lds = [&](int part) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = wm * (BM / 2) + i * 16;             // of the tile
      if (row / HALF == part) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int x = 0; x < 4; ++x)
            Cs[(row % HALF + g * 4 + x) * C_STRIDE + wn * 64 + j * 16 + c] = acc[i][j][x];
      }
    }
    __syncthreads();
  };
  to_lds(0);
  tile_epilogue<HALF, BN, NT, EPI>(Cs, e, m0, n0, M, N, tid, s_pos, s_page, s_freq, s_bias);
  __syncthreads();
  to_lds(1);
  tile_epilogue<BM - HALF, BN, NT, EPI>(Cs, e, m0 + HALF, n0, M, N, tid, s_pos + (QKV ? HALF : 0),
                                        s_page + (QKV ? HALF : 0), s_freq, s_bias);
}

// ================================================================ float32
// Debug interface: 1 = products of many rows by the plain FMA kernel instead of the matrix
// cores (tests compare the two).
static int g_f32_fma = 0;
extern "C" void llmlab_debug_f32_fma(int on) { g_f32_fma = on; }

// BM x BN outputs per block of 256 threads (16 x 16); thread (ty, tx) owns the TM = BM/16
// rows ty*TM + i and the TN = BN/16 columns tx + 16*j, so for SWIGLU columns j = 0, 2, ..
// are gate and j = 1, 3, .. the up values of the same outputs.  K steps of 8 through LDS
// (both operands transposed, so that a thread reads its TM rows as vectors); the next
// step's numbers are on their way from memory while this one is multiplied.  Plain FMAs.
template <int EPI, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A,
                                                        const float* __restrict__ W, EpiArgs e, int M,
                                                        int N, int K, int vec) {
  constexpr int BK = 8, TM = BM / 16, TN = BN / 16;
  constexpr int LA = BM * BK / 256, LB = BN * BK / 256;      // numbers per thread and step: 2 or 4
  __shared__ __attribute__((aligned(16))) float As[BK][BM + 4];
  __shared__ __attribute__((aligned(16))) float Bs[BK][BN + 4];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;
  // a thread fetches LA (LB) consecutive k of one row of x (of W)
  const int arow = tid / (BK / LA), ak = (tid % (BK / LA)) * LA;
  const int brow = tid / (BK / LB), bk = (tid % (BK / LB)) * LB;
  const float* ap = A + (size_t)min(m0 + arow, M - 1) * K;
  const float* bp = W + (size_t)min(n0 + brow, N - 1) * K;
  float ra[LA], rb[LB];
  auto fetch = [&](int k0) {
    if (vec && k0 + BK <= K) {
      if constexpr (LA == 4) {
        const floatx4 v = *(const floatx4*)(ap + k0 + ak);
        ra[0] = v[0]; ra[1] = v[1]; ra[2] = v[2]; ra[3] = v[3];
      } else {
        ra[0] = ap[k0 + ak]; ra[1] = ap[k0 + ak + 1];
      }
      if constexpr (LB == 4) {
        const floatx4 v = *(const floatx4*)(bp + k0 + bk);
        rb[0] = v[0]; rb[1] = v[1]; rb[2] = v[2]; rb[3] = v[3];
      } else {
        rb[0] = bp[k0 + bk]; rb[1] = bp[k0 + bk + 1];
      }
    } else {
#pragma unroll
      for (int x = 0; x < LA; ++x) ra[x] = k0 + ak + x < K ? ap[k0 + ak + x] : 0.f;
#pragma unroll
      for (int x = 0; x < LB; ++x) rb[x] = k0 + bk + x < K ? bp[k0 + bk + x] : 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
#pragma unroll
    for (int x = 0; x < LA; ++x) As[ak + x][arow] = ra[x];
#pragma unroll
    for (int x = 0; x < LB; ++x) Bs[bk + x][brow] = rb[x];
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; i += 4) {
        const floatx4 v = *(const floatx4*)&As[kk][ty * TM + i];
        a[i] = v[0]; a[i + 1] = v[1]; a[i + 2] = v[2]; a[i + 3] = v[3];
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Bs[kk][tx + 16 * j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if constexpr (EPI == EPI_SWIGLU) {
        if (j & 1) continue;
        const int nb = n0 + 16 * j;
        const int o = (nb >> 5) * 16 + tx;
        if (o < e.n_out) {
          const float z = acc[i][j];
          ((float*)e.out)[(size_t)m * e.ldo + o] = z / (1.f + expf(-z)) * acc[i][j + 1];
        }
      } else {
        const int n = n0 + tx + 16 * j;
        if (n < N) epi_store<float, EPI>(e, m, n, acc[i][j]);
      }
    }
  }
}

// Many rows in float32 on the matrix cores: v_mfma_f32_32x32x2_f32 multiplies and sums in
// true 32 bits (no reduced-precision mode) at twice the rate of unpacked FMAs and with one
// LDS read per operand and instruction.  BM x BN outputs per block of four waves (2 x 2);
// both operands through LDS in steps of 16 of the inner size (rows padded to 17 floats:
// the lanes of an instruction read one number each from 32 consecutive rows without
// bank conflicts), the next step's numbers on their way from memory meanwhile.  The
// product is taken transposed, C^T[n, m] = W x^T, so that a lane holds one row m of the
// output and 16 of its columns, four and four next to each other, and for SWIGLU the gate
// and the up value of an output in the same lane.
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
template <int EPI, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(const float* __restrict__ A,
                                                             const float* __restrict__ W, EpiArgs e, int M,
                                                             int N, int K, int vec) {
  constexpr int KT = 16, LD = KT + 1;
  constexpr int TM = BM / 64, TN = BN / 64;            // 32 x 32 tiles per wave along m and n
  constexpr int LA = BM * KT / 4 / 256, LB = BN * KT / 4 / 256;     // 16-byte pieces per thread and step
  __shared__ float Xs[BM * LD];
  __shared__ float Ws[BN * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int r32 = lane & 31, kk = lane >> 5;
  floatx16 acc[TN][TM];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int x = 0; x < 16; ++x) acc[j][i][x] = 0.f;
  floatx4 ra[LA], rb[LB];
  // piece p of a tile: row p / 4, numbers 4 (p % 4) .. + 3 of the step
  auto fetch = [&](int k0) {
#pragma unroll
    for (int x = 0; x < LA; ++x) {
      const int p = tid + x * 256, row = p >> 2, kq = (p & 3) * 4;
      const float* src = A + (size_t)min(m0 + row, M - 1) * K + k0 + kq;
      if (vec && k0 + kq + 4 <= K) ra[x] = *(const floatx4*)src;
      else
#pragma unroll
        for (int c = 0; c < 4; ++c) ra[x][c] = k0 + kq + c < K ? src[c] : 0.f;
    }
#pragma unroll
    for (int x = 0; x < LB; ++x) {
      const int p = tid + x * 256, row = p >> 2, kq = (p & 3) * 4;
      const float* src = W + (size_t)min(n0 + row, N - 1) * K + k0 + kq;
      if (vec && k0 + kq + 4 <= K) rb[x] = *(const floatx4*)src;
      else
#pragma unroll
        for (int c = 0; c < 4; ++c) rb[x][c] = k0 + kq + c < K ? src[c] : 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += KT) {
    __syncthreads();
#pragma unroll
    for (int x = 0; x < LA; ++x) {
      const int p = tid + x * 256, row = p >> 2, kq = (p & 3) * 4;
#pragma unroll
      for (int c = 0; c < 4; ++c) Xs[row * LD + kq + c] = ra[x][c];
    }
#pragma unroll
    for (int x = 0; x < LB; ++x) {
      const int p = tid + x * 256, row = p >> 2, kq = (p & 3) * 4;
#pragma unroll
      for (int c = 0; c < 4; ++c) Ws[row * LD + kq + c] = rb[x][c];
    }
    __syncthreads();
    if (k0 + KT < K) fetch(k0 + KT);
#pragma unroll
    for (int s2 = 0; s2 < KT; s2 += 2) {
      float wv[TN], xv[TM];
#pragma unroll
      for (int j = 0; j < TN; ++j) wv[j] = Ws[(wn * (BN / 2) + j * 32 + r32) * LD + s2 + kk];
#pragma unroll
      for (int i = 0; i < TM; ++i) xv[i] = Xs[(wm * (BM / 2) + i * 32 + r32) * LD + s2 + kk];
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[j], xv[i], acc[j][i], 0, 0, 0);
    }
  }
  // lane (r32, kk) holds, of every 32 x 32 tile, output row m = r32 and the columns
  // n = 8 (x / 4) + 4 kk + x % 4 for x = 0 .. 15
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * (BM / 2) + i * 32 + r32;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int nb = n0 + wn * (BN / 2) + j * 32;
      if constexpr (EPI == EPI_SWIGLU) {
        // columns 0 .. 15 of the 32 are gate, 16 .. 31 the up values of the same outputs
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          const int o = (nb >> 5) * 16 + 8 * (x >> 2) + 4 * kk + (x & 3);
          if (o < e.n_out) {
            const float z = acc[j][i][x];
            ((float*)e.out)[(size_t)m * e.ldo + o] = z / (1.f + expf(-z)) * acc[j][i][x + 8];
          }
        }
      } else {
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          const int n = nb + 8 * (x >> 2) + 4 * kk + (x & 3);
          if (n < N) epi_store<float, EPI>(e, m, n, acc[j][i][x]);
        }
      }
    }
  }
}

// The largest tile that still gives every compute unit a block.
template <int EPI>
static void launch_f32_tiled(const float* A, const float* W, const EpiArgs& e, int M, int N, int K,
                             int num_cus, hipStream_t stream) {
  const int vec = (K % 4 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  auto blocks = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  if (g_f32_fma == 0) {       // the matrix cores (the plain FMA kernels below stay as their reference)
    if (blocks(128, 128) >= num_cus)
      hipLaunchKernelGGL((gemm_f32_mfma_kernel<EPI, 128, 128>), dim3((N + 127) / 128, (M + 127) / 128), dim3(256),
                         0, stream, A, W, e, M, N, K, vec);
    else
      hipLaunchKernelGGL((gemm_f32_mfma_kernel<EPI, 64, 64>), dim3((N + 63) / 64, (M + 63) / 64), dim3(256), 0,
                         stream, A, W, e, M, N, K, vec);
    return;
  }
  if (blocks(128, 128) >= num_cus)
    hipLaunchKernelGGL((gemm_f32_kernel<EPI, 128, 128>), dim3((N + 127) / 128, (M + 127) / 128), dim3(256), 0,
                       stream, A, W, e, M, N, K, vec);
  else if (blocks(128, 64) >= num_cus)
    hipLaunchKernelGGL((gemm_f32_kernel<EPI, 128, 64>), dim3((N + 63) / 64, (M + 127) / 128), dim3(256), 0,
                       stream, A, W, e, M, N, K, vec);
  else
    hipLaunchKernelGGL((gemm_f32_kernel<EPI, 64, 64>), dim3((N + 63) / 64, (M + 63) / 64), dim3(256), 0,
                       stream, A, W, e, M, N, K, vec);
}

// Few rows in float32 (decode steps, short portions): a block owns NB = 4 rows of W, its KW
// waves split the inner size, and a wave's lanes split its share, four numbers a lane and
// step, so that a wave instruction reads 1 KB of a row of W in a row (any inner size: one
// number at a time where rows are not 16-byte aligned).  Two steps are on their way from
// memory at a time.  MB rows of x go with them (they stay in the caches); the MB x NB sums
// meet by lane shuffles and, across the waves, in LDS in a fixed order.  For SWIGLU the four
// rows are two gate rows and the up rows of the same two outputs.  Still plain FMAs in 32
// bits.  (One wave per block left a narrow output, 224 blocks of the down product, with one
// wave per compute unit walking 19 steps one after the other: 26 us for 17 MB.)
template <int EPI, int MB, int KW>
__global__ __launch_bounds__(64 * KW) void gemm_f32_rows_kernel(const float* __restrict__ A,
                                                                 const float* __restrict__ W, EpiArgs e, int M,
                                                                 int N, int K, int vec) {
  constexpr int NB = 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m0 = blockIdx.y * MB;
  int rows_w[NB];
  if constexpr (EPI == EPI_SWIGLU) {
    const int n = (blockIdx.x >> 3) * 32 + (blockIdx.x & 7) * 2;     // two gate rows; their up rows 16 on
    rows_w[0] = n; rows_w[1] = n + 1; rows_w[2] = n + 16; rows_w[3] = n + 17;
  } else {
#pragma unroll
    for (int j = 0; j < NB; ++j) rows_w[j] = blockIdx.x * NB + j;
  }
  const float* wp[NB];
  const float* xp[MB];
#pragma unroll
  for (int j = 0; j < NB; ++j) wp[j] = W + (size_t)min(rows_w[j], N - 1) * K;   // clamped: read, never stored
#pragma unroll
  for (int i = 0; i < MB; ++i) xp[i] = A + (size_t)min(m0 + i, M - 1) * K;
  float acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) acc[i][j] = 0.f;
  if (vec) {
    constexpr int STEP = 256 * KW;
    auto mac = [&](const floatx4 (&w4)[NB], const floatx4 (&x4)[MB]) {
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int c = 0; c < 4; ++c) acc[i][j] = fmaf(x4[i][c], w4[j][c], acc[i][j]);
    };
    int k = (wave * 64 + lane) * 4;
    for (; k + STEP < K; k += 2 * STEP) {            // two steps at a time
      floatx4 w4[2][NB], x4[2][MB];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int j = 0; j < NB; ++j) w4[u][j] = *(const floatx4*)(wp[j] + k + u * STEP);
#pragma unroll
        for (int i = 0; i < MB; ++i) x4[u][i] = *(const floatx4*)(xp[i] + k + u * STEP);
      }
      mac(w4[0], x4[0]);
      mac(w4[1], x4[1]);
    }
    for (; k < K; k += STEP) {
      floatx4 w4[NB], x4[MB];
#pragma unroll
      for (int j = 0; j < NB; ++j) w4[j] = *(const floatx4*)(wp[j] + k);
#pragma unroll
      for (int i = 0; i < MB; ++i) x4[i] = *(const floatx4*)(xp[i] + k);
      mac(w4, x4);
    }
  } else {
    for (int k = wave * 64 + lane; k < K; k += 64 * KW) {
      float w1[NB], x1[MB];
#pragma unroll
      for (int j = 0; j < NB; ++j) w1[j] = wp[j][k];
#pragma unroll
      for (int i = 0; i < MB; ++i) x1[i] = xp[i][k];
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) acc[i][j] = fmaf(x1[i], w1[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) acc[i][j] = wave_sum(acc[i][j]);
  if constexpr (KW > 1) {
    __shared__ float red[KW][MB][NB];
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) red[wave][i][j] = acc[i][j];
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        float t = red[0][i][j];
#pragma unroll
        for (int w = 1; w < KW; ++w) t += red[w][i][j];
        acc[i][j] = t;
      }
  } else {
    if (lane != 0) return;
  }
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int m = m0 + i;
    if (m >= M) continue;
    if constexpr (EPI == EPI_SWIGLU) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int o = (rows_w[j] >> 5) * 16 + (rows_w[j] & 15);
        if (o < e.n_out) {
          const float z = acc[i][j];
          ((float*)e.out)[(size_t)m * e.ldo + o] = z / (1.f + expf(-z)) * acc[i][j + 2];
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < NB; ++j)
        if (rows_w[j] < N) epi_store<float, EPI>(e, m, rows_w[j], acc[i][j]);
    }
  }
}

template <int EPI, int KW>
static void launch_f32_rows_kw(const float* A, const float* W, const EpiArgs& e, int M, int N, int K, int vec,
                               unsigned groups, hipStream_t stream) {
  if (M == 1)
    hipLaunchKernelGGL((gemm_f32_rows_kernel<EPI, 1, KW>), dim3(groups, 1), dim3(64 * KW), 0, stream, A, W, e, M, N, K, vec);
  else if (M == 2)
    hipLaunchKernelGGL((gemm_f32_rows_kernel<EPI, 2, KW>), dim3(groups, 1), dim3(64 * KW), 0, stream, A, W, e, M, N, K, vec);
  else if (M <= 4)
    hipLaunchKernelGGL((gemm_f32_rows_kernel<EPI, 4, KW>), dim3(groups, 1), dim3(64 * KW), 0, stream, A, W, e, M, N, K, vec);
  else
    hipLaunchKernelGGL((gemm_f32_rows_kernel<EPI, 8, KW>), dim3(groups, (M + 7) / 8), dim3(64 * KW), 0, stream, A, W, e,
                       M, N, K, vec);
}

// Waves per block: as many as give every wave at least two steps of its own, up to 8, fewer
// where the blocks alone already put several waves on every compute unit.
template <int EPI>
static void launch_f32_rows(const float* A, const float* W, const EpiArgs& e, int M, int N, int K, int num_cus,
                            hipStream_t stream) {
  const int vec = (K % 4 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  const unsigned groups = EPI == EPI_SWIGLU ? (unsigned)(N / 32) * 8 : (unsigned)((N + 3) / 4);
  const long blocks = (long)groups * ((M + 7) / 8);
  const int steps = (K + 255) / 256;
  int kw = 1;
  while (kw < 8 && steps >= 4 * kw && blocks * kw < 8L * num_cus) kw *= 2;
  if (kw >= 8) launch_f32_rows_kw<EPI, 8>(A, W, e, M, N, K, vec, groups, stream);
  else if (kw == 4) launch_f32_rows_kw<EPI, 4>(A, W, e, M, N, K, vec, groups, stream);
  else if (kw == 2) launch_f32_rows_kw<EPI, 2>(A, W, e, M, N, K, vec, groups, stream);
  else launch_f32_rows_kw<EPI, 1>(A, W, e, M, N, K, vec, groups, stream);
}
constexpr int F32_ROWS_MAX = 64;     // up to here the few-row kernel (the tiled one would run on N / 64 blocks)

// ================================================================ dispatch
// Four tile shapes with x through LDS and W straight from the packed matrix: 64 x 64 (four
// waves 2 x 2) for small products; 64 x 128 and 128 x 128 with four waves and 128 x 256
// with eight, side by side along the columns (1 x 4, 1 x 8), so that every fragment of W
// is read by one wave only and the rows of x in LDS are shared by all of them; and the
// 256 x 256 tile of gemm_bf16_pingpong for the largest products.  The shape
// is picked by an estimate of the time, fitted to sweeps of the four products of a layer
// at three model shapes and 576 to 8192 rows (its picks cost 0.8 % over the best shape
// there):
//   time = L + rounds * (f + K tiles * tk),  rounds = max(1, blocks / (units * resident)).
// One block of the 128 x 256 tile fills a compute unit (its epilogue stages 133 KB), so
// its rounds are whole: ceil(blocks / units).  Where its blocks fill their rounds it is
// the fastest by 5 to 20 % (2048 rows, 3584 x 18944: 301 us against 337 with 128 x 128;
// 8192 rows, 37888 x 3584: 2320 against 2577), where the last round is nearly empty the
// slowest (2048 rows, 5120 x 27648: 852 against 731).
// With few rows the product is bound by the read of W instead: a block draws `stream`
// bytes a microsecond, the chip 5.3e6 at most (one tile of rows, 17 to 64 of them, of
// matrices from 9 to 283 MB, in 4 or 8 pieces: the estimate is within 2 us of the
// measurement).
enum { TILE_64 = 0, TILE_64x128 = 1, TILE_128 = 2, TILE_128x256 = 3, TILE_256 = 4, TILE_192 = 5, TILE_KINDS = 6 };
struct TileModel {
  int bm, bn;
  double L, f, tk, resident, stream;
  int whole_rounds;
};
static const TileModel TILE_MODELS[TILE_KINDS] = {{64, 64, 6.39, 0.79, 0.289, 1.0, 20e3, 0},
                                                  {64, 128, 6.54, 0.71, 0.5, 1.5, 27e3, 0},
                                                  {128, 128, 8.0, 0.48, 0.66, 1.0, 24e3, 0},
                                                  {128, 256, 0.0, 6.16, 0.945, 1.0, 24e3, 1},
                                                  {256, 256, 0.0, 9.2, 1.8, 1.0, 24e3, 1},
                                                  {192, 256, 0.0, 9.2, 1.4, 1.0, 24e3, 1}};
constexpr double CHIP_STREAM = 5.3e6;     // bytes a microsecond

// The tiles of the two groups of waves: whole rounds of one block a unit; with 256 rows a
// step of 32 of the inner size takes 0.82 us in a full round and from 0.56 us in a round of
// few blocks (the chip clocks higher), and 9.6 us pass before and after the loop; with 192
// rows 0.64, 0.47 and 7.6 us (fitted to the same sweeps, inner sizes from 896 to 27648: 8
// and 9 % rms).
static double pingpong_cost(int bm, int M, int N, int K, int num_cus, int pieces) {
  const double rounds = (double)((M + bm - 1) / bm) * ((N + 255) / 256) * pieces / num_cus;
  const double whole = floor(rounds + 1e-9), last = rounds - whole;
  const int steps = pieces > 1 ? 2 * (((K + 63) / 64 + pieces - 1) / pieces) : (K + 31) / 32;
  const double before_after = bm == 256 ? 9.6 : 7.6, full = bm == 256 ? 0.816 : 0.637, few = bm == 256 ? 0.555 : 0.472;
  double t = whole * (before_after + steps * full);
  if (last > 1e-9) t += before_after + steps * (few + (full - few) * last);
  return t;
}

static double tile_cost(int kind, int M, int N, int K, int num_cus, int pieces) {
  if (kind == TILE_256 || kind == TILE_192) return pingpong_cost(TILE_MODELS[kind].bm, M, N, K, num_cus, pieces);
  const TileModel& t = TILE_MODELS[kind];
  const double blocks = (double)((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn) * pieces;
  double rounds = blocks / (num_cus * t.resident);
  // (the 64 x 64 tile beyond 64 rows: measured, a block more than the units hold costs a whole
  // round: 256 rows of 4608 x 3584, 288 blocks, 32 us against 29 with 144 blocks of 64 x 128,
  // and 192 rows, 216 blocks, 26 against 29)
  if (t.whole_rounds || (kind == TILE_64 && M > 64)) rounds = ceil(rounds - 1e-9);
  const int nk = ((K + 63) / 64 + pieces - 1) / pieces;
  const double compute = (rounds > 1.0 ? rounds : 1.0) * (t.f + nk * t.tk);
  const double rate = blocks * t.stream < CHIP_STREAM ? blocks * t.stream : CHIP_STREAM;
  const double read = (double)N * K * 2.0 / rate;
  return t.L + (compute > read ? compute : read);
}

// Debug interface (kernels/debug.py): a tile can be forced, for tests and measurements
// (0 = choose; 64, 130 = 64 x 128, 129 = 128 x 128, 131 = 128 x 256, 132 = 256 x 256, 133 =
// 192 x 256; -131 = choose among the first three; -256 and below: the tiles of two groups
// of waves from so many rows on).
static int g_force_tile = 0, g_without_wide = 0, g_pp_min_rows = 512;
// The 128 x 256 tile is weighed from so many rows on.  (By the product alone it would pay from
// 768: 1,536 rows of 5120 x 27648 447 us against 543; inside prefill steps of 768 to 1,536
// tokens of five shapes that is between 1.4 % faster and 1.3 % slower than from 2,048 on.)
constexpr int WIDE_TILE_MIN_ROWS = 2048;
constexpr int PP_MIN_INNER = 896;      // the shortest inner size the estimates of those tiles were fitted to
extern "C" void llmlab_debug_gemm_tile(int tile) {
  g_force_tile = tile > 0 ? tile : 0;
  g_without_wide = tile == -131;
  g_pp_min_rows = tile <= -256 ? -tile : 512;
}

static int choose_tile(int M, int N, int K, int num_cus) {
  if (g_force_tile == 64) return TILE_64;
  if (g_force_tile == 130) return TILE_64x128;
  if (g_force_tile == 129 || g_force_tile == 128) return TILE_128;
  if (g_force_tile == 131) return TILE_128x256;
  if (g_force_tile == 132) return TILE_256;
  if (g_force_tile == 133) return TILE_192;
  // One or two tiles of rows of a wide matrix (the head, gate and up at larger shapes):
  // bound by the read of W, which the wider tiles stream better than the estimate
  // knows, and the 128-row tile reads W once where two 64-row tiles read it twice
  // (64 rows, 152064 x 3584: 220 us against 250 with the 64 x 64 tile; 128 rows,
  // 55296 x 5120: 127 against 157).
  const long wide = (N + 127) / 128;
  if (M <= 64 && wide >= num_cus) return TILE_64x128;
  // ... and of a matrix of 32,768 to 65,536 rows the 128 x 256 tile (96 / 128 rows of 37888 x
  // 3584: 81 / 77 us against 83 / 84; of 59136 x 8192: 195 / 201 against 200 / 209; a decode
  // step of 128 requests of the 7B shape 6.99 -> 6.86 ms, of the 32B shape 24.8 -> 24.4; a
  // vocabulary of 152,064 gains nothing from it)
  if (M > 64 && M <= 128 && N >= 32768 && N <= 65536 && K >= 1024 && !g_without_wide) return TILE_128x256;
  if (M > 64 && M <= 128 && wide >= 3L * num_cus / 2) return TILE_128;
  // The 128 x 256 tile from 2048 rows on: with 576 and 1024 rows it wins or loses a few
  // percent by the product alone, and a prefill step of 1024 tokens as a whole is 1 to
  // 2 % slower with it than without (steps of 2048: from 0.6 % slower to 3 % faster by
  // the shape of the model, of 4096 and 8192: 3 to 7 % faster at the larger shapes), and
  // an inner size of 1024 on: with 896 its one block per unit shows its start and its
  // epilogue, and steps of 4096 are 1.7 % slower with it.
  const int kinds = M >= WIDE_TILE_MIN_ROWS && K >= 1024 && !g_without_wide ? TILE_256 : TILE_128x256;
  double cost[TILE_KINDS];
  int best = 0;
  for (int kind = 0; kind < kinds; ++kind) {
    cost[kind] = tile_cost(kind, M, N, K, num_cus, 1);
    if (cost[kind] < cost[best]) best = kind;
  }
  // Enough 128 x 128 tiles for four rounds of blocks: a large tile, whatever the
  // estimate makes of the rows it pads (576 rows, 37888 x 3584: 206 us against 221 with
  // 64 x 128; 1024 rows: 324 against 370).  Which of the two, the estimates cannot tell
  // here (they err by 10 % in opposite directions): the 128 x 256 tile unless its last
  // round is less than half full and one of few (2048 rows, 37888 x 3584, 9.25 rounds:
  // 640 us against 588 inside a prefill step; 18.5 rounds: 1246 against 1273; 37: 2302
  // against 2517; 3.5 rounds, 7168 x 5120: 359 against 379).
  if (((long)(M + 127) / 128) * wide >= 4L * num_cus) {
    best = TILE_128;
    if (kinds > TILE_128x256) {
      const double rounds = (double)((M + 127) / 128) * ((N + 255) / 256) / num_cus;
      const double last = rounds - floor(rounds);
      if (last < 1e-9 || last >= 0.5 || rounds >= 16.0) best = TILE_128x256;
    }
  }
  // The tiles of the two groups of waves where the estimate of one is the lowest (over the
  // sweeps the 256 x 256 tile is then 10 to 24 % faster than the best of the others: 2048
  // rows, 37888 x 3584: 501 us against 623; 55296 x 5120: 999 against 1245; with a quarter
  // of a round of blocks it is twice as slow; the 192 x 256 tile where its blocks fill
  // their rounds better: 2048 rows, 5120 x 27648: 534 us against 655 with 256 rows).
  // From 512 rows on (prefill steps of 512 to 960 tokens as a whole: 2.4 to 6.8 % faster at
  // the 7B shape, 3 to 4.6 % at the 32B shape; from 256 rows a step of 384 tokens would be
  // 13 % slower at the 7B shape: the estimates are not fitted there) and an inner size of
  // 896, the shortest measured (steps of 1024 / 4096 / 8192 tokens of the 0.5B shape: 5.8 /
  // 3.5 / 5.8 % faster, 576 and 2048 unchanged).  (The same two groups of waves on a 128 x
  // 256 tile, 64 x 64 a wave, are as fast as the 128 x 256 tile above and no faster: a wave
  // then reads as many bytes from LDS per MFMA as there, and LDS is the limit of both.)
  // ... and from 129 rows on for a wide matrix, where one or two tiles of rows already fill the
  // chip (192 / 256 / 384 rows of 55296 x 5120: 153 / 171 / 261 us against 187 / 199 / 274 with the
  // best of the others; of 59136 x 8192: 229 / 263 / 392 against 305 / 316 / 437)
  const bool pp_rows = M >= g_pp_min_rows || (g_pp_min_rows == 512 && M > 128 && N >= 16384);
  if (pp_rows && K >= PP_MIN_INNER && !g_without_wide) {
    double least = tile_cost(best, M, N, K, num_cus, 1);
    for (int kind = TILE_256; kind <= TILE_192; ++kind) {
      const double c = tile_cost(kind, M, N, K, num_cus, 1);
      if (c < least) {
        least = c;
        best = kind;
      }
    }
  }
  return best;
}

template <int EPI>
static void launch_tile(int kind, const bf16_t* A, const bf16_t* W, const EpiArgs& e, int M, int N, int K,
                        int pieces, hipStream_t stream) {
  const TileModel& t = TILE_MODELS[kind];
  dim3 grid((N + t.bn - 1) / t.bn, (M + t.bm - 1) / t.bm, pieces);
  if (kind == TILE_64)
    hipLaunchKernelGGL((gemm_bf16_tiled<64, 64, 64, 2, 2, EPI>), grid, dim3(256), 0, stream, A, W, e, M, N, K);
  else if (kind == TILE_64x128)
    hipLaunchKernelGGL((gemm_bf16_tiled<64, 128, 64, 1, 4, EPI>), grid, dim3(256), 0, stream, A, W, e, M, N, K);
  else if (kind == TILE_128)
    hipLaunchKernelGGL((gemm_bf16_tiled<128, 128, 64, 1, 4, EPI>), grid, dim3(256), 0, stream, A, W, e, M, N, K);
  else if (kind == TILE_128x256)
    hipLaunchKernelGGL((gemm_bf16_tiled<128, 256, 64, 1, 8, EPI>), grid, dim3(512), 0, stream, A, W, e, M, N, K);
  else {
    if (kind == TILE_256)
      hipLaunchKernelGGL((gemm_bf16_pingpong<256, EPI>), grid, dim3(512), 0, stream, A, W, e, M, N, K);
    else
      hipLaunchKernelGGL((gemm_bf16_pingpong<192, EPI>), grid, dim3(512), 0, stream, A, W, e, M, N, K);
  }
}

// Whether (and into how many pieces along K) a product that adds into float32 rows should
// be left unsummed, and with which tile: out = {pieces (1: no), tile kind}.  A piece costs
// a write and a read of the result by whoever sums it up later.
extern "C" void llmlab_linear_plan(int M, int N, int K, int num_cus, int max_pieces, int min_tiles_per_piece,
                                   int* out) {
  if (num_cus <= 0) num_cus = 256;
  const int nk = (K + 63) / 64;
  const double piece = (double)M * N * 2.2e-6 + 0.3;
  int best_kind = choose_tile(M, N, K, num_cus), best_pieces = 1;
  double best_cost = tile_cost(best_kind, M, N, K, num_cus, 1);
  // 65 to 128 rows: one tile of 128 rows reads W once where two of 64 read it twice, which
  // the estimate does not know (128 rows of 3584 x 18944 in pieces: 45 us against 57, a decode
  // step of 128 requests of that shape 7.11 ms against 7.30)
  const bool one_tile_of_128 = M > 64 && M <= 128 && g_force_tile == 0 && (double)N * K * 2.0 >= 64e6;
  if (one_tile_of_128) {
    best_kind = TILE_128;
    best_cost = tile_cost(TILE_128, M, N, K, num_cus, 1);
  }
  for (int kind = TILE_64x128; kind < TILE_KINDS; ++kind) {
    if (kind == TILE_128x256) continue;
    if (one_tile_of_128 && kind != TILE_128) continue;
    if (kind >= TILE_256 && !(M >= g_pp_min_rows && K >= PP_MIN_INNER && !g_without_wide)) continue;
    if (g_force_tile != 0 && kind != choose_tile(M, N, K, num_cus)) continue;
    for (int s = 2; s <= max_pieces; ++s) {
      if ((nk + s - 1) / s < min_tiles_per_piece) break;
      const double c = tile_cost(kind, M, N, K, num_cus, s) + s * piece;
      if (c < best_cost) {
        best_cost = c;
        best_kind = kind;
        best_pieces = s;
      }
    }
  }
  // Two or three well-filled tiles of 128 rows of a matrix 5,120 to 16,383 wide: four pieces of
  // the 128 x 128 tile, which the estimate prices too high there (with the norm that folds
  // them, 384 rows of 8192 x 29568: 248 us against 365 whole with 64 x 128; of 5120 x 27648:
  // 150 against 183 in two pieces; 256 rows of 8192 x 8192: 65 against 70; at 3,584 columns
  // it loses as often as it wins).  Inside prefill steps of 256 / 320 / 384 tokens of the 14B
  // shape 14.5 -> 14.2 / 16.5 -> 15.5 / 17.6 -> 16.7 ms, of the 32B shape 27.3 -> 27.0 / 34.0 ->
  // 31.2 / 35.9 -> 33.8; at 192 rows the 32B shape loses 5 % with it, hence from 256 on.
  if (M >= 256 && M <= 384 && 4 * M >= 3 * ((M + 127) / 128) * 128 && N >= 5120 && N < 16384 &&
      g_force_tile == 0 && max_pieces >= 4 && (nk + 3) / 4 >= min_tiles_per_piece) {
    best_kind = TILE_128;
    best_pieces = 4;
  }
  // One tile of rows in pieces: the small tile, if its blocks still find a compute unit
  // each (17 to 64 rows of matrices from 9 to 45 MB: 8.6 against 11.0, 12.4 against
  // 15.8, 15.1 against 18.8 us; with more blocks than units it is the slower one)
  if (M <= 64 && best_pieces > 1 && g_force_tile == 0 && (long)((N + 63) / 64) * best_pieces <= num_cus)
    best_kind = TILE_64;
  out[0] = best_pieces;
  out[1] = best_kind;
}

// q/k/v projection of many rows with bias, rotation and cache write in the epilogue
// (bfloat16).  The tile is chosen as for any product; the head size must divide it.
extern "C" int llmlab_linear_qkv(const void* x, const void* w, const void* bias, int bias_dtype, void* q_out,
                                 int M, int N, int K, int ldo, const float* inv_freq, const int* positions,
                                 const int* row_req, const int* table, int table_stride, int page_size,
                                 void* kcache, void* vcache, int nq, int nkv, int d, int num_cus,
                                 hipStream_t stream) {
  LLMLAB_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 8 == 0, "linear_qkv: bad sizes M=%d N=%d K=%d", M, N, K);
  LLMLAB_REQUIRE(d >= 16 && d % 16 == 0 && nq > 0 && nkv > 0 && N == (nq + 2 * nkv) * d && ldo >= nq * d,
                 "linear_qkv: %d + 2 x %d heads of %d do not make %d columns (row stride %d)", nq, nkv, d, N, ldo);
  LLMLAB_REQUIRE((kcache == nullptr) == (vcache == nullptr), "linear_qkv: both caches or none");
  LLMLAB_REQUIRE(positions != nullptr && (kcache == nullptr || (table && row_req && page_size > 0)),
                 "linear_qkv: positions and block table are needed");
  LLMLAB_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
                 ((uintptr_t)kcache % 16 == 0) && ((uintptr_t)vcache % 16 == 0),
                 "linear_qkv: operands must be 16-byte aligned");
  if (M == 0) return 0;
  if (num_cus <= 0) num_cus = 256;
  EpiArgs e{q_out, bias, bias_dtype == DT_BF16, ldo, N, 0, 0, inv_freq, positions, row_req, table,
            (bf16_t*)kcache, (bf16_t*)vcache, table_stride, page_size, nq, nkv, d};
  const int kind = choose_tile(M, N, K, num_cus);
  LLMLAB_REQUIRE(TILE_MODELS[kind].bn % d == 0, "linear_qkv: heads of %d do not divide the tile of %d columns", d,
                 TILE_MODELS[kind].bn);
  launch_tile<EPI_QKV>(kind, (const bf16_t*)x, (const bf16_t*)w, e, M, N, K, 1, stream);
  LLMLAB_LAUNCH_CHECK("linear_qkv");
  return 0;
}

// The width of the tile (64, 128 or 256 columns) that a product of these sizes gets: for
// callers that must know whether a head fits it.
extern "C" int llmlab_linear_tile(int M, int N, int K, int num_cus) {
  if (num_cus <= 0) num_cus = 256;
  return TILE_MODELS[choose_tile(M, N, K, num_cus)].bn;
}

// parts[z] = x[:, K_z] . W[:, K_z]^T for `ksplit` ranges K_z of the inner size (whole K
// tiles of 64 each); bias in parts[0].  bfloat16 only; `tile` as llmlab_linear_plan gives it.
extern "C" int llmlab_linear_partials(const void* x, const void* w, float* parts, const void* bias,
                                      int bias_dtype, int M, int N, int K, int ldo, int ksplit,
                                      size_t part_stride, int tile, hipStream_t stream) {
  LLMLAB_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 8 == 0, "linear_partials: bad sizes M=%d N=%d K=%d", M, N, K);
  LLMLAB_REQUIRE(ksplit >= 1 && ksplit <= 16 && ldo >= N && part_stride >= (size_t)M * ldo,
                 "linear_partials: %d pieces, row stride %d", ksplit, ldo);
  LLMLAB_REQUIRE(tile >= TILE_64 && tile < TILE_KINDS, "linear_partials: unknown tile %d", tile);
  LLMLAB_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0),
                 "linear_partials: operands must be 16-byte aligned");
  if (M == 0) return 0;
  const int nk = (K + 63) / 64;
  EpiArgs e{parts, bias, bias_dtype == DT_BF16, ldo, N, (nk + ksplit - 1) / ksplit, part_stride,
            nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0};
  launch_tile<EPI_PART>(tile, (const bf16_t*)x, (const bf16_t*)w, e, M, N, K, ksplit, stream);
  LLMLAB_LAUNCH_CHECK("linear_partials");
  return 0;
}

// x [M,K] (dtype), w [N,K] (float32: row-major; bfloat16: packed); epilogue selects what `out` is.  For SWIGLU N
// is the number of interleaved weight rows (2 * ceil16(n_out)).
extern "C" int llmlab_linear(const void* x, const void* w, int dtype, int epilogue, void* out,
                             const void* bias, int bias_dtype, int M, int N, int K, int ldo, int n_out,
                             int num_cus, hipStream_t stream) {
  LLMLAB_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
  LLMLAB_REQUIRE(epilogue >= 0 && epilogue <= 3, "linear: unknown epilogue %d", epilogue);
  if (epilogue == EPI_SWIGLU) {
    LLMLAB_REQUIRE(N % 32 == 0 && n_out > 0 && 2 * ((n_out + 15) / 16 * 16) == N,
                   "linear(swiglu): %d weight rows do not interleave %d outputs", N, n_out);
    LLMLAB_REQUIRE(bias == nullptr, "linear(swiglu): no bias");
  } else {
    LLMLAB_REQUIRE(n_out == N, "linear: n_out %d != N %d", n_out, N);
  }
  LLMLAB_REQUIRE(ldo >= n_out, "linear: output row stride %d < %d columns", ldo, n_out);
  if (M == 0) return 0;
  EpiArgs e{out, bias, bias_dtype == DT_BF16, ldo, n_out, 0, 0,
            nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0};
  if (num_cus <= 0) num_cus = 256;
  if (dtype == DT_BF16) {
    LLMLAB_REQUIRE(K % 8 == 0, "linear(bfloat16): inner size %d must be a multiple of 8", K);
    LLMLAB_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0),
                   "linear(bfloat16): operands must be 16-byte aligned");
    const bf16_t* A = (const bf16_t*)x;
    const bf16_t* W = (const bf16_t*)w;
    const int kind = choose_tile(M, N, K, num_cus);
    switch (epilogue) {
      case EPI_STORE: launch_tile<EPI_STORE>(kind, A, W, e, M, N, K, 1, stream); break;
      case EPI_RESID: launch_tile<EPI_RESID>(kind, A, W, e, M, N, K, 1, stream); break;
      case EPI_F32: launch_tile<EPI_F32>(kind, A, W, e, M, N, K, 1, stream); break;
      default: launch_tile<EPI_SWIGLU>(kind, A, W, e, M, N, K, 1, stream); break;
    }
  } else {
    const float* A = (const float*)x;
    const float* W = (const float*)w;
    if (M <= F32_ROWS_MAX) {
      switch (epilogue) {
        case EPI_STORE: launch_f32_rows<EPI_STORE>(A, W, e, M, N, K, num_cus, stream); break;
        case EPI_RESID: launch_f32_rows<EPI_RESID>(A, W, e, M, N, K, num_cus, stream); break;
        case EPI_F32: launch_f32_rows<EPI_F32>(A, W, e, M, N, K, num_cus, stream); break;
        default: launch_f32_rows<EPI_SWIGLU>(A, W, e, M, N, K, num_cus, stream); break;
      }
      LLMLAB_LAUNCH_CHECK("linear(float32, few rows)");
      return 0;
    }
    switch (epilogue) {
      case EPI_STORE: launch_f32_tiled<EPI_STORE>(A, W, e, M, N, K, num_cus, stream); break;
      case EPI_RESID: launch_f32_tiled<EPI_RESID>(A, W, e, M, N, K, num_cus, stream); break;
      case EPI_F32: launch_f32_tiled<EPI_F32>(A, W, e, M, N, K, num_cus, stream); break;
      default: launch_f32_tiled<EPI_SWIGLU>(A, W, e, M, N, K, num_cus, stream); break;
    }
  }
  LLMLAB_LAUNCH_CHECK("linear");
  return 0;
}
