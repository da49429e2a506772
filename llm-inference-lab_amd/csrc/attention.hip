// Grouped-query attention over the paged cache, for one head size (HEAD_DIM is
// given on the compiler's command line; the library is built once per head size
// that a model needs).  gfx950 only.
//
// Cache of one layer: per page and kv head P keys of D numbers and as many values,
// each in the order of this kernel's MFMA fragments (kcache_index / vcache_index in
// common.h): a 16-key block is 16 D consecutive numbers, and every fragment load of
// a wave is lane-contiguous.  Position p of the b-th request of the step lives in
// page table[b][p / P] at offset p % P (P a power of two, at least 16).  The query at position p sees the keys lo..p, lo = max(0, p -
// window + 1) with a window and 0 without.
//
// bfloat16 kernel (matrix cores).  A tile is 16*QB "rows", a row being a (token,
// head of the group) pair of one request and one kv head, so the heads that share
// a kv head share its key and value fragments.  Everything is computed
// transposed so that no data has to move between lanes:
//   S^T[key, row]  = K . Q^T     A = key fragment (16 keys x 32 d), B = query fragment
//   O^T[d,  row]   = V^T . P^T   A = value fragment (16 d x 32 keys), B = probabilities
// The result layout of S^T (lane: column = row l%16, keys 4*(l/16)+i of each
// 16-key block) is exactly the B layout of the second product once the 32 keys
// of a step are taken in the order {4g..4g+3 of block 0, 4g..4g+3 of block 1} for
// lane group g; the value fragment is loaded in that same order.  Scores, the
// running maximum, the exponentials and the sums are float32; the softmax works in
// base 2 (scores pre-multiplied by log2 e).
//
// Decode (at most 16 rows per request and kv head): the waves of a block split the
// block's keys and merge their unnormalised sums, maxima and denominators through
// LDS; blockIdx.y also counts splits of the key range over blocks.  Each such block
// writes its merged partial result, and a second kernel merges the splits in their
// order:  out = sum_s w_s acc_s / sum_s w_s l_s,  w_s = 2^(m_s - m).
//
// float32 kernel: the same scheme on the float32 matrix instruction (true 32-bit
// products and sums), in steps of 16 keys.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256,
              "head sizes are multiples of 16 up to 256");

constexpr int D = HEAD_DIM;
constexpr float NEG_INF = -__builtin_huge_valf();

// 2^x for x <= 0 by the hardware instruction (one ulp; results below 2^-126 become 0,
// which is what a softmax wants of them)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Stores and loads of device scope: the value goes through the L2 of this die to memory
// (and comes from there), so that blocks on different dies, each behind an L2 of its own,
// can hand results to each other within one kernel without flushing those caches.
__device__ __forceinline__ void store_device(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_device(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Maxima across the four lanes that hold the keys of one row, by the lane-swap
// instructions of gfx950 instead of LDS permutes.  (No inline assembly for the
// maxima themselves: the compiler does not see the wait states an MFMA result needs
// before a hand-written instruction reads it.)
__device__ __forceinline__ float max_raw(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ float max3_raw(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }
__device__ __forceinline__ float max_across_32(float v) {      // with lane l ^ 32
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return max_raw(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_across_16(float v) {      // with lane l ^ 16
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return max_raw(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
constexpr float LAZY_MAX = 8.f;    // see compute(): slack of the running maximum, in powers of two

struct AttnArgs {
  const void* q;      // [rows, q_stride], head h at h*D
  const void* kc;     // this layer's key pages
  const void* vc;     // this layer's value pages
  const int* table;   // [reqs, table_stride]
  const int* q_start; // [reqs + 1]
  const int* start_pos;  // [reqs]
  void* out;          // [rows, out_stride]
  float* o_part;      // [rows*nq, splits, D]      (splits > 1)
  float* ml_part;     // [rows*nq, splits, 2]
  int* arrived;       // [reqs * nkv] counters, zero between launches: the split blocks of a
                      // (request, kv head) count themselves here and the last one merges
                      // (null: a kernel of its own merges)
  int q_stride, out_stride, table_stride, page_size;
  int nq, nkv, window, splits;
  int page_shift;     // log2(page_size); page sizes are powers of two
  int tiles;          // paired kernel: tiles of rows per request (blocks take two each)
  int qlen_lo, qlen_hi;  // only requests that bring so many tokens are worked on (a step may be
                         // served by two launches: its short requests by one, its long ones by the other)
  float scale;
};

// ------------------------------------------------------------- bf16, MFMA
// The fragments of one step of 32 keys: two blocks of 16 keys, and the values of
// those keys for every 16-wide block of d.
template <int DC, int DB>
struct KeyStep {
  bf16x8 k[2][DC];
  bf16x4 v[2][DB];
  bool ok[2];
};

// DECODE = false: every wave owns a tile of 16*QB rows and walks all its keys.
// DECODE = true (QB = 1, at most 16 rows per request and kv head): the waves of a
// block share one tile and split the block's keys; they merge through LDS, and
// blocks that split the keys further merge through global memory (see below).
constexpr int DECODE_WAVES = D <= 64 ? 8 : (D <= 128 ? 4 : 2);
#ifndef MAX_KEY_SPLITS
#define MAX_KEY_SPLITS 128
#endif

// RING (decode only): key steps a wave keeps in flight; 1 when a wave has one or two
// steps at all (nothing to run ahead of), 2 for longer shares (deeper rings measured
// no faster).
// PH (prefill only): the block has PH groups of four waves; group ph takes the ph-th 64 keys
// of every 64*PH the block stages, and the groups' sums meet in LDS at the end.  Two
// groups double the waves of a launch whose tiles of rows would leave a SIMD with one
// wave or none: a wave's step is a chain (LDS, scores, maximum, exponentials, products)
// that only another wave can fill.
// LDS of the decode branch (the waves' sums, their maxima and denominators, the flag of the block
// that arrives last, the splits' maxima where they do not fit in the sums' place): the kernel
// declares it and hands it in, so that a kernel that runs two kinds of blocks has it once.
template <int QB>
constexpr int decode_lds_floats() {
  return 2 * DECODE_WAVES * 16 * QB + DECODE_WAVES * 16 * QB * D + 4 +
         (((size_t)DECODE_WAVES * 16 * D >= (size_t)2 * 16 * MAX_KEY_SPLITS) ? 0 : 2 * 16 * MAX_KEY_SPLITS);
}

// `xblk`, `by`, `bz`: the block's tile of rows, its (kv head, split) and its request (a kernel of
// one kind of blocks passes its block indices).
template <int QB, bool DECODE, int RING, int PH = 1>
__device__ __forceinline__ void attention_tile(const AttnArgs& a, const int xblk, const int by, const int bz,
                                               float* dlds) {
  constexpr int DC = (D + 31) / 32;  // 32-wide chunks of d for Q.K
  constexpr int DB = D / 16;         // 16-wide blocks of d for P.V
  constexpr bool PIPE = DECODE;
  const int lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same for all lanes: kept scalar
  const int c = lane & 15, g = lane >> 4;
  const int b = bz;
  const int kvh = by / a.splits, split = by % a.splits;
  const int G = a.nq / a.nkv;
  const int r0 = a.q_start[b], qlen = a.q_start[b + 1] - r0, sp = a.start_pos[b];
  const int rows_total = qlen * G;
  const int nwr = DECODE ? 1 : nw / PH;          // prefill: waves side by side along the rows
  const int ph = DECODE ? 0 : wave / nwr;        // ... and this wave's group
  const int row0 = DECODE ? xblk * (16 * QB) : (xblk * nwr + wave % nwr) * (16 * QB);
  if ((DECODE ? row0 : xblk * nwr * (16 * QB)) >= rows_total) return;   // the whole block is past the rows
  if (qlen < a.qlen_lo || qlen > a.qlen_hi) return;                     // another launch's request
  const bool wave_live = row0 < rows_total;      // a wave without rows still helps to stage keys
  const bf16_t* q = (const bf16_t*)a.q;
  const bf16_t* kc = (const bf16_t*)a.kc;
  const bf16_t* vc = (const bf16_t*)a.vc;
  const int P = a.page_size;
  const int pshift = a.page_shift;
  auto page_index = [&](int pos) { return pos >> pshift; };
  auto page_offset = [&](int pos) { return pos & (P - 1); };
  const float scale2 = a.scale * 1.4426950408889634f;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16x4 zero4 = {0, 0, 0, 0};

  // this lane's row in each 16-row block
  bool valid[QB];
  int tok[QB], head[QB], pos[QB], lo[QB];
  bf16x8 qf[QB][DC];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int rr = row0 + qb * 16 + c;
    valid[qb] = wave_live && rr < rows_total;
    tok[qb] = valid[qb] ? rr / G : 0;
    head[qb] = kvh * G + (valid[qb] ? rr % G : 0);
    pos[qb] = sp + tok[qb];
    lo[qb] = a.window > 0 ? max(0, pos[qb] - a.window + 1) : 0;
    const bf16_t* qp = q + (size_t)(r0 + tok[qb]) * a.q_stride + (size_t)head[qb] * D;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      const int dd = dc * 32 + g * 8;
      qf[qb][dc] = (valid[qb] && dd < D) ? *(const bf16x8*)(qp + dd) : zero8;
    }
  }

  // keys this tile can see, and this split's share of them in steps of 32
  const int last_row = min(row0 + 16 * QB, rows_total) - 1;
  const int p_first = sp + row0 / G, p_last = sp + last_row / G;
  const int key_lo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int key_hi = wave_live ? p_last : -1;
  // every key >= full_lo is inside the window of every row of the tile
  const int full_lo = a.window > 0 ? max(0, p_last - a.window + 1) : 0;
  const int blk_lo = key_lo >> 5, blk_hi = key_hi >> 5;
  const int per = (blk_hi - blk_lo + 1 + a.splits - 1) / a.splits;
  int my_blk0 = blk_lo + split * per;
  int my_blk1 = min(my_blk0 + per, blk_hi + 1);
  if constexpr (DECODE) {
    // this wave's share of the block's steps
    const int per_wave = (max(my_blk1 - my_blk0, 0) + nw - 1) / nw;
    my_blk0 += wave * per_wave;
    my_blk1 = min(my_blk0 + per_wave, my_blk1);
  }

  floatx4 o[QB][DB];
  float m[QB], lsum[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m[qb] = NEG_INF;
    lsum[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) o[qb][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // One step of 32 keys for every row block of the tile.  The running maximum is
  // kept in the units of the exponent (score * scale * log2 e) and is only raised
  // when a score exceeds it by more than LAZY_MAX: until then p = 2^(s - m) may be as
  // large as 2^LAZY_MAX, which float32 sums and bfloat16 probabilities hold without
  // loss, and the rescaling of the sums (a pass over all of o) becomes rare.
  auto compute = [&](int blk, const KeyStep<DC, DB>& f) {
    const int kb = blk << 5;
    floatx4 s[2][QB];
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) s[h2][qb] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (f.ok[h2]) {
#pragma unroll
        for (int dc = 0; dc < DC; ++dc)
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            s[h2][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[h2][dc], qf[qb][dc], s[h2][qb], 0, 0, 0);
      }
    }
    // all 32 keys visible to every row of the tile (the common case below the diagonal
    // and inside the window): no comparisons, no infinities
    const bool all_visible = f.ok[0] && f.ok[1] && kb + 31 <= p_first && kb >= full_lo;
    bf16x8 pf[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float sv[8];
      if (all_visible) {
#pragma unroll
        for (int i = 0; i < 8; ++i) sv[i] = s[i >> 2][qb][i & 3];
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int h2 = i >> 2;
          const int j = kb + h2 * 16 + g * 4 + (i & 3);
          const bool vis = f.ok[h2] && valid[qb] && j <= pos[qb] && j >= lo[qb];
          sv[i] = vis ? s[h2][qb][i & 3] : NEG_INF;
        }
      }
      // into the units of the exponent (a product is a canonical number, so the maxima
      // below need no quieting of their inputs)
#pragma unroll
      for (int i = 0; i < 8; ++i) sv[i] *= scale2;
      float mx = max3_raw(max3_raw(sv[0], sv[1], sv[2]), max3_raw(sv[3], sv[4], sv[5]), max_raw(sv[6], sv[7]));
      mx = max_across_32(mx);
      mx = max_across_16(mx);
      const bool grow = mx > m[qb] + LAZY_MAX;
      if (__any(grow)) {            // some row's maximum grew: rescale what is summed so far
        const float m_new = grow ? mx : m[qb];
        const float alpha = grow ? fast_exp2(m[qb] - m_new) : 1.f;     // 2^-inf = 0 the first time
        lsum[qb] *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db) o[qb][db] *= alpha;
        m[qb] = m_new;
      }
      // no visible key yet (masked steps only): every p of the row is 2^-inf = 0
      const float neg_m = (!all_visible && m[qb] == NEG_INF) ? 0.f : -m[qb];
      float pv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) pv[i] = fast_exp2(sv[i] + neg_m);
      lsum[qb] += ((pv[0] + pv[1]) + (pv[2] + pv[3])) + ((pv[4] + pv[5]) + (pv[6] + pv[7]));
#pragma unroll
      for (int i = 0; i < 8; ++i) pf[qb][i] = (bf16_t)pv[i];
    }
    // keys past the last written position hold stale values: keep them out of
    // the product even though their probability is zero
    const bool tail = kb + 31 > key_hi;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x8 vf = __builtin_shufflevector(f.v[0][db], f.v[1][db], 0, 1, 2, 3, 4, 5, 6, 7);
      if (tail) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int j = kb + (i >> 2) * 16 + g * 4 + (i & 3);
          if (j > key_hi) vf[i] = (bf16_t)0.f;
        }
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
        o[qb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[qb], o[qb][db], 0, 0, 0);
    }
  };

  // prefill: the keys and values of a staged tile (64 keys for each group of waves)
  static_assert(PH == 1 || PH == 2, "one or two groups of waves");
  constexpr int KT = 64 * PH;
  constexpr int STAGES = PH;                   // of keys and values in LDS
  __shared__ __attribute__((aligned(16))) bf16_t kv_lds[DECODE ? 8 : STAGES * 2 * KT * D];
  if constexpr (PIPE) {
    // The loads of the next steps are in flight while this one is computed.  Every
    // load in the loop is unconditional (a load under a branch makes the compiler
    // wait for all loads in flight where the branch ends, and the ring stalls): a
    // step past the end reads the last step again, a missing page reads page 0, and
    // the flags keep what was read out of the sums.  The page numbers of up to 32
    // steps are read ahead of the loop, one 16-key group per lane.
    KeyStep<DC, DB> ring[RING];
    for (int cb = my_blk0; cb < my_blk1; cb += 32) {
      const int ce = min(cb + 32, my_blk1);
      int pages_v;
      {
        const int pos16 = (cb * 2 + lane) * 16;
        const bool in = cb * 2 + lane < ce * 2 && pos16 <= key_hi && pos16 + 15 >= key_lo;
        const int pg = a.table[(size_t)b * a.table_stride + min(page_index(pos16), a.table_stride - 1)];
        pages_v = in ? pg : -1;
      }
      auto fetch = [&](int blk, KeyStep<DC, DB>& f) {
        const int bl = min(blk, ce - 1);
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const int page = __builtin_amdgcn_readlane(pages_v, (bl - cb) * 2 + h2);
          const bool ok = blk < ce && page >= 0;
          f.ok[h2] = ok;
          // the 16-key block of the page: its keys and its values are 16 D numbers each,
          // in fragment order (see common.h), so every load below is lane-contiguous
          const size_t blk16 = ((size_t)max(page, 0) * a.nkv + kvh) * P * D +
                               (size_t)(page_offset(bl * 32 + h2 * 16) >> 4) * (16 * D);
          const bf16_t* kp = kc + blk16 + c * 8;
          const bf16_t* vp = vc + blk16 + lane * 4;
#pragma unroll
          for (int dc = 0; dc < DC; ++dc)     // a piece past D meets zeros of the query fragment
            f.k[h2][dc] = *(const bf16x8*)(kp + min(dc * 4 + g, D / 8 - 1) * 128);
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const bf16x4 v = *(const bf16x4*)(vp + db * 256);
            f.v[h2][db] = ok ? v : zero4;
          }
        }
      };
#pragma unroll
      for (int p = 0; p < RING; ++p) fetch(cb + p, ring[p]);
      int blk0 = cb;
      for (; blk0 + RING < ce; blk0 += RING) {      // rounds that refill the ring
#pragma unroll
        for (int p = 0; p < RING; ++p) {
          const KeyStep<DC, DB> cur = ring[p];
          fetch(blk0 + p + RING, ring[p]);
          __builtin_amdgcn_sched_barrier(0);
          compute(blk0 + p, cur);
        }
      }
#pragma unroll
      for (int p = 0; p < RING; ++p)               // the last round drains it
        if (blk0 + p < ce) compute(blk0 + p, ring[p]);
    }
  } else {
    // ---- prefill: tiles of 64 keys go through LDS once per block and serve all its
    // waves; the next tile is fetched into registers while this one is multiplied
    constexpr int NCH = D / 16;                     // 16-byte pieces per thread and tile (64 threads per 16 keys)
    constexpr int NT = 256 * PH;                    // threads of the block
    constexpr int KT_SHIFT = PH == 1 ? 6 : 7;
    // the tile's 16-key blocks as they lie in the cache (fragment order): the
    // copy is straight, and every fragment read below is lane-contiguous
    // With two groups of waves two stages, the tile after this one being put in while this
    // one is multiplied: one barrier per tile, and the copy of one wave passes behind the
    // arithmetic of the others (a block of eight waves is alone on its compute unit; two
    // blocks of four fill each other's waits, and measured no faster with two stages).
    auto ks_of = [&](int stage) { return kv_lds + stage * (2 * KT * D); };
    auto vs_of = [&](int stage) { return kv_lds + stage * (2 * KT * D) + KT * D; };
    // The values lie in LDS so that one 16-byte read gives a lane its MFMA operand of a
    // step of 32 keys: [pair of 16-key blocks][16-wide block of d][lane][even block's 4 |
    // odd block's 4].  A 16-byte piece as it comes from the cache (two lanes' values of
    // one 16-key block) goes there in two halves.
    auto vs_at = [&](int sub, int db, int ln) { return (((sub >> 1) * DB + db) * 64 + ln) * 8 + (sub & 1) * 4; };
    auto vs_store = [&](bf16_t* Vs, int sub, int rem, const bf16x8& v) {     // piece `rem` of 16-key block `sub`
      bf16_t* dst = Vs + vs_at(sub, rem >> 5, (rem & 31) * 2);
      *(bf16x4*)dst = __builtin_shufflevector(v, v, 0, 1, 2, 3);
      *(bf16x4*)(dst + 8) = __builtin_shufflevector(v, v, 4, 5, 6, 7);
    };
    __shared__ int s_ok_all[STAGES][4 * PH];
    constexpr int PAGE_CAP = 2048;
    __shared__ int s_pages[PAGE_CAP + 1];           // the block's slice of its request's block table (a slice that starts inside a page touches one more)
    const int tid = threadIdx.x;
    const int blk_row0 = xblk * nwr * (16 * QB);
    const int blk_last = min(blk_row0 + nwr * 16 * QB, rows_total) - 1;
    const int bkey_hi = sp + blk_last / G;
    const int bkey_lo = a.window > 0 ? max(0, sp + blk_row0 / G - a.window + 1) : 0;
    // PD tiles are on their way from memory at any time (a ring of register buffers):
    // one tile's arithmetic is far shorter than the memory latency.  The loads of the
    // ring are unconditional (see the decode branch): a tile past the end reads the
    // last tile again, a missing page reads page 0, and the flag zeroes what came.
    constexpr int PD = NCH <= 4 ? 3 : 2;
    bf16x8 regs[PD][NCH];
    bool rok[PD][NCH];
    const int tile_lo = bkey_lo >> KT_SHIFT, tile_hi = bkey_hi >> KT_SHIFT;
    // The page numbers come from LDS, PAGE_CAP pages at a time (one slice is enough
    // for any common context), so that a tile costs one memory round trip, not two.
    const int tiles_per_slice = (PAGE_CAP << pshift) >> KT_SHIFT;
    for (int ct = tile_lo; ct <= tile_hi; ct += tiles_per_slice) {
      const int ce = min(ct + tiles_per_slice - 1, tile_hi);
      const int page_first = page_index(ct * KT);
      const int page_count = page_index(ce * KT + KT - 1) - page_first + 1;
      __syncthreads();
      for (int i = tid; i < page_count; i += NT) {
        const int pi = page_first + i;
        s_pages[i] = pi < a.table_stride ? a.table[(size_t)b * a.table_stride + pi] : -1;
      }
      __syncthreads();
      // (a block of 4 waves and head sizes in steps of 32: a 16-key block is 2 D pieces
      // of 16 bytes, a whole number of pieces per lane)
      constexpr bool FAST_PIECES = D % 32 == 0;
      auto fetch_tile = [&](int slot, int tile) {
        const int tl = min(tile, ce);
        if constexpr (FAST_PIECES) {
          // wave w copies the w-th 16-key block of the tile, keys and values: one page
          // lookup and one address for all pieces of a thread
          const int pos16 = tl * KT + wave * 16;
          const int page = s_pages[page_index(pos16) - page_first];
          const bool ok = tile <= ce && pos16 <= bkey_hi && pos16 + 15 >= bkey_lo && page >= 0;
          const size_t at = ((size_t)max(page, 0) * a.nkv + kvh) * P * D +
                            (size_t)(page_offset(pos16) >> 4) * (16 * D) + lane * 8;
#pragma unroll
          for (int n = 0; n < NCH / 2; ++n) {
            rok[slot][n] = rok[slot][n + NCH / 2] = ok;
            regs[slot][n] = *(const bf16x8*)(kc + at + n * 512);
            regs[slot][n + NCH / 2] = *(const bf16x8*)(vc + at + n * 512);
          }
          return;
        }
#pragma unroll
        for (int n = 0; n < NCH; ++n) {
          const int i = tid + n * NT;
          const bool is_v = i >= 8 * D * PH;
          const int j = is_v ? i - 8 * D * PH : i;
          const int sub = j / (2 * D), rem = j - sub * (2 * D);
          const int pos16 = tl * KT + sub * 16;
          const int page = s_pages[page_index(pos16) - page_first];
          rok[slot][n] = tile <= ce && pos16 <= bkey_hi && pos16 + 15 >= bkey_lo && page >= 0;
          const size_t blk16 = ((size_t)max(page, 0) * a.nkv + kvh) * P * D +
                               (size_t)(page_offset(pos16) >> 4) * (16 * D);
          regs[slot][n] = *(const bf16x8*)((is_v ? vc : kc) + blk16 + rem * 8);
        }
      };
      auto store_tile = [&](int slot, int stage) {
        bf16_t* Ks = ks_of(stage);
        bf16_t* Vs = vs_of(stage);
        int* s_ok = s_ok_all[stage];
        if constexpr (FAST_PIECES) {
#pragma unroll
          for (int n = 0; n < NCH / 2; ++n) {
            // (what came for a 16-key block that is not there goes in as it is: s_ok keeps
            // the keys out of the scores, and the values are zeroed where they are read)
            *(bf16x8*)(Ks + wave * (16 * D) + (lane + n * 64) * 8) = regs[slot][n];
            vs_store(Vs, wave, lane + n * 64, regs[slot][n + NCH / 2]);
          }
          if (lane == 0) s_ok[wave] = rok[slot][0];
          return;
        }
#pragma unroll
        for (int n = 0; n < NCH; ++n) {
          const int i = tid + n * NT;
          const bool is_v = i >= 8 * D * PH;
          const int j = is_v ? i - 8 * D * PH : i;
          const int sub = j / (2 * D), rem = j - sub * (2 * D);
          const bf16x8 v = rok[slot][n] ? regs[slot][n] : zero8;
          if (is_v) vs_store(Vs, sub, rem, v);
          else *(bf16x8*)(Ks + sub * (16 * D) + rem * 8) = v;
          if (!is_v && rem == 0) s_ok[sub] = rok[slot][n];
        }
      };
#pragma unroll
      for (int p = 0; p < PD; ++p) fetch_tile(p, ct + p);
      // two stages: tile t lies in stage t & 1; it is put there during tile t - 1 (the first one: now)
      if constexpr (STAGES == 2) {
        store_tile(0, ct & 1);
        fetch_tile(0, ct + PD);
        __syncthreads();
      }
      for (int tile0 = ct; tile0 <= ce; tile0 += PD) {
#pragma unroll
        for (int p = 0; p < PD; ++p) {
          const int tile = tile0 + p;
          const bool live = tile <= ce;
          const int stage = STAGES == 2 ? (tile & 1) : 0;
          if constexpr (STAGES == 2) {
            const int pn = (p + 1) % PD;              // ring slot of the next tile (a constant once unrolled)
            if (tile + 1 <= ce) store_tile(pn, stage ^ 1);
            fetch_tile(pn, tile + 1 + PD);
          } else {
            if (live) {
              store_tile(p, 0);
              __syncthreads();
            }
            fetch_tile(p, tile + PD);
          }
          __builtin_amdgcn_sched_barrier(0);
          const bf16_t* Ks = ks_of(stage);
          const bf16_t* Vs = vs_of(stage);
          const int* s_ok = s_ok_all[stage];
          const int kb0 = tile * KT + ph * 64;      // this group's 64 keys of the tile
          const int sub0 = ph * 4;                  // ... and their first 16-key block in LDS
          // 64 keys below the diagonal of all rows of the wave and inside their windows,
          // with all their pages there: in one piece, without comparisons
          const bool interior = live && wave_live && kb0 + 63 <= p_first && kb0 >= full_lo &&
                                (s_ok[sub0] & s_ok[sub0 + 1] & s_ok[sub0 + 2] & s_ok[sub0 + 3]) != 0;
          if (interior) {
            // with one row block the whole tile of 64 keys at once, with two in halves of
            // 32 (registers): scores of the piece, one maximum, exponentials, products
            constexpr int SUBS = (QB == 1 && D <= 64) ? 4 : 2;        // 16-key blocks per piece
#pragma unroll
            for (int piece = 0; piece < 4 / SUBS; ++piece) {
              bf16x8 kf[SUBS][DC];
              bf16x8 vf[SUBS / 2][DB];
#pragma unroll
              for (int u = 0; u < SUBS; ++u) {
                const int sub = sub0 + piece * SUBS + u;
#pragma unroll
                for (int dc = 0; dc < DC; ++dc)
                  kf[u][dc] = *(const bf16x8*)(Ks + sub * (16 * D) + min(dc * 4 + g, D / 8 - 1) * 128 + c * 8);
              }
              // the values of a step of 32 keys (two 16-key blocks): one read per operand
#pragma unroll
              for (int st = 0; st < SUBS / 2; ++st)
#pragma unroll
                for (int db = 0; db < DB; ++db)
                  vf[st][db] = *(const bf16x8*)(Vs + vs_at(sub0 + piece * SUBS + st * 2, db, lane));
              floatx4 s4[SUBS][QB];
#pragma unroll
              for (int u = 0; u < SUBS; ++u)
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                  s4[u][qb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                  for (int dc = 0; dc < DC; ++dc)
                    s4[u][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][dc], qf[qb][dc], s4[u][qb], 0, 0, 0);
                }
              bf16x8 pf[SUBS / 2][QB];
#pragma unroll
              for (int qb = 0; qb < QB; ++qb) {
                // the maximum of the raw scores, then into the units of the exponent (the
                // scale is positive); the scores themselves are scaled inside the FMA below
                float mx = NEG_INF;
#pragma unroll
                for (int u = 0; u < SUBS; ++u)
                  mx = max3_raw(max3_raw(s4[u][qb][0], s4[u][qb][1], s4[u][qb][2]), s4[u][qb][3], mx);
                mx = max_across_32(mx);
                mx = max_across_16(mx);
                mx *= scale2;
                const bool grow = mx > m[qb] + LAZY_MAX;
                if (__any(grow)) {
                  const float m_new = grow ? mx : m[qb];
                  const float alpha = grow ? fast_exp2(m[qb] - m_new) : 1.f;
                  lsum[qb] *= alpha;
#pragma unroll
                  for (int db = 0; db < DB; ++db) o[qb][db] *= alpha;
                  m[qb] = m_new;
                }
                const float neg_m = -m[qb];
                float psum = 0.f;
#pragma unroll
                for (int st = 0; st < SUBS / 2; ++st) {
                  float pv[8];
#pragma unroll
                  for (int i = 0; i < 8; ++i)
                    pv[i] = fast_exp2(fmaf(s4[st * 2 + (i >> 2)][qb][i & 3], scale2, neg_m));
                  psum += ((pv[0] + pv[1]) + (pv[2] + pv[3])) + ((pv[4] + pv[5]) + (pv[6] + pv[7]));
#pragma unroll
                  for (int i = 0; i < 8; ++i) pf[st][qb][i] = (bf16_t)pv[i];
                }
                lsum[qb] += psum;
              }
#pragma unroll
              for (int st = 0; st < SUBS / 2; ++st)
#pragma unroll
                for (int db = 0; db < DB; ++db) {
#pragma unroll
                  for (int qb = 0; qb < QB; ++qb)
                    o[qb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[st][db], pf[st][qb], o[qb][db], 0, 0, 0);
                }
            }
            __syncthreads();
          } else if (live) {
#pragma unroll
            for (int st = 0; st < 2; ++st) {
              const int kb = kb0 + st * 32;
              if (kb <= key_hi && kb + 31 >= key_lo) {        // this wave sees some of these keys
                KeyStep<DC, DB> f;
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                  const int sub = sub0 + st * 2 + h2;
                  f.ok[h2] = s_ok[sub] != 0;
#pragma unroll
                  for (int dc = 0; dc < DC; ++dc)
                    f.k[h2][dc] = *(const bf16x8*)(Ks + sub * (16 * D) + min(dc * 4 + g, D / 8 - 1) * 128 + c * 8);
#pragma unroll
                  for (int db = 0; db < DB; ++db)
                    f.v[h2][db] = f.ok[h2] ? *(const bf16x4*)(Vs + vs_at(sub, db, lane)) : zero4;
                }
                compute(kb >> 5, f);
              }
            }
            __syncthreads();
          }
        }
      }
    }
  }

  if constexpr (!DECODE && PH > 1) {
    // The second group hands its sums to the first, lane to lane (both hold the same rows in
    // the same places); the staged keys are done with after the last tile's barrier.
    //   o = 2^(m0 - m) o0 + 2^(m1 - m) o1,  l likewise,  m = max(m0, m1)
    float* xo = (float*)kv_lds;                        // [row tile][qb][db][lane][4]
    __shared__ float x_m[4][QB][64], x_l[4][QB][64];
    const int rt = wave % nwr;
    if (ph == 1) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        x_m[rt][qb][lane] = m[qb];
        x_l[rt][qb][lane] = lsum[qb];
#pragma unroll
        for (int db = 0; db < DB; ++db) *(floatx4*)(xo + (((rt * QB + qb) * DB + db) * 64 + lane) * 4) = o[qb][db];
      }
    }
    __syncthreads();
    if (ph != 0) return;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float m1 = x_m[rt][qb][lane], m_new = fmaxf(m[qb], m1);
      const float a0 = m[qb] == NEG_INF ? 0.f : fast_exp2(m[qb] - m_new);
      const float a1 = m1 == NEG_INF ? 0.f : fast_exp2(m1 - m_new);
      lsum[qb] = lsum[qb] * a0 + x_l[rt][qb][lane] * a1;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const floatx4 o1 = *(const floatx4*)(xo + (((rt * QB + qb) * DB + db) * 64 + lane) * 4);
        o[qb][db] = o[qb][db] * a0 + o1 * a1;
      }
    }
  }
  if constexpr (!DECODE) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float l = lsum[qb];
      l += __shfl_xor(l, 16, WAVE);
      l += __shfl_xor(l, 32, WAVE);
      if (!valid[qb]) continue;
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16_t* dst = (bf16_t*)a.out + (size_t)(r0 + tok[qb]) * a.out_stride + (size_t)head[qb] * D;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        bf16x4 w = {(bf16_t)(o[qb][db][0] * inv), (bf16_t)(o[qb][db][1] * inv),
                    (bf16_t)(o[qb][db][2] * inv), (bf16_t)(o[qb][db][3] * inv)};
        *(bf16x4*)(dst + db * 16 + g * 4) = w;
      }
    }
  } else {
    // ---- merge the waves of the block through LDS
    //   acc = sum_w 2^(m_w - m) acc_w,  l = sum_w 2^(m_w - m) l_w,  m = max_w m_w
    float (*s_m)[16 * QB] = reinterpret_cast<float (*)[16 * QB]>(dlds);
    float (*s_l)[16 * QB] = reinterpret_cast<float (*)[16 * QB]>(dlds + DECODE_WAVES * 16 * QB);
    float (*s_o)[16 * QB][D] = reinterpret_cast<float (*)[16 * QB][D]>(dlds + 2 * DECODE_WAVES * 16 * QB);   // (16-byte aligned)
    float* const after_sums = dlds + 2 * DECODE_WAVES * 16 * QB + DECODE_WAVES * 16 * QB * D;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float l = lsum[qb];
      l += __shfl_xor(l, 16, WAVE);
      l += __shfl_xor(l, 32, WAVE);
      if (g == 0) {
        s_m[wave][qb * 16 + c] = m[qb];               // already in the units of the exponent
        s_l[wave][qb * 16 + c] = l;
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) *(floatx4*)(&s_o[wave][qb * 16 + c][db * 16 + g * 4]) = o[qb][db];
    }
    __syncthreads();
    const int nrows = min(16 * QB, rows_total - row0);
    // sum the `count` entries of s_m / s_l / s_o in their order; write the result
    // (final: normalised, to `out`; else: as this block's partial result)
    auto merge = [&](int count, bool final) {
      for (int idx = threadIdx.x; idx < nrows * D; idx += blockDim.x) {
        const int r = idx / D, dd = idx - r * D;
        float mmax = NEG_INF;
        for (int w = 0; w < count; ++w) mmax = fmaxf(mmax, s_m[w][r]);
        float num = 0.f, den = 0.f;
        for (int w = 0; w < count; ++w) {
          const float wt = s_m[w][r] == NEG_INF ? 0.f : exp2f(s_m[w][r] - mmax);
          num += wt * s_o[w][r][dd];
          den += wt * s_l[w][r];
        }
        const int t = (row0 + r) / G, hh = kvh * G + (row0 + r) % G;
        if (final) {
          ((bf16_t*)a.out)[(size_t)(r0 + t) * a.out_stride + (size_t)hh * D + dd] =
              (bf16_t)(den > 0.f ? num / den : 0.f);
        } else {
          // (stores of device scope: written through to memory, where a block on another
          // die finds them without a fence; see below)
          const size_t at = ((size_t)(r0 + t) * a.nq + hh) * a.splits + split;
          store_device(&a.o_part[at * D + dd], num);
          if (dd == 0) {
            store_device(&a.ml_part[at * 2], mmax);
            store_device(&a.ml_part[at * 2 + 1], den);
          }
        }
      }
    };
    merge(nw, a.splits == 1);
    if constexpr (QB == 1) {        // (tiles of more rows are never split over blocks)
    if (a.splits == 1 || a.arrived == nullptr) return;
    // ---- the block that arrives last merges the splits of its (request, kv head):
    //   out = sum_s w_s acc_s / sum_s w_s l_s,  w_s = 2^(m_s - max m)
    // No fence: a fence of device scope writes back and invalidates the whole L2 of the
    // die, which costs more than the kernel it saves.  Instead the partial results are
    // stored and loaded with device scope (they pass the L2 of the die by), every thread
    // waits until its stores are done, the block meets at a barrier, and then one thread
    // counts the block in with an atomic of device scope.  Whoever reads splits - 1 there
    // knows that all other blocks' results are in memory.  It sets the counter back to
    // zero for the next launch.  Nobody waits for anybody: a block that is not the last
    // simply ends.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    int& s_last = *reinterpret_cast<int*>(after_sums);
    if (threadIdx.x == 0) {
      int* counter = a.arrived + (size_t)b * a.nkv + kvh;
      const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = before == a.splits - 1;
      if (s_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    // maxima and denominators of all splits of the block's rows, through LDS: [row][split];
    // where the waves' own sums (done with behind the barriers above) leave room, in their place
    constexpr bool FITS = (size_t)DECODE_WAVES * 16 * D >= (size_t)2 * 16 * MAX_KEY_SPLITS;
    float* x_m = FITS ? &s_o[0][0][0] : after_sums + 4;
    float* x_l = x_m + 16 * MAX_KEY_SPLITS;
    const int S = a.splits;
    for (int i = threadIdx.x; i < nrows * S; i += blockDim.x) {
      const int r = i / S, sidx = i - r * S;
      const int t = (row0 + r) / G, hh = kvh * G + (row0 + r) % G;
      const size_t at = ((size_t)(r0 + t) * a.nq + hh) * S + sidx;
      x_m[r * S + sidx] = load_device(&a.ml_part[at * 2]);
      x_l[r * S + sidx] = load_device(&a.ml_part[at * 2 + 1]);
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < nrows * D; idx += blockDim.x) {
      const int r = idx / D, dd = idx - r * D;
      const int t = (row0 + r) / G, hh = kvh * G + (row0 + r) % G;
      const float* part = a.o_part + ((size_t)(r0 + t) * a.nq + hh) * S * D + dd;
      float mmax = NEG_INF;
      for (int u = 0; u < S; ++u) mmax = fmaxf(mmax, x_m[r * S + u]);
      float num = 0.f, den = 0.f;
      for (int u0 = 0; u0 < S; u0 += 8) {           // eight loads on their way at a time, summed in order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = load_device(part + (size_t)min(u0 + u, S - 1) * D);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (u0 + u >= S) break;
          const float mu = x_m[r * S + u0 + u];
          const float wt = mu == NEG_INF ? 0.f : exp2f(mu - mmax);
          num += wt * v[u];
          den += wt * x_l[r * S + u0 + u];
        }
      }
      ((bf16_t*)a.out)[(size_t)(r0 + t) * a.out_stride + (size_t)hh * D + dd] =
          (bf16_t)(den > 0.f ? num / den : 0.f);
    }
    }
  }
}

// One tile of rows per block; the blocks with the longest histories (the last rows)
// are dispatched first.
template <int QB, bool DECODE, int RING = 1, int PH = 1>
__global__ __launch_bounds__(DECODE ? 64 * DECODE_WAVES : 256 * PH, (!DECODE && D <= 64 && PH == 1) ? 2 : 1) void attention_bf16_kernel(AttnArgs a) {
  if constexpr (DECODE) {
    __shared__ __attribute__((aligned(16))) float dlds[decode_lds_floats<QB>()];
    attention_tile<QB, DECODE, RING, PH>(a, (int)(gridDim.x - 1 - blockIdx.x), (int)blockIdx.y, (int)blockIdx.z, dlds);
  } else {
    attention_tile<QB, DECODE, RING, PH>(a, (int)(gridDim.x - 1 - blockIdx.x), (int)blockIdx.y, (int)blockIdx.z, nullptr);
  }
}

// A mixed step in one launch: the first `long_blocks` blocks of a request (x) are the tiles of
// rows of a portion times the kv heads, each with the keys of its tile split over its waves; the
// others are the (kv head, split) pairs of a request of a few tokens, whose keys are split over
// blocks as in a decode step.  A block finds in its request's length which of the two it is
// for and ends at once if it is for the other kind.  In two launches the decoding requests'
// blocks, which stream their histories, wait for the portion's, which are a chain of small
// products, although they need different parts of a compute unit.
template <int QBL, int RL, int RS>
__global__ __launch_bounds__(64 * DECODE_WAVES) void attention_bf16_mixed_kernel(AttnArgs al, AttnArgs as, int long_tiles) {
  __shared__ __attribute__((aligned(16))) float dlds[decode_lds_floats<QBL>()];
  const int x = (int)blockIdx.x, long_blocks = long_tiles * al.nkv;
  if (x < long_blocks)
    attention_tile<QBL, true, RL>(al, long_tiles - 1 - x / al.nkv, x % al.nkv, (int)blockIdx.z, dlds);
  else
    attention_tile<1, true, RS>(as, 0, x - long_blocks, (int)blockIdx.z, dlds);
}

// Two tiles of rows per block, one after the other: tile t from the end and tile t
// from the start.  Under a causal mask their histories add up to the same length for
// every t, so all blocks of a prompt carry the same load; with one tile per block the
// last tiles' blocks run on while the units of the first ones idle.
template <int QB, int PH = 1>
__global__ __launch_bounds__(256 * PH, (D <= 64 && PH == 1) ? 2 : 1) void attention_bf16_paired_kernel(AttnArgs a) {
  const int late = a.tiles - 1 - (int)blockIdx.x, early = (int)blockIdx.x;
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1 && early >= late) break;
    attention_tile<QB, false, 1, PH>(a, pass == 0 ? late : early, (int)blockIdx.y, (int)blockIdx.z, nullptr);
    __syncthreads();
  }
}

// Merge of the key splits of a decode step, one block of four waves per (row, head):
//   out = sum_s w_s acc_s / sum_s w_s l_s,  w_s = 2^(m_s - max m).
// Every wave takes a quarter of the splits (lane = element of the head), has all of
// its partial sums on their way before the first is used (sixteen at a time: up to 64
// splits cost one trip to memory), and the quarters meet in LDS in their order.  Up to
// sixteen splits are one wave's work, and the block is launched with one.
// A kernel of its own for more than a few splits: within one kernel, results of blocks on
// other dies need either device-wide fences, which cost far more than a launch (measured:
// the last block to arrive, found by an atomic counter behind a fence, merging in place of
// this kernel made the decode step of 24 layers 1.88 ms instead of 0.97), or stores and
// loads of device scope, a chain of trips to memory that pays with few splits only (see
// launch_key_split_decode).
constexpr int MERGE_WAVES = 4;
template <typename T>
__global__ __launch_bounds__(64 * MERGE_WAVES) void attention_merge_kernel(
    const float* __restrict__ o_part, const float* __restrict__ ml_part, T* __restrict__ out,
    int out_stride, int nq, int splits, const int* __restrict__ row_req, const int* __restrict__ q_start,
    int qlen_hi) {
  constexpr int PER = (D + 63) / 64;
  __shared__ float s_num[MERGE_WAVES][PER * 64];
  const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (row_req) {      // rows of requests that another launch serves have no partial results
    const int b = row_req[row];
    if (q_start[b + 1] - q_start[b] > qlen_hi) return;
  }
  const size_t at0 = ((size_t)row * nq + head) * splits;
  // in every wave, lane l holds the maxima and sums of the splits l and l + 64
  float ms[2] = {NEG_INF, NEG_INF}, ls[2] = {0.f, 0.f};
#pragma unroll
  for (int h = 0; h < 2; ++h)
    if (h * 64 + lane < splits) {
      ms[h] = ml_part[(at0 + h * 64 + lane) * 2];
      ls[h] = ml_part[(at0 + h * 64 + lane) * 2 + 1];
    }
  const int nw = (int)blockDim.x >> 6;      // four waves, or one for sixteen splits or fewer
  const int quarter = (splits + nw - 1) / nw;
  const int u_lo = wave * quarter, u_hi = min(u_lo + quarter, splits);
  float num[PER];
#pragma unroll
  for (int p = 0; p < PER; ++p) num[p] = 0.f;
  float mmax = NEG_INF, w[2] = {0.f, 0.f};
  for (int u0 = u_lo; u0 < u_hi; u0 += 16) {
    float v[PER][16];
#pragma unroll
    for (int p = 0; p < PER; ++p)
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int dd = p * 64 + lane;
        v[p][u] = (u0 + u < u_hi && dd < D) ? o_part[(at0 + u0 + u) * D + dd] : 0.f;
      }
    if (u0 == u_lo) {     // the weights, while the first loads are under way
      mmax = wave_max(fmaxf(ms[0], ms[1]));
#pragma unroll
      for (int h = 0; h < 2; ++h) w[h] = ms[h] == NEG_INF ? 0.f : exp2f(ms[h] - mmax);
    }
#pragma unroll
    for (int p = 0; p < PER; ++p)
#pragma unroll
      for (int u = 0; u < 16; ++u) num[p] += __shfl(u0 + u < 64 ? w[0] : w[1], (u0 + u) & 63, WAVE) * v[p][u];
  }
#pragma unroll
  for (int p = 0; p < PER; ++p) s_num[wave][p * 64 + lane] = num[p];
  __syncthreads();
  if (wave != 0) return;
  const float den = wave_sum(w[0] * ls[0] + w[1] * ls[1]);
  const float inv = den > 0.f ? 1.f / den : 0.f;
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int dd = p * 64 + lane;
    float total = 0.f;
#pragma unroll
    for (int q = 0; q < nw; ++q) total += s_num[q][dd];
    if (dd < D) out[(size_t)row * out_stride + (size_t)head * D + dd] = (T)(total * inv);
  }
}

// ------------------------------------------------------------ float32
// True 32-bit arithmetic on the matrix cores: v_mfma_f32_16x16x4_f32 multiplies and sums
// in float32 (no reduced-precision mode).  Same transposed scheme as the bfloat16 kernel,
// in steps of 16 keys:
//   S^T[key, row] = K . Q^T    A = keys (16 keys x 4 d), B = queries (4 d x 16 rows)
//   O^T[d,  row]  = V^T . P^T  A = values (16 d x 4 keys), B = probabilities (4 keys x 16 rows)
// An instruction contracts over four slots, one per group g of sixteen lanes.  Which d (or
// key) sits in which slot is free as long as both operands agree, so lane (c, g) takes
// the four consecutive numbers 16 M + 4 g .. + 3 of its key c (one 16-byte load in the
// cache's order) and uses them in four instructions; for the second product the result
// layout of S^T (lane (c, g): row c, keys 4 g .. 4 g + 3) already is the B operand, and
// the values of keys 4 g .. 4 g + 3 at number c of a block of d are 16 consecutive bytes.
// Scores, maxima, exponentials and sums in float32.
//
// A tile is 16 QB rows ((token, head of the group) pairs of one request and kv head, so the
// heads of a group share the keys they read).  SPLIT = false: every wave owns a tile and
// walks all its keys (steps whose tiles fill the chip over few keys).  SPLIT = true: the NW
// waves of a block share one tile and split its keys, merge through LDS (all other steps of
// many rows), and blockIdx.y also counts splits over blocks whose partial results the merge
// kernel sums (decode steps).
template <int QB, bool SPLIT, int NW>
__global__ __launch_bounds__(64 * NW) void attention_f32_kernel(AttnArgs a) {
  constexpr int DQ = D / 16;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int b = blockIdx.z;
  const int kvh = blockIdx.y / a.splits, split = blockIdx.y % a.splits;
  const int G = a.nq / a.nkv;
  const int r0 = a.q_start[b], qlen = a.q_start[b + 1] - r0, sp = a.start_pos[b];
  const int rows_total = qlen * G;
  if (qlen < a.qlen_lo || qlen > a.qlen_hi) return;                  // another launch's request
  // tiles with the longest histories (the last rows) first
  const int xblk = (int)(gridDim.x - 1 - blockIdx.x);
  const int row0 = (SPLIT ? xblk : xblk * NW + wave) * (16 * QB);
  if (row0 >= rows_total) {
    if (!SPLIT || xblk * 16 * QB >= rows_total) return;              // (without SPLIT no wave waits for another)
  }
  const bool wave_live = row0 < rows_total;
  const float* q = (const float*)a.q;
  const float* kc = (const float*)a.kc;
  const float* vc = (const float*)a.vc;
  const int P = a.page_size, pshift = a.page_shift;
  const float scale2 = a.scale * 1.4426950408889634f;

  bool valid[QB];
  int tok[QB], head[QB], pos[QB], lo[QB];
  floatx4 qf[QB][DQ];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int rr = row0 + qb * 16 + c;
    valid[qb] = wave_live && rr < rows_total;
    tok[qb] = valid[qb] ? rr / G : 0;
    head[qb] = kvh * G + (valid[qb] ? rr % G : 0);
    pos[qb] = sp + tok[qb];
    lo[qb] = a.window > 0 ? max(0, pos[qb] - a.window + 1) : 0;
    const float* qp = q + (size_t)(r0 + tok[qb]) * a.q_stride + (size_t)head[qb] * D + g * 4;
#pragma unroll
    for (int mb = 0; mb < DQ; ++mb)
      qf[qb][mb] = valid[qb] ? *(const floatx4*)(qp + mb * 16) : floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const int last_row = min(row0 + 16 * QB, rows_total) - 1;
  const int p_first = sp + row0 / G, p_last = sp + last_row / G;
  const int key_lo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int key_hi = wave_live ? p_last : -1;
  const int full_lo = a.window > 0 ? max(0, p_last - a.window + 1) : 0;   // from here on inside every row's window
  const int blk_lo = key_lo >> 4, blk_hi = key_hi >> 4;
  const int per = (blk_hi - blk_lo + 1 + a.splits - 1) / a.splits;
  int my0 = blk_lo + split * per;
  int my1 = min(my0 + per, blk_hi + 1);
  if constexpr (SPLIT) {
    const int per_wave = (max(my1 - my0, 0) + NW - 1) / NW;
    my0 += wave * per_wave;
    my1 = min(my0 + per_wave, my1);
  }

  floatx4 o[QB][DQ];
  float m[QB], lsum[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m[qb] = NEG_INF;
    lsum[qb] = 0.f;
#pragma unroll
    for (int mb = 0; mb < DQ; ++mb) o[qb][mb] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  struct Step {
    floatx4 k[DQ], v[DQ];
    bool ok;
  };
  auto compute = [&](int blk, const Step& f) {
    if (!f.ok) return;                      // (the same for the whole wave)
    const int kb = blk << 4;
    const bool all_visible = kb + 15 <= p_first && kb >= full_lo;
    const bool tail = kb + 15 > key_hi;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      floatx4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int mb = 0; mb < DQ; ++mb)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          sc = __builtin_amdgcn_mfma_f32_16x16x4f32(f.k[mb][t], qf[qb][mb][t], sc, 0, 0, 0);
      // scores in units of the binary exponent (score * scale * log2 e); the exponentials by
      // the hardware's 2^x (one unit in the last place; a softmax asks no more of them)
      float sv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = kb + g * 4 + i;
        const bool vis = all_visible || (valid[qb] && j <= pos[qb] && j >= lo[qb]);
        sv[i] = vis ? sc[i] * scale2 : NEG_INF;
      }
      float mx = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
      mx = max_across_32(mx);
      mx = max_across_16(mx);
      const float m_new = fmaxf(m[qb], mx);
      if (__any(m_new != m[qb])) {        // some row's maximum grew: rescale what is summed so far
        // (nothing visible yet, m_new = -inf: the sums are 0 and stay 0)
        const float alpha = m_new == NEG_INF ? 1.f : fast_exp2(m[qb] - m_new);
        lsum[qb] *= alpha;
#pragma unroll
        for (int mb = 0; mb < DQ; ++mb) o[qb][mb] *= alpha;
        m[qb] = m_new;
      }
      float pv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) pv[i] = sv[i] == NEG_INF ? 0.f : fast_exp2(sv[i] - m_new);
      lsum[qb] += (pv[0] + pv[1]) + (pv[2] + pv[3]);
#pragma unroll
      for (int mb = 0; mb < DQ; ++mb) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          // (a position past the last one written holds whatever was there: kept out of
          // the product although its weight is zero)
          const float vv = (tail && kb + g * 4 + u > key_hi) ? 0.f : f.v[mb][u];
          o[qb][mb] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv, pv[u], o[qb][mb], 0, 0, 0);
        }
      }
    }
  };

  // The next steps' keys and values are on their way while this one is multiplied; the
  // loads are unconditional (a load under a branch makes the compiler wait for all loads
  // in flight where the branch ends): a step past the end reads the last one again, a
  // page that is not there reads page 0, and the flag keeps it out of the sums.  The page
  // numbers of 64 steps are read ahead, one step per lane.
  for (int cb = my0; cb < my1; cb += 64) {
    const int ce = min(cb + 64, my1);
    int pages_v;
    {
      const int pos16 = (cb + lane) * 16;
      const bool in = cb + lane < ce && pos16 <= key_hi && pos16 + 15 >= key_lo;
      const int pg = a.table[(size_t)b * a.table_stride + min(pos16 >> pshift, a.table_stride - 1)];
      pages_v = in ? pg : -1;
    }
    auto fetch = [&](int blk, Step& f) {
      const int bl = min(blk, ce - 1);
      const int page = __builtin_amdgcn_readlane(pages_v, bl - cb);
      f.ok = blk < ce && page >= 0;
      const size_t base = ((size_t)max(page, 0) * a.nkv + kvh) * P * D + (size_t)(((bl << 4) & (P - 1)) >> 4) * (16 * D);
      const float* kp = kc + base + (size_t)((g >> 1) * 16 + c) * 8 + 4 * (g & 1);
      const float* vp = vc + base + (size_t)(g * 16 + c) * 4;
#pragma unroll
      for (int mb = 0; mb < DQ; ++mb) {
        f.k[mb] = *(const floatx4*)(kp + mb * 256);      // two octets of d further
        f.v[mb] = *(const floatx4*)(vp + mb * 256);      // the next 16-wide block of d
      }
    };
    // a ring of three: two steps are on their way while one is multiplied (a wave's step is
    // about a microsecond of matrix instructions, a trip to memory takes longer, and a
    // prompt gives a SIMD fewer than two waves to fill the wait with)
    if constexpr (SPLIT) {       // (a wave's share of a split history is a few steps: one ahead is enough)
      Step cur, nxt;
      fetch(cb, cur);
      for (int blk = cb; blk < ce; ++blk) {
        fetch(blk + 1, nxt);
        __builtin_amdgcn_sched_barrier(0);
        compute(blk, cur);
        cur = nxt;
      }
      continue;
    }
    Step r0, r1, r2;
    fetch(cb, r0);
    fetch(cb + 1, r1);
    for (int blk = cb; blk < ce; blk += 3) {
      fetch(blk + 2, r2);
      __builtin_amdgcn_sched_barrier(0);
      compute(blk, r0);
      fetch(blk + 3, r0);
      __builtin_amdgcn_sched_barrier(0);
      compute(blk + 1, r1);          // (a step past the end carries ok = false)
      fetch(blk + 4, r1);
      __builtin_amdgcn_sched_barrier(0);
      compute(blk + 2, r2);
    }
  }

  if constexpr (!SPLIT) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float l = lsum[qb];
      l += __shfl_xor(l, 16, WAVE);
      l += __shfl_xor(l, 32, WAVE);
      if (!valid[qb]) continue;
      const float inv = l > 0.f ? 1.f / l : 0.f;
      float* dst = (float*)a.out + (size_t)(r0 + tok[qb]) * a.out_stride + (size_t)head[qb] * D + g * 4;
#pragma unroll
      for (int mb = 0; mb < DQ; ++mb) *(floatx4*)(dst + mb * 16) = o[qb][mb] * inv;
    }
  } else {
    // ---- merge the waves of the block through LDS (see the bfloat16 kernel)
    __shared__ float s_m[NW][16 * QB], s_l[NW][16 * QB];
    __shared__ __attribute__((aligned(16))) float s_o[NW][16 * QB][D];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float l = lsum[qb];
      l += __shfl_xor(l, 16, WAVE);
      l += __shfl_xor(l, 32, WAVE);
      if (g == 0) {
        s_m[wave][qb * 16 + c] = m[qb];
        s_l[wave][qb * 16 + c] = l;
      }
#pragma unroll
      for (int mb = 0; mb < DQ; ++mb) *(floatx4*)(&s_o[wave][qb * 16 + c][mb * 16 + g * 4]) = o[qb][mb];
    }
    __syncthreads();
    const int nrows = min(16 * QB, rows_total - row0);
    for (int idx = threadIdx.x; idx < nrows * D; idx += blockDim.x) {
      const int r = idx / D, dd = idx - r * D;
      float mmax = NEG_INF;
#pragma unroll
      for (int w = 0; w < NW; ++w) mmax = fmaxf(mmax, s_m[w][r]);
      float num = 0.f, den = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float wt = s_m[w][r] == NEG_INF ? 0.f : exp2f(s_m[w][r] - mmax);
        num += wt * s_o[w][r][dd];
        den += wt * s_l[w][r];
      }
      const int t = (row0 + r) / G, hh = kvh * G + (row0 + r) % G;
      if (a.splits == 1) {
        ((float*)a.out)[(size_t)(r0 + t) * a.out_stride + (size_t)hh * D + dd] = den > 0.f ? num / den : 0.f;
      } else {
        const size_t at = ((size_t)(r0 + t) * a.nq + hh) * a.splits + split;
        a.o_part[at * D + dd] = num;
        if (dd == 0) {
          a.ml_part[at * 2] = mmax;
          a.ml_part[at * 2 + 1] = den;
        }
      }
    }
  }
}

// ---------------------------------------------------------------- dispatch
extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

extern "C" int llmlab_attention_head_dim() { return D; }

// Debug interface (kernels/debug.py): the number of key splits can be fixed, for tests and
// measurements (0: chosen here).
static int g_force_splits = 0;
extern "C" void llmlab_debug_attention_splits(int splits) { g_force_splits = splits; }
// ... and the launch that steps of many rows take: 1 = the waves of a block split the keys of
// a tile of 32 rows, 2 = tiles of 32 rows per wave, 3 = late and early tiles in pairs,
// 4 = tiles of 16 rows per wave, 5 and 6 = 3 and 4 with two groups of waves that take the
// staged keys in turn (0: chosen here).
static int g_force_path = 0;
extern "C" void llmlab_debug_attention_path(int path) { g_force_path = path; }
// ... and who merges the key splits: 1 = the merge kernel even where the last block could.
// -1 = the last block whatever the number of splits.
static int g_force_merge_kernel = 0;
extern "C" void llmlab_debug_attention_merge_kernel(int on) { g_force_merge_kernel = on; }
constexpr int MERGE_IN_PLACE_SPLITS = 2;

// The decode-like launch: a block of DECODE_WAVES waves per (request, kv head, split); a
// wave gets about two steps of 32 keys, a block's waves merge in LDS, and only what is
// left is split over blocks; the merge kernel follows.  `live` requests (of `reqs`) pass
// the filter of `a`, `ctx_len` is their longest context.
// A decode-like launch made ready: its arguments, the depth of its ring of key steps, and
// whether a kernel of its own merges the splits afterwards.
struct KeySplitLaunch {
  AttnArgs a;
  int ring;
  bool merge_kernel;
};

static KeySplitLaunch prepare_key_split_decode(AttnArgs a, int reqs, int live, int ctx_len, int window, int total_rows,
                                               int nq, int nkv, float* workspace, size_t workspace_floats, int num_cus,
                                               int* arrived, size_t arrived_ints) {
  const int visible = window > 0 ? min(window, ctx_len) : ctx_len;
  const int steps32 = (visible + 31) / 32 + 1;
  // A unit's memory rate is the limit, so the keys are spread over the units: as many
  // splits as still give every block a unit of its own.  One block more than units
  // would double the load of the busiest one (24 requests of 4 kv heads over 4,096
  // keys: 2 splits 44 us, 3 splits 59 us); and once there are more blocks than units
  // anyway, splitting only adds work.
  const long base = (long)live * nkv;
  int splits = (int)(num_cus / base);
  const int most = (steps32 + DECODE_WAVES - 1) / DECODE_WAVES;      // one step per wave at least
  if (splits > most) splits = most;
  if (splits > MAX_KEY_SPLITS) splits = MAX_KEY_SPLITS;       // what the merge kernel takes: two per lane
  // A split costs the merge kernel (4 to 5 us with its launch), which a short history does
  // not earn back: one block reads 256 KB of keys and values in about that time, and with
  // few splits to be had (many blocks already) twice as much (64 requests of 2 kv heads of
  // 64 over 1,024 keys: 10.3 us unsplit, 13.2 in two splits; 32 requests of 4 kv heads of
  // 128 over 1,024 keys: 20.3 and 22.8; 8 requests of those over 1,024 keys: 14.8 unsplit,
  // 13.5 in eight splits).
  const size_t block_bytes = (size_t)visible * D * 2 * sizeof(bf16_t);
  if (block_bytes < (384u << 10) || (splits <= 4 && block_bytes < (768u << 10))) splits = 1;
  if (g_force_splits > 0) splits = min(g_force_splits, MAX_KEY_SPLITS);
  if (splits < 1) splits = 1;
  const size_t per_split = (size_t)total_rows * nq * (D + 2);
  while (splits > 1 && per_split * splits > workspace_floats) --splits;
  if (splits < 1) splits = 1;
  a.splits = splits;
  // Who merges the splits: two splits the last block of each (request, kv head) to arrive,
  // if the caller brought counters for them (zero now, zero again afterwards); more a
  // kernel of its own.  The last block's way is a chain of trips to memory (its stores
  // done, the counter, the other blocks' results) of about 2 us each, a kernel boundary
  // costs less than two of them: measured at context 4096 of the 0.5B shape, 64 requests in
  // 2 splits take 1.743 ms a step against 1.781 with the kernel, 8 requests in 16 splits
  // 1.001 against 0.962; at the 32B shape, 8 requests in 4 splits, 55.4 us a layer against
  // 51.6 + 4.8 (no difference).
  const bool merge_in_place = splits > 1 && arrived != nullptr && (size_t)reqs * nkv <= arrived_ints &&
                              g_force_merge_kernel == 0 && (splits <= MERGE_IN_PLACE_SPLITS || g_force_merge_kernel < 0);
  a.arrived = merge_in_place ? arrived : nullptr;
  if (splits > 1) {
    a.o_part = workspace;
    a.ml_part = workspace + (size_t)total_rows * nq * splits * D;
  }
  const int steps_per_wave = ((steps32 + splits - 1) / splits + DECODE_WAVES - 1) / DECODE_WAVES;
  return KeySplitLaunch{a, steps_per_wave > 2 ? 2 : 1, splits > 1 && !merge_in_place};
}

static int launch_split_merge(const KeySplitLaunch& k, int total_rows, int nq, const int* row_req, void* out,
                              int out_stride, hipStream_t stream) {
  if (!k.merge_kernel) return 0;
  hipLaunchKernelGGL(attention_merge_kernel<bf16_t>, dim3(total_rows, nq), dim3(k.a.splits > 16 ? 64 * MERGE_WAVES : 64), 0,
                     stream, k.a.o_part, k.a.ml_part, (bf16_t*)out, out_stride, nq, k.a.splits, row_req, k.a.q_start,
                     k.a.qlen_hi);
  LLMLAB_LAUNCH_CHECK("attention merge");
  return 0;
}

static int launch_key_split_decode(const KeySplitLaunch& k, int reqs, int total_rows, int nq, int nkv,
                                   const int* row_req, void* out, int out_stride, hipStream_t stream) {
  dim3 grid(1, nkv * k.a.splits, reqs), block(64 * DECODE_WAVES);
  if (k.ring == 2)
    hipLaunchKernelGGL((attention_bf16_kernel<1, true, 2>), grid, block, 0, stream, k.a);
  else
    hipLaunchKernelGGL((attention_bf16_kernel<1, true, 1>), grid, block, 0, stream, k.a);
  LLMLAB_LAUNCH_CHECK("attention(bfloat16, decode)");
  return launch_split_merge(k, total_rows, nq, row_req, out, out_stride, stream);
}

// 1: a mixed step always in two launches; -1: in one wherever a kernel for it exists (measurements)
static int g_force_two_launches = 0;
extern "C" void llmlab_debug_attention_two_launches(int on) { g_force_two_launches = on; }

// float32.  Steps of at most 16 rows per request and kv head (decode) split the keys over
// the waves of a block and over blocks, as many splits as still give every block a compute
// unit of its own (the same rule as in bfloat16, for twice the bytes), and the merge kernel
// sums the splits.  Steps of more rows take one block per tile of 32 rows (16 for heads
// above 128: registers) whose waves split the keys, or, once the tiles fill the chip, one
// wave per tile (launch_attention_f32 says when).
constexpr int F32_SPLIT_WAVES = D <= 64 ? 8 : 4;
constexpr int F32_QB = D <= 128 ? 2 : 1;
static int launch_f32_key_split(AttnArgs a, int reqs, int live, int ctx_len, int window, int total_rows,
                                float* workspace, size_t workspace_floats, int num_cus, const int* row_req,
                                hipStream_t stream) {
  const int visible = window > 0 ? min(window, ctx_len) : ctx_len;
  const int steps16 = (visible + 15) / 16 + 1;
  int splits = (int)(num_cus / ((long)live * a.nkv));
  const int most = (steps16 + 2 * F32_SPLIT_WAVES - 1) / (2 * F32_SPLIT_WAVES);     // two steps per wave at least
  if (splits > most) splits = most;
  if (splits > MAX_KEY_SPLITS) splits = MAX_KEY_SPLITS;
  const size_t block_bytes = (size_t)visible * D * 2 * sizeof(float);
  if (block_bytes < (384u << 10) || (splits <= 4 && block_bytes < (768u << 10))) splits = 1;
  if (g_force_splits > 0) splits = min(g_force_splits, MAX_KEY_SPLITS);
  if (splits < 1) splits = 1;
  const size_t per_split = (size_t)total_rows * a.nq * (D + 2);
  while (splits > 1 && per_split * splits > workspace_floats) --splits;
  a.splits = splits;
  if (splits > 1) {
    a.o_part = workspace;
    a.ml_part = workspace + (size_t)total_rows * a.nq * splits * D;
  }
  hipLaunchKernelGGL((attention_f32_kernel<1, true, F32_SPLIT_WAVES>), dim3(1, a.nkv * splits, reqs),
                     dim3(64 * F32_SPLIT_WAVES), 0, stream, a);
  LLMLAB_LAUNCH_CHECK("attention(float32, decode)");
  if (splits > 1) {
    hipLaunchKernelGGL(attention_merge_kernel<float>, dim3(total_rows, a.nq), dim3(splits > 16 ? 64 * MERGE_WAVES : 64),
                       0, stream, a.o_part, a.ml_part, (float*)a.out, a.out_stride, a.nq, splits, row_req,
                       a.q_start, a.qlen_hi);
    LLMLAB_LAUNCH_CHECK("attention merge (float32)");
  }
  return 0;
}

// Which launch a float32 step of many rows takes: 1 = the waves of a block split the keys of a
// tile, anything else = a wave per tile.  `blocks`: tiles of rows times kv heads times requests.
static int choose_many_rows_launch_f32(long blocks, int max_q_len, int max_ctx_len, int num_cus, int forced) {
  if (forced != 0) return forced;
  // (how few the keys must be for a wave per tile, by how many times the tiles fill the chip)
  int few_keys;
  // (heads above 64: portions of 1,024 tokens and more keep the key split until their tiles fill
  // the chip seven times, since the late tiles of a long portion walk many more keys than the
  // early ones and a wave per tile leaves that uneven: one prompt of 1,024 tokens 148 us against
  // 184, of 2,048 453 against 512, two of 1,024 290 against 305; four of 1,024 562 against 501)
  if (D > 64) few_keys = blocks > (max_q_len >= 1024 ? 7L : 2L) * num_cus ? 0x7fffffff
                         : blocks >= (7L * num_cus) / 4 && max_q_len < 1024 ? 128 : 0;
  else few_keys = blocks >= 14L * num_cus ? 1024 : blocks >= 7L * num_cus ? 768 : blocks >= (7L * num_cus) / 2 ? 256
                  : blocks >= (7L * num_cus) / 4 ? 128 : 0;
  return max_ctx_len <= few_keys ? 2 : 1;
}

static int launch_attention_f32(AttnArgs a, int reqs, int max_q_len, int max_ctx_len, int window, int total_rows,
                                float* workspace, size_t workspace_floats, int num_cus, const int* row_req,
                                int short_len, int n_short, int short_ctx, hipStream_t stream) {
  LLMLAB_REQUIRE(a.q_stride % 4 == 0 && a.out_stride % 4 == 0 && ((uintptr_t)a.q % 16 == 0) &&
                 ((uintptr_t)a.out % 16 == 0) && ((uintptr_t)a.kc % 16 == 0) && ((uintptr_t)a.vc % 16 == 0),
                 "attention(float32): operands are not aligned for 16-byte loads");
  const int G = a.nq / a.nkv;
  const long max_rows = (long)max_q_len * G;
  if (max_rows <= 16)
    return launch_f32_key_split(a, reqs, reqs, max_ctx_len, window, total_rows, workspace, workspace_floats,
                                num_cus, nullptr, stream);
  int live = reqs;
  if (row_req != nullptr && n_short > 0 && n_short < reqs && (long)short_len * G <= 16) {
    // a mixed step: its requests of a few tokens by the launch that splits their keys
    AttnArgs s = a;
    s.qlen_hi = short_len;
    const int rc = launch_f32_key_split(s, reqs, n_short, short_ctx, window, total_rows, workspace,
                                        workspace_floats, num_cus, row_req, stream);
    if (rc) return rc;
    a.qlen_lo = short_len + 1;
    live = reqs - n_short;
  }
  constexpr int ROWS = 16 * F32_QB;
  const long tiles = (max_rows + ROWS - 1) / ROWS;
  // Which launch, from a sweep of 1 to 32 requests of 64 to 8,192 tokens behind 0 to 4,096 keys
  // (14 heads of 64 over 2, 28 of 128 over 4).  A block whose waves split the keys of a tile
  // (1) wins wherever a wave per tile (2) would leave compute units idle or walk a long
  // history alone: 512 tokens behind 1,024 keys at heads of 64 take 43 us so and 162 with a
  // wave per tile, a prompt of 2,048 tokens 117 against 217.  A wave per tile wins once the
  // tiles fill the chip and the keys are few (16 requests of 512 tokens from their start,
  // heads of 64: 137 us against 187), at heads above 64 from two tiles a unit on whatever the
  // keys (4 requests of 256 tokens: 58 against 81).
  const int path = choose_many_rows_launch_f32(tiles * a.nkv * live, max_q_len, max_ctx_len, num_cus, g_force_path);
  if (path == 1) {
    hipLaunchKernelGGL((attention_f32_kernel<F32_QB, true, F32_SPLIT_WAVES>), dim3((unsigned)tiles, a.nkv, reqs),
                       dim3(64 * F32_SPLIT_WAVES), 0, stream, a);
  } else {
    hipLaunchKernelGGL((attention_f32_kernel<F32_QB, false, 4>), dim3((unsigned)((tiles + 3) / 4), a.nkv, reqs),
                       dim3(256), 0, stream, a);
  }
  LLMLAB_LAUNCH_CHECK("attention(float32)");
  return 0;
}

constexpr bool TWO_GROUPS = D <= 128;      // (the staged keys and values of two groups at larger heads: more LDS than there is)

// Which launch a step of many rows takes (bfloat16): `max_rows` (token, head of the group) pairs
// at most per request and kv head, `live` requests, the longest portion and context, the window.
static int choose_many_rows_launch(long max_rows, int nkv, int live, int max_q_len, int max_ctx_len, int window,
                                   int num_cus, int forced) {
  // The launch, from measurements of 64 to 4,096 tokens behind 0 and 4,096 keys, one to
  // eight requests, heads of 64 (14 over 2) and 128 (28 over 4, 40 over 8):
  //   1  few tiles of rows behind a history: the waves of a block split the keys of
  //      one tile of 32 rows and merge in LDS, so that the work still spreads over the
  //      chip (64 to 512 tokens behind 4,096 keys, heads of 64: 27 to 31 us against 41 to
  //      46 for the next best; at the start of a short prompt it is the slowest)
  //   6  every wave owns 16 rows, the block's two groups of four waves take the staged
  //      keys in turn: for heads above 64, where a block of four waves is alone on its
  //      compute unit (2,048 tokens behind 4,096 keys, 28 heads of 128: 313 us against
  //      374 to 470 for the others), and for heads of 64 when the tiles of rows would
  //      leave a SIMD with one wave or none, or the longest tile of a long prompt's
  //      triangle decides (2,048 tokens from 0: 32 us against 38; four prompts of 512: 19
  //      against 15, so not for those)
  //   4  the same with one group of four waves (two blocks share a compute unit at heads
  //      of 64)
  //   2  32 rows per wave, when that still gives every compute unit two blocks
  //   3  late and early tiles in pairs (see below)
  const long blocks16 = ((max_rows + 63) / 64) * nkv * live;
  const long blocks32 = ((max_rows + 127) / 128) * nkv * live;
  // (from how long a history on the key split of launch 1 pays, few tiles of rows given: 128
  // to 512 tokens of 14 heads of 64 behind 512 / 1,536 / 2,560 keys take 12 to 14 / 17 to 19 /
  // 21 to 24 us so and 13 to 16 / 21 to 24 / 29 to 32 with launch 6, at the start of a prompt
  // 9 to 11 against 7 to 11; of 28 heads of 128 behind 1,024 / 1,536 / 2,560 keys 29 / 34 / 44
  // against 25 / 32 / 47)
  const bool long_history = (long)max_ctx_len - max_q_len >= (D <= 64 ? 384 : 1792);
  const bool triangle = window <= 0 && 16L * (max_ctx_len - max_q_len) <= max_q_len;
  int path = forced;
  if (!TWO_GROUPS && (path == 5 || path == 6)) path = 0;
  if (path == 0) {
    // (the rules below are fitted to sweeps of 1 to 64 requests of 32 to 16,384 tokens behind
    // 0 to 8,192 keys at the three head shapes, 470 cases: they lose 0.7 % to the best launch
    // of each case on average, and more than 7 % in 16 of them)
    const bool short_rows = max_q_len <= 128;
    if (blocks16 <= num_cus / 2 && long_history) path = 1;
    // larger heads, short prompts from their start that leave units idle: one group of waves
    // (64 tokens of 28 heads of 128: 8.4 us against 9.8)
    else if (D > 64 && triangle && short_rows && blocks16 <= num_cus) path = 4;
    // ... and many short portions behind short histories: 32 rows a wave (8 requests of 64
    // tokens, 40 heads of 128 over 8: 11 us against 18; of 128 tokens, 28 over 4: 14 against 19)
    else if (D > 64 && D <= 128 && blocks16 > num_cus && max_ctx_len <= 1024 &&
             (short_rows || (max_q_len <= 256 && triangle))) path = 2;
    else if (TWO_GROUPS && D > 64 && !(blocks16 >= 4L * num_cus && max_ctx_len <= 1024)) path = 6;
    // heads of 64: two groups of waves when at most a tile of rows a unit is to be had, unless
    // the prompts are short and at their start (16 requests of 64 tokens: 6.8 us with one
    // group against 8.0), and for long portions up to three tiles a unit
    else if (TWO_GROUPS && D <= 64 && blocks16 <= num_cus / 2 && max_ctx_len >= 384) path = 6;
    else if (TWO_GROUPS && D <= 64 && blocks16 > num_cus / 2 &&
             ((blocks16 <= num_cus && (max_q_len >= 256 || !triangle)) ||
              (blocks16 <= 3L * num_cus && max_q_len >= 1536))) path = 6;
    else if (blocks16 < num_cus) path = 4;
    // 32 rows a wave once its blocks fill the chip twice; at heads of 64 a little earlier,
    // but only for portions up to 1,024 tokens behind a history (8 requests of 512 tokens behind
    // 2,048 keys: 75 us against 83; two prompts of 4,096 from their start: 161 against 132), and
  // for prompts of 8,192 tokens and more (221 us against 235)
    else if (D > 64 ? (D <= 128 && blocks32 >= 2L * num_cus)
                    : (blocks32 >= (7L * num_cus) / 4 && ((max_q_len <= 1024 && !triangle) || max_q_len >= 8192))) path = 2;
    // not enough tiles to keep every unit busy with what the longest ones leave over:
    // pair late and early tiles (no window: then the loads add up evenly).  Only at the
    // start of a prompt: behind a history all tiles carry about the same load, and the
    // pairs only halve the blocks (2,048 tokens behind 8,192, head size 64: 246 us in
    // pairs, 172 without); and only at larger heads (heads of 64: 8 requests of 256 tokens
    // 13.6 us in pairs, 10.6 without; 2 of 1,024: 23.5 against 21.5)
    else if (D > 64 && triangle && blocks16 >= (3L * num_cus) / 2) path = 3;
    else path = 4;
  }
  return path;
}

// Whether the blocks of a mixed step's portions (keys split over the waves of a block) and of its
// decoding requests go in one launch: see llmlab_paged_attention.
static bool mixed_step_in_one_launch(long long_blocks, long short_blocks, int num_cus, int forced) {
  if (forced > 0) return false;
  if (forced < 0) return true;
  const long places = (D <= 64 ? 1L : 2L) * num_cus;      // blocks of the portion's kind that the chip holds at a time
  return 2 * long_blocks <= places || 4 * (long_blocks + short_blocks) <= 5 * places;
}

// How many attention launches a mixed step in bfloat16 takes (the merge of key splits not
// counted): `n_short` of its requests decode behind at most `short_ctx` keys, the others bring
// portions of at most `max_q_len` tokens (for tests and tuning; 0: not a mixed step).
extern "C" int llmlab_attention_mixed_launches(int nq, int nkv, int reqs, int n_short, int max_q_len, int max_ctx_len,
                                               int short_ctx, int window, int num_cus) {
  if (num_cus <= 0) num_cus = 256;
  if (nq <= 0 || nkv <= 0 || nq % nkv != 0 || n_short <= 0 || n_short >= reqs || max_q_len <= 0) return 0;
  const long max_rows = (long)max_q_len * (nq / nkv);
  if (max_rows <= 16) return 0;
  const int live = reqs - n_short;
  if (choose_many_rows_launch(max_rows, nkv, live, max_q_len, max_ctx_len, window, num_cus, 0) != 1) return 2;
  AttnArgs a{};
  const KeySplitLaunch shorts = prepare_key_split_decode(a, reqs, n_short, short_ctx, window, reqs, nq, nkv, nullptr,
                                                         ~(size_t)0 >> 8, num_cus, nullptr, 0);
  return mixed_step_in_one_launch((max_rows + 31) / 32 * nkv * live, (long)nkv * shorts.a.splits * n_short, num_cus, 0)
             ? 1 : 2;
}

// The launch that llmlab_paged_attention would take for a step of many rows of these sizes
// (for tests and tuning; 0: the sizes make a decode step, whose keys are split over blocks).
extern "C" int llmlab_attention_launch(int dtype, int nq, int nkv, int reqs, int max_q_len, int max_ctx_len, int window,
                                       int num_cus) {
  if (num_cus <= 0) num_cus = 256;
  if (nq <= 0 || nkv <= 0 || nq % nkv != 0 || reqs <= 0 || max_q_len <= 0) return -1;
  const long max_rows = (long)max_q_len * (nq / nkv);
  if (max_rows <= 16) return 0;
  if (dtype == DT_F32) {
    constexpr int ROWS = 16 * F32_QB;
    return choose_many_rows_launch_f32((max_rows + ROWS - 1) / ROWS * nkv * reqs, max_q_len, max_ctx_len, num_cus, 0);
  }
  return choose_many_rows_launch(max_rows, nkv, reqs, max_q_len, max_ctx_len, window, num_cus, 0);
}

// q rows are the step's packed rows; reqs requests; max_q_len / max_ctx_len are
// the largest portion and the longest context in the step (they size the grid
// and choose the key splits).  workspace: float32 scratch for split partials.
// A mixed step (portions of prompts beside single decoded tokens) may say so:
// n_short of its requests bring at most short_len tokens each, the longest context
// among those is short_ctx, and row_req[row] is the request of a row.  Its short
// requests are then served by the decode-like launch and the others by the tiled one;
// in one launch the few rows of a decoding request would walk its whole history in
// one wave while the rest of the chip waits.
extern "C" int llmlab_paged_attention(const void* q, int dtype, int q_stride, int nq, int nkv,
                                      const void* kcache, const void* vcache, const int* table,
                                      int table_stride, int page_size, const int* q_start,
                                      const int* start_pos, int reqs, int max_q_len, int max_ctx_len,
                                      int window, float scale, void* out, int out_stride,
                                      float* workspace, size_t workspace_floats, int total_rows,
                                      int num_cus, const int* row_req, int short_len, int n_short,
                                      int short_ctx, int* arrived, size_t arrived_ints, hipStream_t stream) {
  LLMLAB_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attention: %d heads, %d kv heads", nq, nkv);
  LLMLAB_REQUIRE(page_size >= 16 && (page_size & (page_size - 1)) == 0,
                 "attention: page size %d is not a power of two >= 16", page_size);
  LLMLAB_REQUIRE(q_stride >= nq * D && out_stride >= nq * D, "attention: row strides too small");
  LLMLAB_REQUIRE(reqs >= 0 && reqs <= 65535 && nq <= 65535, "attention: grid too large");
  LLMLAB_REQUIRE(window >= 0, "attention: negative window");
  LLMLAB_REQUIRE(scale > 0.f, "attention: the score scale must be positive, got %g", (double)scale);
  LLMLAB_REQUIRE(n_short >= 0 && n_short <= reqs && short_len >= 0 && short_ctx >= 0 && short_ctx <= max_ctx_len,
                 "attention: bad description of the short requests");
  if (reqs == 0 || max_q_len <= 0) return 0;
  if (num_cus <= 0) num_cus = 256;
  AttnArgs a;
  a.q = q; a.kc = kcache; a.vc = vcache; a.table = table; a.q_start = q_start; a.start_pos = start_pos;
  a.out = out; a.o_part = nullptr; a.ml_part = nullptr; a.arrived = nullptr;
  a.q_stride = q_stride; a.out_stride = out_stride; a.table_stride = table_stride; a.page_size = page_size;
  a.nq = nq; a.nkv = nkv; a.window = window; a.splits = 1; a.scale = scale;
  a.page_shift = 0;
  a.tiles = 0;
  a.qlen_lo = 0; a.qlen_hi = 0x7fffffff;
  while ((1 << a.page_shift) < page_size) ++a.page_shift;
  if (dtype == DT_F32)
    return launch_attention_f32(a, reqs, max_q_len, max_ctx_len, window, total_rows, workspace, workspace_floats,
                                num_cus, row_req, short_len, n_short, short_ctx, stream);
  LLMLAB_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && out_stride % 4 == 0 &&
                 ((uintptr_t)out % 8 == 0) && ((uintptr_t)kcache % 16 == 0) && ((uintptr_t)vcache % 16 == 0),
                 "attention(bfloat16): operands are not aligned for vector loads");
  const int G = nq / nkv;
  const long max_rows = (long)max_q_len * G;
  if (max_rows <= 16)
    return launch_key_split_decode(prepare_key_split_decode(a, reqs, reqs, max_ctx_len, window, total_rows, nq, nkv,
                                                            workspace, workspace_floats, num_cus, arrived, arrived_ints),
                                   reqs, total_rows, nq, nkv, nullptr, out, out_stride, stream);
  int live = reqs;
  const bool mixed = row_req != nullptr && n_short > 0 && n_short < reqs && (long)short_len * G <= 16;
  KeySplitLaunch shorts{};
  if (mixed) {
    AttnArgs s = a;
    s.qlen_hi = short_len;
    shorts = prepare_key_split_decode(s, reqs, n_short, short_ctx, window, total_rows, nq, nkv, workspace,
                                      workspace_floats, num_cus, arrived, arrived_ints);
    a.qlen_lo = short_len + 1;
    live = reqs - n_short;
  }
  const int path = choose_many_rows_launch(max_rows, nkv, live, max_q_len, max_ctx_len, window, num_cus, g_force_path);
  if (mixed && path != 1) {
    const int rc = launch_key_split_decode(shorts, reqs, total_rows, nq, nkv, row_req, out, out_stride, stream);
    if (rc) return rc;
  }
  if (path == 1) {
    const int steps32 = (max_ctx_len + 31) / 32 + 1;
    const int steps_per_wave = (steps32 + DECODE_WAVES - 1) / DECODE_WAVES;
    // Both kinds of blocks in one launch (see attention_bf16_mixed_kernel) where the portion's
    // blocks leave half of the chip's places free, or all blocks together hardly exceed the
    // places: every block of the one launch holds the registers of the portion's kind, so the
    // decoding requests' blocks, which stream and want company on their unit, lose places
    // (a unit holds one block at heads up to 64, two above).  Heads of 64, a portion of 128
    // tokens behind 2,048 keys beside 63 requests decoding at 2,048: 28 us against 38 in two
    // launches; a portion of 512 (224 blocks) beside 31 at 1,024: 27 against 30, beside 127 at
    // 1,024: 68 against 59, hence not there.  Heads of 128, 128 tokens beside 63 at 2,048: 75
    // against 90.
    const int long_tiles = (int)((max_rows + 31) / 32);
    const bool one_launch = mixed && mixed_step_in_one_launch((long)long_tiles * nkv * live,
                                                              (long)nkv * shorts.a.splits * n_short, num_cus,
                                                              g_force_two_launches);
    if (mixed && !one_launch) {
      const int rc = launch_key_split_decode(shorts, reqs, total_rows, nq, nkv, row_req, out, out_stride, stream);
      if (rc) return rc;
    }
    if (one_launch) {
      const long gx = (long)long_tiles * nkv + (long)nkv * shorts.a.splits;
      LLMLAB_REQUIRE(gx <= 0x7fffffffL, "attention: grid too large");
      dim3 mgrid((unsigned)gx, 1, reqs), mblock(64 * DECODE_WAVES);
      const bool deep = steps_per_wave > 2;
      if (deep && shorts.ring == 2)
        hipLaunchKernelGGL((attention_bf16_mixed_kernel<2, 2, 2>), mgrid, mblock, 0, stream, a, shorts.a, long_tiles);
      else if (deep)
        hipLaunchKernelGGL((attention_bf16_mixed_kernel<2, 2, 1>), mgrid, mblock, 0, stream, a, shorts.a, long_tiles);
      else if (shorts.ring == 2)
        hipLaunchKernelGGL((attention_bf16_mixed_kernel<2, 1, 2>), mgrid, mblock, 0, stream, a, shorts.a, long_tiles);
      else
        hipLaunchKernelGGL((attention_bf16_mixed_kernel<2, 1, 1>), mgrid, mblock, 0, stream, a, shorts.a, long_tiles);
      LLMLAB_LAUNCH_CHECK("attention(bfloat16, mixed)");
      return launch_split_merge(shorts, total_rows, nq, row_req, out, out_stride, stream);
    }
    dim3 grid((unsigned)((max_rows + 31) / 32), nkv, reqs), block(64 * DECODE_WAVES);
    if (steps_per_wave > 2)
      hipLaunchKernelGGL((attention_bf16_kernel<2, true, 2>), grid, block, 0, stream, a);
    else
      hipLaunchKernelGGL((attention_bf16_kernel<2, true, 1>), grid, block, 0, stream, a);
    LLMLAB_LAUNCH_CHECK("attention(bfloat16, key split)");
    return 0;
  }
  if (path == 2) {
    dim3 grid((unsigned)((max_rows + 127) / 128), nkv, reqs), block(256);
    hipLaunchKernelGGL((attention_bf16_kernel<2, false>), grid, block, 0, stream, a);
  } else if (path == 5) {
    if constexpr (TWO_GROUPS) {
      a.tiles = (int)((max_rows + 63) / 64);
      dim3 grid((unsigned)((a.tiles + 1) / 2), nkv, reqs), block(512);
      hipLaunchKernelGGL((attention_bf16_paired_kernel<1, 2>), grid, block, 0, stream, a);
    }
  } else if (path == 6) {
    if constexpr (TWO_GROUPS) {
      dim3 grid((unsigned)((max_rows + 63) / 64), nkv, reqs), block(512);
      hipLaunchKernelGGL((attention_bf16_kernel<1, false, 1, 2>), grid, block, 0, stream, a);
    }
  } else if (path == 3) {
    a.tiles = (int)((max_rows + 63) / 64);
    dim3 grid((unsigned)((a.tiles + 1) / 2), nkv, reqs), block(256);
    hipLaunchKernelGGL((attention_bf16_paired_kernel<1>), grid, block, 0, stream, a);
  } else {
    dim3 grid((unsigned)((max_rows + 63) / 64), nkv, reqs), block(256);
    hipLaunchKernelGGL((attention_bf16_kernel<1, false>), grid, block, 0, stream, a);
  }
  LLMLAB_LAUNCH_CHECK("attention(bfloat16, prefill)");
  return 0;
}
