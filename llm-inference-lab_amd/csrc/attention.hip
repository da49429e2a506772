// Grouped-query attention over the paged cache, for one head size (HEAD_DIM is
// given on the compiler's command line; the library is built once per head size
// that a model needs).  gfx950 only.
//
// Cache of one layer:   keys   K[page][kv_head][P][D]
//                        values V[page][kv_head][D][P]   (transposed)
// Position p of the b-th request of the step lives in page table[b][p / P] at
// offset p % P.  The query at position p sees the keys lo..p, lo = max(0, p -
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
// Split keys (decode): blockIdx.y also counts splits of the key range; each split
// writes its unnormalised sum, maximum and denominator, and a second kernel merges
// them:  out = sum_s w_s acc_s / sum_s w_s l_s,  w_s = 2^(m_s - m).
//
// float32 kernel: one wave per (token, head), lanes over keys, plain FMA; true
// 32-bit arithmetic.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256,
              "head sizes are multiples of 16 up to 256");

constexpr int D = HEAD_DIM;
constexpr float NEG_INF = -__builtin_huge_valf();

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
  int q_stride, out_stride, table_stride, page_size;
  int nq, nkv, window, splits;
  float scale;
};

// ------------------------------------------------------------- bf16, MFMA
template <int QB>
__global__ __launch_bounds__(256) void attention_bf16_kernel(AttnArgs a) {
  constexpr int DC = (D + 31) / 32;  // 32-wide chunks of d for Q.K
  constexpr int DB = D / 16;         // 16-wide blocks of d for P.V
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int b = blockIdx.z;
  const int kvh = blockIdx.y / a.splits, split = blockIdx.y % a.splits;
  const int G = a.nq / a.nkv;
  const int r0 = a.q_start[b], qlen = a.q_start[b + 1] - r0, sp = a.start_pos[b];
  const int rows_total = qlen * G;
  const int row0 = (blockIdx.x * nw + wave) * (16 * QB);
  if (row0 >= rows_total) return;
  const bf16_t* q = (const bf16_t*)a.q;
  const bf16_t* kc = (const bf16_t*)a.kc;
  const bf16_t* vc = (const bf16_t*)a.vc;
  const int P = a.page_size;
  const float scale2 = a.scale * 1.4426950408889634f;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // this lane's row in each 16-row block
  bool valid[QB];
  int tok[QB], head[QB], pos[QB], lo[QB];
  bf16x8 qf[QB][DC];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int rr = row0 + qb * 16 + c;
    valid[qb] = rr < rows_total;
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

  // keys this tile can see, and this split's share of them in blocks of 32
  const int last_row = min(row0 + 16 * QB, rows_total) - 1;
  const int p_first = sp + row0 / G, p_last = sp + last_row / G;
  const int key_lo = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  const int key_hi = p_last;
  const int blk_lo = key_lo >> 5, blk_hi = key_hi >> 5;
  const int per = (blk_hi - blk_lo + 1 + a.splits - 1) / a.splits;
  const int my_blk0 = blk_lo + split * per;
  const int my_blk1 = min(my_blk0 + per, blk_hi + 1);

  floatx4 o[QB][DB];
  float m[QB], lsum[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m[qb] = NEG_INF;
    lsum[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) o[qb][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  for (int blk = my_blk0; blk < my_blk1; ++blk) {
    const int kb = blk << 5;
    floatx4 s[2][QB];
    bool ok[2];
    const bf16_t* vbase[2];
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) s[h2][qb] = floatx4{0.f, 0.f, 0.f, 0.f};
      const int pos16 = kb + h2 * 16;
      ok[h2] = pos16 <= key_hi && pos16 + 15 >= key_lo;
      int page = -1;
      if (ok[h2]) page = a.table[(size_t)b * a.table_stride + pos16 / P];
      ok[h2] = ok[h2] && page >= 0;
      vbase[h2] = vc;
      if (ok[h2]) {
        const int off = pos16 % P;
        const bf16_t* kp = kc + (((size_t)page * a.nkv + kvh) * P + off + c) * D;
        vbase[h2] = vc + ((size_t)page * a.nkv + kvh) * D * P + off;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
          const int dd = dc * 32 + g * 8;
          const bf16x8 kf = (dd < D) ? *(const bf16x8*)(kp + dd) : zero8;
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            s[h2][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[qb][dc], s[h2][qb], 0, 0, 0);
        }
      }
    }

    bf16x8 pf[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float sv[8];
      float mx = NEG_INF;
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = kb + h2 * 16 + g * 4 + i;
          const bool vis = ok[h2] && valid[qb] && j <= pos[qb] && j >= lo[qb];
          const float v = vis ? s[h2][qb][i] * scale2 : NEG_INF;
          sv[h2 * 4 + i] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
      mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
      const float m_new = fmaxf(m[qb], mx);
      const bool none = m_new == NEG_INF;
      const float alpha = none ? 1.f : exp2f(m[qb] - m_new);
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float p = none ? 0.f : exp2f(sv[i] - m_new);
        pf[qb][i] = (bf16_t)p;
        psum += (float)pf[qb][i];   // the denominator sums what the product uses
      }
      lsum[qb] = lsum[qb] * alpha + psum;
      m[qb] = m_new;
#pragma unroll
      for (int db = 0; db < DB; ++db) o[qb][db] *= alpha;
    }

    // keys past the last written position hold stale values: keep them out of
    // the product even though their probability is zero
    const bool tail = kb + 31 > key_hi;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x4 v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
      const size_t drow = (size_t)(db * 16 + c) * P + g * 4;
      if (ok[0]) v0 = *(const bf16x4*)(vbase[0] + drow);
      if (ok[1]) v1 = *(const bf16x4*)(vbase[1] + drow);
      bf16x8 vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
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
  }

#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    float l = lsum[qb];
    l += __shfl_xor(l, 16, WAVE);
    l += __shfl_xor(l, 32, WAVE);
    if (!valid[qb]) continue;
    const size_t row = (size_t)(r0 + tok[qb]);
    if (a.splits == 1) {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16_t* dst = (bf16_t*)a.out + row * a.out_stride + (size_t)head[qb] * D;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        bf16x4 w = {(bf16_t)(o[qb][db][0] * inv), (bf16_t)(o[qb][db][1] * inv),
                    (bf16_t)(o[qb][db][2] * inv), (bf16_t)(o[qb][db][3] * inv)};
        *(bf16x4*)(dst + db * 16 + g * 4) = w;
      }
    } else {
      const size_t at = (row * a.nq + head[qb]) * a.splits + split;
      float* dst = a.o_part + at * D;
#pragma unroll
      for (int db = 0; db < DB; ++db) *(floatx4*)(dst + db * 16 + g * 4) = o[qb][db];
      if (g == 0) {
        a.ml_part[at * 2] = m[qb];
        a.ml_part[at * 2 + 1] = l;
      }
    }
  }
}

// out[row, head, :] = sum_s 2^(m_s - m) acc_s / sum_s 2^(m_s - m) l_s
template <typename T>
__global__ void attention_merge_kernel(const float* __restrict__ o_part,
                                       const float* __restrict__ ml_part, T* __restrict__ out,
                                       int out_stride, int nq, int splits) {
  const int row = blockIdx.x, head = blockIdx.y;
  const size_t base = ((size_t)row * nq + head) * splits;
  float mmax = NEG_INF;
  for (int s = 0; s < splits; ++s) mmax = fmaxf(mmax, ml_part[(base + s) * 2]);
  for (int dd = threadIdx.x; dd < D; dd += blockDim.x) {
    float num = 0.f, den = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float ms = ml_part[(base + s) * 2];
      const float w = ms == NEG_INF ? 0.f : exp2f(ms - mmax);
      num += w * o_part[(base + s) * D + dd];
      den += w * ml_part[(base + s) * 2 + 1];
    }
    out[(size_t)row * out_stride + (size_t)head * D + dd] = from_float<T>(den > 0.f ? num / den : 0.f);
  }
}

// ------------------------------------------------------------ f32, scalar
__global__ __launch_bounds__(64) void attention_f32_kernel(AttnArgs a) {
  __shared__ float qs[D];
  const int lane = threadIdx.x;
  const int t = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int r0 = a.q_start[b], qlen = a.q_start[b + 1] - r0;
  if (t >= qlen) return;
  const int G = a.nq / a.nkv, kvh = h / G;
  const int p = a.start_pos[b] + t;
  const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
  const int P = a.page_size;
  const float* q = (const float*)a.q + (size_t)(r0 + t) * a.q_stride + (size_t)h * D;
  const float* kc = (const float*)a.kc;
  const float* vc = (const float*)a.vc;
  for (int dd = lane; dd < D; dd += 64) qs[dd] = q[dd];
  __syncthreads();

  float o[D];
#pragma unroll
  for (int dd = 0; dd < D; ++dd) o[dd] = 0.f;
  float m = NEG_INF, l = 0.f;
  for (int j = lo + lane; j <= p; j += 64) {
    const int page = a.table[(size_t)b * a.table_stride + j / P];
    const int off = j % P;
    const float* kp = kc + (((size_t)page * a.nkv + kvh) * P + off) * D;
    const float* vp = vc + ((size_t)page * a.nkv + kvh) * D * P + off;
    float dot = 0.f;
#pragma unroll
    for (int dd = 0; dd < D; ++dd) dot = fmaf(qs[dd], kp[dd], dot);
    const float s = dot * a.scale;
    const float m_new = fmaxf(m, s);
    const float alpha = expf(m - m_new);  // m = -inf on the first key: exp(-inf) = 0
    const float pr = expf(s - m_new);
    l = l * alpha + pr;
#pragma unroll
    for (int dd = 0; dd < D; ++dd) o[dd] = fmaf(pr, vp[(size_t)dd * P], o[dd] * alpha);
    m = m_new;
  }
  const float mmax = wave_max(m);
  const float w = m == NEG_INF ? 0.f : expf(m - mmax);
  const float ltot = wave_sum(l * w);
  const float inv = ltot > 0.f ? 1.f / ltot : 0.f;
  float* dst = (float*)a.out + (size_t)(r0 + t) * a.out_stride + (size_t)h * D;
#pragma unroll
  for (int dd = 0; dd < D; ++dd) {
    const float tot = wave_sum(o[dd] * w);
    if ((dd & 63) == lane) dst[dd] = tot * inv;
  }
}

// ---------------------------------------------------------------- dispatch
extern "C" const char* llmlab_last_error() { return g_llmlab_error; }

extern "C" int llmlab_attention_head_dim() { return D; }

// q rows are the step's packed rows; reqs requests; max_q_len / max_ctx_len are
// the largest portion and the longest context in the step (they size the grid
// and choose the key splits).  workspace: float32 scratch for split partials.
extern "C" int llmlab_paged_attention(const void* q, int dtype, int q_stride, int nq, int nkv,
                                      const void* kcache, const void* vcache, const int* table,
                                      int table_stride, int page_size, const int* q_start,
                                      const int* start_pos, int reqs, int max_q_len, int max_ctx_len,
                                      int window, float scale, void* out, int out_stride,
                                      float* workspace, size_t workspace_floats, int total_rows,
                                      int num_cus, hipStream_t stream) {
  LLMLAB_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attention: %d heads, %d kv heads", nq, nkv);
  LLMLAB_REQUIRE(page_size > 0 && page_size % 16 == 0, "attention: page size %d is not a multiple of 16",
                 page_size);
  LLMLAB_REQUIRE(q_stride >= nq * D && out_stride >= nq * D, "attention: row strides too small");
  LLMLAB_REQUIRE(reqs >= 0 && reqs <= 65535 && nq <= 65535, "attention: grid too large");
  LLMLAB_REQUIRE(window >= 0, "attention: negative window");
  if (reqs == 0 || max_q_len <= 0) return 0;
  if (num_cus <= 0) num_cus = 256;
  AttnArgs a;
  a.q = q; a.kc = kcache; a.vc = vcache; a.table = table; a.q_start = q_start; a.start_pos = start_pos;
  a.out = out; a.o_part = nullptr; a.ml_part = nullptr;
  a.q_stride = q_stride; a.out_stride = out_stride; a.table_stride = table_stride; a.page_size = page_size;
  a.nq = nq; a.nkv = nkv; a.window = window; a.splits = 1; a.scale = scale;
  if (dtype == DT_F32) {
    dim3 grid(max_q_len, nq, reqs), block(64);
    hipLaunchKernelGGL(attention_f32_kernel, grid, block, 0, stream, a);
    LLMLAB_LAUNCH_CHECK("attention(float32)");
    return 0;
  }
  LLMLAB_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && out_stride % 4 == 0 &&
                 ((uintptr_t)out % 8 == 0) && ((uintptr_t)kcache % 16 == 0) && ((uintptr_t)vcache % 16 == 0),
                 "attention(bfloat16): operands are not aligned for vector loads");
  const int G = nq / nkv;
  const long max_rows = (long)max_q_len * G;
  if (max_rows <= 16) {
    // decode-like step: one wave per (request, kv head, split)
    int splits = 1;
    const long base = (long)reqs * nkv;
    const int visible = window > 0 ? min(window, max_ctx_len) : max_ctx_len;
    const int blocks32 = (visible + 31) / 32 + 1;
    if (base < 4L * num_cus) {
      splits = (int)((4L * num_cus + base - 1) / base);
      const int cap = blocks32 / 4 > 0 ? blocks32 / 4 : 1;   // at least 128 keys per split
      if (splits > cap) splits = cap;
      if (splits > 64) splits = 64;
      const size_t per_split = (size_t)total_rows * nq * (D + 2);
      while (splits > 1 && per_split * splits > workspace_floats) --splits;
    }
    a.splits = splits;
    if (splits > 1) {
      a.o_part = workspace;
      a.ml_part = workspace + (size_t)total_rows * nq * splits * D;
    }
    dim3 grid(1, nkv * splits, reqs), block(64);
    hipLaunchKernelGGL(attention_bf16_kernel<1>, grid, block, 0, stream, a);
    LLMLAB_LAUNCH_CHECK("attention(bfloat16, decode)");
    if (splits > 1) {
      dim3 mgrid(total_rows, nq), mblock(64);
      hipLaunchKernelGGL(attention_merge_kernel<bf16_t>, mgrid, mblock, 0, stream, a.o_part, a.ml_part,
                         (bf16_t*)out, out_stride, nq, splits);
      LLMLAB_LAUNCH_CHECK("attention merge");
    }
    return 0;
  }
  constexpr int QB = 2;
  const int rows_per_block = 4 * 16 * QB;
  dim3 grid((unsigned)((max_rows + rows_per_block - 1) / rows_per_block), nkv, reqs), block(256);
  hipLaunchKernelGGL(attention_bf16_kernel<QB>, grid, block, 0, stream, a);
  LLMLAB_LAUNCH_CHECK("attention(bfloat16, prefill)");
  return 0;
}
