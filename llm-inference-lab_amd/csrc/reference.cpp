// Plain C++ references of the operations the HIP kernels of this folder compute: one
// straightforward function per operation, for the host, in natural layouts, with sums in
// double precision.  Nothing here is on the product path: the tests hold every kernel
// against its function here (tests/test_cpp_reference_gpu.py) beside the PyTorch
// references.  Formulas as in the reference engine:
//   embedding                 rust/engine/src/runner/model/qwen2/kernels.rs:46-57
//   RMSNorm                   kernels.rs:546-582
//   linear (+ bias)           kernels.rs:393-420
//   rotary, split halves      kernels.rs:587-631
//   SwiGLU                    kernels.rs:1469-1486
//   causal GQA attention      kernels.rs:702-1452 (scores, mask, softmax, values)
//   argmax, ties to the first kernels.rs:1488-1552
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <limits>
#include <vector>

extern "C" {

// out[r, :] = table[ids[r], :]
void ref_embedding(const float* table, const int* ids, int rows, int hidden, float* out) {
  for (int r = 0; r < rows; ++r)
    for (int i = 0; i < hidden; ++i) out[(size_t)r * hidden + i] = table[(size_t)ids[r] * hidden + i];
}

// out[r, :] = x[r, :] * rsqrt(mean(x[r]^2) + eps) * w
void ref_rmsnorm(const float* x, const float* w, float eps, int rows, int hidden, float* out) {
  for (int r = 0; r < rows; ++r) {
    double ss = 0.0;
    for (int i = 0; i < hidden; ++i) ss += (double)x[(size_t)r * hidden + i] * x[(size_t)r * hidden + i];
    const double inv = 1.0 / std::sqrt(ss / hidden + (double)eps);
    for (int i = 0; i < hidden; ++i) out[(size_t)r * hidden + i] = (float)(x[(size_t)r * hidden + i] * inv * w[i]);
  }
}

// out[m, n] = sum_k x[m, k] w[n, k] (+ bias[n])
void ref_linear(const float* x, const float* w, const float* bias, int m, int n, int k, float* out) {
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      double s = bias ? (double)bias[j] : 0.0;
      for (int t = 0; t < k; ++t) s += (double)x[(size_t)i * k + t] * w[(size_t)j * k + t];
      out[(size_t)i * n + j] = (float)s;
    }
}

// x[r, h, :] rotated by position[r]: pairs (i, i + d/2), angle = position * theta^(-2i/d)
void ref_rope(float* x, const int* positions, int rows, int heads, int d, double theta) {
  const int half = d / 2;
  for (int r = 0; r < rows; ++r)
    for (int h = 0; h < heads; ++h) {
      float* v = x + ((size_t)r * heads + h) * d;
      for (int i = 0; i < half; ++i) {
        const double angle = (double)positions[r] * std::pow(theta, -2.0 * i / d);
        const double c = std::cos(angle), s = std::sin(angle);
        const double lo = v[i], hi = v[i + half];
        v[i] = (float)(lo * c - hi * s);
        v[i + half] = (float)(hi * c + lo * s);
      }
    }
}

// out = silu(gate) * up
void ref_swiglu(const float* gate, const float* up, int n, float* out) {
  for (int i = 0; i < n; ++i) out[i] = (float)((double)gate[i] / (1.0 + std::exp(-(double)gate[i])) * up[i]);
}

// Attention of a packed step over a paged cache in natural order: keys and values
// [pages][nkv][page_size][d]; request b brings the rows q_start[b] .. q_start[b+1]-1 at
// positions start_pos[b] + t and sees the keys lo .. position (lo = position - window + 1
// with a window, 0 without) through table[b][position / page_size].
void ref_paged_attention(const float* q, const float* keys, const float* values, const int* table,
                         int table_stride, int page_size, const int* q_start, const int* start_pos, int reqs,
                         int nq, int nkv, int d, int window, float scale, float* out) {
  const int group = nq / nkv;
  std::vector<double> p;
  for (int b = 0; b < reqs; ++b)
    for (int r = q_start[b]; r < q_start[b + 1]; ++r) {
      const int pos = start_pos[b] + (r - q_start[b]);
      const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
      for (int h = 0; h < nq; ++h) {
        const int kvh = h / group;
        const float* qv = q + ((size_t)r * nq + h) * d;
        p.assign(pos - lo + 1, 0.0);
        double mx = -std::numeric_limits<double>::infinity();
        for (int j = lo; j <= pos; ++j) {
          const int page = table[(size_t)b * table_stride + j / page_size];
          const float* kv = keys + (((size_t)page * nkv + kvh) * page_size + j % page_size) * d;
          double s = 0.0;
          for (int i = 0; i < d; ++i) s += (double)qv[i] * kv[i];
          p[j - lo] = s * scale;
          if (p[j - lo] > mx) mx = p[j - lo];
        }
        double den = 0.0;
        for (double& v : p) {
          v = std::exp(v - mx);
          den += v;
        }
        float* o = out + ((size_t)r * nq + h) * d;
        for (int i = 0; i < d; ++i) {
          double s = 0.0;
          for (int j = lo; j <= pos; ++j) {
            const int page = table[(size_t)b * table_stride + j / page_size];
            s += p[j - lo] * values[(((size_t)page * nkv + kvh) * page_size + j % page_size) * d + i];
          }
          o[i] = (float)(s / den);
        }
      }
    }
}

// the index of the largest logit, the first of equals; -1 for a row without a number
int ref_argmax(const float* logits, int vocab) {
  int best = -1;
  for (int i = 0; i < vocab; ++i)
    if (!std::isnan(logits[i]) && (best < 0 || logits[i] > logits[best])) best = i;
  return best;
}

// probs = softmax(logits / temperature)
void ref_softmax(const float* logits, int vocab, float temperature, double* probs) {
  double mx = -std::numeric_limits<double>::infinity();
  for (int i = 0; i < vocab; ++i)
    if ((double)logits[i] / temperature > mx) mx = (double)logits[i] / temperature;
  double den = 0.0;
  for (int i = 0; i < vocab; ++i) den += std::exp((double)logits[i] / temperature - mx);
  for (int i = 0; i < vocab; ++i) probs[i] = std::exp((double)logits[i] / temperature - mx) / den;
}

// the first token at which the cumulative probability of softmax(logits / temperature)
// reaches u, tokens of probability 0 never (the last token with a probability if rounding
// leaves the sum below u)
int ref_sample(const float* logits, int vocab, float temperature, float u) {
  std::vector<double> probs(vocab);
  ref_softmax(logits, vocab, temperature, probs.data());
  double cum = 0.0;
  int last = -1;
  for (int i = 0; i < vocab; ++i) {
    if (probs[i] > 0.0) {
      last = i;
      cum += probs[i];
      if (cum >= (double)u) return i;
    }
  }
  return last;
}

}  // extern "C"
