#include "reference.h"

#include <algorithm>
#include <cmath>
#include <vector>

extern "C" void ref_embed_gather(const float* table, const int* ids, float* out, int T, int D) {
  for (int t = 0; t < T; ++t)
    for (int d = 0; d < D; ++d) out[(size_t)t * D + d] = table[(size_t)ids[t] * D + d];
}

extern "C" void ref_add_rmsnorm(float* h, const float* delta, int n_planes, long long plane_stride, const float* gamma,
                                float* out, const int* rows, int n_out, int D, float eps, int write_h) {
  std::vector<double> v(D);
  for (int i = 0; i < n_out; ++i) {
    const int r = rows ? rows[i] : i;
    double ss = 0.0;
    for (int d = 0; d < D; ++d) {
      double x = h[(size_t)r * D + d];
      if (delta)
        for (int p = 0; p < n_planes; ++p) x += delta[(size_t)p * plane_stride + (size_t)r * D + d];
      v[d] = x;
      ss += x * x;
    }
    const double inv = 1.0 / std::sqrt(ss / D + (double)eps);
    for (int d = 0; d < D; ++d) {
      if (delta && write_h) h[(size_t)r * D + d] = (float)v[d];
      out[(size_t)i * D + d] = (float)(v[d] * inv * gamma[d]);
    }
  }
}

extern "C" void ref_rope_kv_write(float* qkv, const int* positions, const int* token_seq, const int* block_table,
                                  int table_width, const float* cos_sin, float* kcache, float* vcache, int page_size,
                                  int T, int nh, int nkv, int hd, int pairing) {
  const int half = hd / 2, row_len = (nh + 2 * nkv) * hd;
  for (int t = 0; t < T; ++t) {
    const int b = token_seq[t];
    if (b < 0) continue;
    const int pos = positions[t];
    const int page = block_table[(size_t)b * table_width + pos / page_size], at = pos % page_size;
    float* row = qkv + (size_t)t * row_len;
    for (int head = 0; head < nh + nkv; ++head) {
      float* x = row + (size_t)head * hd;
      for (int i = 0; i < half; ++i) {
        const int i0 = pairing == 0 ? 2 * i : i, i1 = pairing == 0 ? 2 * i + 1 : i + half;
        const double c = cos_sin[((size_t)pos * half + i) * 2], s = cos_sin[((size_t)pos * half + i) * 2 + 1];
        const double x0 = x[i0], x1 = x[i1];
        x[i0] = (float)(x0 * c - x1 * s);
        x[i1] = (float)(x0 * s + x1 * c);
      }
      if (head >= nh && page >= 0)
        for (int d = 0; d < hd; ++d) kcache[(((size_t)page * nkv + (head - nh)) * page_size + at) * hd + d] = x[d];
    }
    if (page >= 0)
      for (int kv = 0; kv < nkv; ++kv)
        for (int d = 0; d < hd; ++d)
          vcache[(((size_t)page * nkv + kv) * hd + d) * page_size + at] = row[(size_t)(nh + nkv + kv) * hd + d];
  }
}

extern "C" void ref_swiglu(const float* gate_up, float* out, int T, int I) {
  for (int t = 0; t < T; ++t)
    for (int i = 0; i < I; ++i) {
      const double g = gate_up[(size_t)t * 2 * I + i], u = gate_up[(size_t)t * 2 * I + I + i];
      out[(size_t)t * I + i] = (float)(g / (1.0 + std::exp(-g)) * u);
    }
}

extern "C" void ref_attention(const float* q, int q_row_stride, float* out, const int* positions, const int* token_seq,
                              const int* block_table, int table_width, const float* kcache, const float* vcache,
                              int page_size, int T, int nh, int nkv, int hd, float scale, int window) {
  const int group = nh / nkv;
  std::vector<double> score, acc(hd);
  for (int t = 0; t < T; ++t) {
    const int b = token_seq[t];
    for (int h = 0; h < nh; ++h) {
      float* o = out + ((size_t)t * nh + h) * hd;
      if (b < 0) {
        std::fill(o, o + hd, 0.f);
        continue;
      }
      const int pos = positions[t], kv = h / group;
      const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
      const float* qh = q + (size_t)t * q_row_stride + (size_t)h * hd;
      score.assign(pos - first + 1, 0.0);
      double top = -INFINITY;
      for (int j = first; j <= pos; ++j) {
        const int page = block_table[(size_t)b * table_width + j / page_size], at = j % page_size;
        const float* k = kcache + (((size_t)page * nkv + kv) * page_size + at) * hd;
        double s = 0.0;
        for (int d = 0; d < hd; ++d) s += (double)qh[d] * k[d];
        score[j - first] = s * scale;
        top = std::max(top, score[j - first]);
      }
      double sum = 0.0;
      std::fill(acc.begin(), acc.end(), 0.0);
      for (int j = first; j <= pos; ++j) {
        const int page = block_table[(size_t)b * table_width + j / page_size], at = j % page_size;
        const double p = std::exp(score[j - first] - top);
        sum += p;
        for (int d = 0; d < hd; ++d) acc[d] += p * vcache[(((size_t)page * nkv + kv) * hd + d) * page_size + at];
      }
      for (int d = 0; d < hd; ++d) o[d] = (float)(acc[d] / sum);
    }
  }
}

extern "C" void ref_linear(const float* A, const float* W, float* C, int M, int N, int K) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double s = 0.0;
      for (int k = 0; k < K; ++k) s += (double)A[(size_t)m * K + k] * W[(size_t)n * K + k];
      C[(size_t)m * N + n] = (float)s;
    }
}

extern "C" void ref_gated_linear(const float* A, const float* W, float* C, int M, int I, int K) {
  for (int m = 0; m < M; ++m)
    for (int i = 0; i < I; ++i) {
      double g = 0.0, u = 0.0;
      for (int k = 0; k < K; ++k) {
        g += (double)A[(size_t)m * K + k] * W[(size_t)i * K + k];
        u += (double)A[(size_t)m * K + k] * W[(size_t)(I + i) * K + k];
      }
      C[(size_t)m * I + i] = (float)(g / (1.0 + std::exp(-g)) * u);
    }
}

extern "C" void ref_argmax(const float* logits, int* out, int R, int V, int ld) {
  for (int r = 0; r < R; ++r) {
    int best = 0;
    for (int v = 1; v < V; ++v)
      if (logits[(size_t)r * ld + v] > logits[(size_t)r * ld + best]) best = v;
    out[r] = best;
  }
}

extern "C" void ref_sample(const float* logits, const float* uniforms, int* out, int R, int V, int ld, float temperature,
                           float top_p) {
  std::vector<double> p(V);
  std::vector<int> order(V);
  std::vector<char> kept(V);
  for (int r = 0; r < R; ++r) {
    const float* x = logits + (size_t)r * ld;
    double top = -INFINITY, sum = 0.0;
    for (int v = 0; v < V; ++v) top = std::max(top, (double)x[v]);
    for (int v = 0; v < V; ++v) sum += p[v] = std::exp(((double)x[v] - top) / temperature);
    for (int v = 0; v < V; ++v) { p[v] /= sum; order[v] = v; }
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return p[a] > p[b]; });
    std::fill(kept.begin(), kept.end(), 0);
    double before = 0.0, mass = 0.0;   // mass of the tokens strictly more likely than the current one
    for (int i = 0; i < V;) {
      int j = i;
      double tied = 0.0;
      while (j < V && p[order[j]] == p[order[i]]) tied += p[order[j++]];
      if (!(before < top_p)) break;
      for (int k = i; k < j; ++k) kept[order[k]] = 1;   // tokens tied with a kept one are kept too
      mass += tied;
      before += tied;
      i = j;
    }
    const double target = (double)uniforms[r] * mass;
    double run = 0.0;
    int pick = -1, last = 0;
    for (int v = 0; v < V && pick < 0; ++v)
      if (kept[v]) {
        run += p[v];
        last = v;
        if (run > target) pick = v;
      }
    out[r] = pick < 0 ? last : pick;
  }
}
