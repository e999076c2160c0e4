// Plain C++ twins of the kernels: each function is the definition its kernel is held to, written from the
// reference's formulas in double precision, one element at a time, sharing nothing with the kernels.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <vector>

namespace plain {

// y_i = x_i * rsqrt(mean(x^2) + eps) * w_i: eps on the mean square (reference: engine/kernels/rmsnorm.cu:26-40).
inline std::vector<double> rmsnorm(const std::vector<double>& x, const std::vector<double>& w, double eps) {
  double ss = 0.0;
  for (double v : x) ss += v * v;
  const double s = 1.0 / std::sqrt(ss / static_cast<double>(x.size()) + eps);
  std::vector<double> y(x.size());
  for (size_t i = 0; i < x.size(); ++i) y[i] = x[i] * s * w[i];
  return y;
}

// Rotate-half pairing over the whole head: (v[p], v[p + d/2]) turned by pos * theta^(-2p/d)
// (reference: engine/kernels/rope.cu:18-55).
inline void rope(double* v, int d, int pos, double theta) {
  for (int p = 0; p < d / 2; ++p) {
    const double a = static_cast<double>(pos) * std::pow(theta, -2.0 * p / d);
    const double lo = v[p], hi = v[p + d / 2];
    v[p] = lo * std::cos(a) - hi * std::sin(a);
    v[p + d / 2] = hi * std::cos(a) + lo * std::sin(a);
  }
}

// out[m][n] = sum_k a[m][k] * w[n][k]: weights stored [out, in] (reference: engine/include/llm/kernels.h:48-57).
inline std::vector<double> gemm(const std::vector<double>& a, const std::vector<double>& w, int m, int n, int k) {
  std::vector<double> out(static_cast<size_t>(m) * n, 0.0);
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      double s = 0.0;
      for (int c = 0; c < k; ++c) s += a[static_cast<size_t>(i) * k + c] * w[static_cast<size_t>(j) * k + c];
      out[static_cast<size_t>(i) * n + j] = s;
    }
  return out;
}

// silu(g) * u, silu(g) = g / (1 + exp(-g)) (reference: engine/kernels/swiglu.cu:22-23).
inline double swiglu(double g, double u) { return g / (1.0 + std::exp(-g)) * u; }

// One row's causal attention: scores q.k / sqrt(d) over keys lo .. pos, softmax, weighted sum of the values
// (reference: engine/kernels/attention_qk.cu:25-68, softmax.cu:28-42, attention_av.cu:32-45).  keys/values:
// [position][d] of the row's key/value head.
inline std::vector<double> attend(const double* q, const std::vector<const double*>& keys,
                                  const std::vector<const double*>& values, int d, int lo, int pos, double scale) {
  std::vector<double> s(pos - lo + 1);
  double mx = -INFINITY;
  for (int j = lo; j <= pos; ++j) {
    double dot = 0.0;
    for (int c = 0; c < d; ++c) dot += q[c] * keys[j][c];
    s[j - lo] = dot * scale;
    mx = std::max(mx, s[j - lo]);
  }
  double total = 0.0;
  for (double& e : s) total += (e = std::exp(e - mx));
  std::vector<double> o(d, 0.0);
  for (int j = lo; j <= pos; ++j)
    for (int c = 0; c < d; ++c) o[c] += s[j - lo] / total * values[j][c];
  return o;
}

// The lowest index of the maximum (reference: engine/kernels/logits_argmax.cu:22-65).
inline int argmax(const std::vector<float>& row) {
  return static_cast<int>(std::max_element(row.begin(), row.end()) - row.begin());
}

// The sampling law (reference: engine/src/sampler.cpp:36-104): weights exp((l - max) / T) in float, their sums
// in double, one uniform number u.  Without a limit the token is the first, in the order of the ids, at which
// u * total minus the running sum turns negative; with top-k / top-p the likeliest tokens (lower id first among
// equals) are walked instead, top-p measured on the top-k set.
inline int sample(const std::vector<float>& logits, float temperature, int top_k, double top_p, double u) {
  const int vocab = static_cast<int>(logits.size());
  const float mx = *std::max_element(logits.begin(), logits.end());
  const float inv_t = 1.0f / temperature;
  std::vector<double> w(vocab);
  double total = 0.0;
  for (int i = 0; i < vocab; ++i) total += (w[i] = static_cast<double>(std::exp((logits[i] - mx) * inv_t)));
  const int k = top_k > 0 ? std::min(top_k, vocab) : vocab;
  if (k == vocab && !(top_p < 1.0)) {
    double left = u * total;
    for (int i = 0; i < vocab; ++i)
      if ((left -= w[i]) < 0.0) return i;
    return argmax(logits);
  }
  std::vector<int> order(vocab);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return w[a] > w[b]; });
  int keep = k;
  if (top_p < 1.0) {
    double kept_total = 0.0, cum = 0.0;
    for (int j = 0; j < k; ++j) kept_total += w[order[j]];
    for (int j = 0; j < k; ++j)
      if ((cum += w[order[j]]) >= top_p * kept_total) {
        keep = j + 1;
        break;
      }
  }
  double mass = 0.0;
  for (int j = 0; j < keep; ++j) mass += w[order[j]];
  double left = u * mass;
  for (int j = 0; j < keep; ++j)
    if ((left -= w[order[j]]) < 0.0) return order[j];
  return order[keep - 1];
}

}  // namespace plain
