// Every kernel family of the library beside its plain C++ twin (plain.h): a test is a function that returns
// false on failure, the program a main() that runs the tests named on its command line (all of them without
// names; --list prints the names) and returns non-zero if one fails -- no test framework, as in the reference's
// engine/tests (engine/CMakeLists.txt:47-65: one executable a test, add_test, a time limit).  Sizes are small and
// unlike any model's: no power of two, rows gathered in another order, pages handed out of order.
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <utility>
#include <vector>

#include "harness.h"
#include "plain.h"

using namespace twin;

namespace {

void* const kStream = nullptr;        // the default stream
const double kBf16 = 1.0 / 128.0;     // a bfloat16 value's rounding, and then some

std::vector<double> take(const std::vector<double>& v, size_t from, size_t n) {
  return std::vector<double>(v.begin() + from, v.begin() + from + n);
}

bool embed() {
  Rng rng(1);
  const int vocab = 50, hidden = 24, n = 7;
  const std::vector<float> table = normals(rng, static_cast<size_t>(vocab) * hidden);
  std::vector<int32_t> ids(n);
  for (int32_t& i : ids) i = rng.below(vocab);
  ids[0] = vocab - 1;
  bool ok = true;
  for (int dtype = 0; dtype < 2; ++dtype) {
    const std::vector<bf16> rounded = as_bf16(table);
    const std::vector<double> source = dtype ? widen(rounded) : widen(table);
    Dev<float> t32(table);
    Dev<bf16> t16(rounded);
    Dev<int32_t> di(ids);
    Dev<float> out(static_cast<size_t>(n) * hidden);
    RUN(bc4g_embed_gather(dtype ? static_cast<const void*>(t16.p) : t32.p, dtype, di.p, out.p, n, hidden, vocab, kStream));
    std::vector<double> want;
    for (int r = 0; r < n; ++r)
      for (int c = 0; c < hidden; ++c) want.push_back(source[static_cast<size_t>(ids[r]) * hidden + c]);
    ok &= close(dtype ? "rows of a bfloat16 table" : "rows of a float table", widen(out.get()), want, 0.0, 0.0);
  }
  return ok;
}

bool rmsnorm() {
  Rng rng(2);
  const int n = 6, hidden = 40, m = 3;
  const float eps = 1e-3f;
  const std::vector<float> x = normals(rng, static_cast<size_t>(n) * hidden, 3.0f);
  std::vector<float> w = normals(rng, hidden, 0.2f);
  for (float& v : w) v += 1.0f;
  const std::vector<int32_t> rows = {3, 0, 5};
  bool ok = true;
  for (int w_dtype = 0; w_dtype < 2; ++w_dtype)
    for (int out_dtype = 0; out_dtype < 2; ++out_dtype) {
      const std::vector<double> scale = w_dtype ? widen(as_bf16(w)) : widen(w);
      Dev<float> dx(x);
      Dev<float> w32(w);
      Dev<bf16> w16(as_bf16(w));
      Dev<int32_t> dr(rows);
      Dev<float> o32(static_cast<size_t>(m) * hidden);
      Dev<bf16> o16(static_cast<size_t>(m) * hidden);
      RUN(bc4g_rmsnorm(dx.p, dr.p, w_dtype ? static_cast<const void*>(w16.p) : w32.p, w_dtype,
                       out_dtype ? static_cast<void*>(o16.p) : o32.p, out_dtype, m, hidden, eps, kStream));
      std::vector<double> want;
      for (int r = 0; r < m; ++r) {
        const std::vector<double> y = plain::rmsnorm(take(widen(x), static_cast<size_t>(rows[r]) * hidden, hidden), scale, eps);
        want.insert(want.end(), y.begin(), y.end());
      }
      const std::vector<double> got = out_dtype ? widen(o16.get()) : widen(o32.get());
      ok &= close("gathered rows", got, want, out_dtype ? kBf16 : 1e-5, 1e-6);
    }
  return ok;
}

bool swiglu() {
  Rng rng(3);
  const int n = 5, inter = 24;
  const std::vector<float> gu = normals(rng, static_cast<size_t>(n) * 2 * inter, 2.0f);
  bool ok = true;
  for (int dtype = 0; dtype < 2; ++dtype)
    for (int interleaved = 0; interleaved < 2; ++interleaved) {
      const std::vector<double> in = dtype ? widen(as_bf16(gu)) : widen(gu);
      Dev<float> g32(gu), o32(static_cast<size_t>(n) * inter);
      Dev<bf16> g16(as_bf16(gu)), o16(static_cast<size_t>(n) * inter);
      RUN(bc4g_swiglu(dtype ? static_cast<const void*>(g16.p) : g32.p, dtype ? static_cast<void*>(o16.p) : o32.p, dtype, n,
                      inter, interleaved, kStream));
      std::vector<double> want;
      for (int t = 0; t < n; ++t)
        for (int i = 0; i < inter; ++i) {
          const size_t row = static_cast<size_t>(t) * 2 * inter;
          // interleaved: blocks of 16 = eight gates, then the eight ups of the same outputs
          const size_t g = interleaved ? row + (i / 8) * 16 + i % 8 : row + i;
          const size_t u = interleaved ? g + 8 : row + inter + i;
          want.push_back(plain::swiglu(in[g], in[u]));
        }
      ok &= close(interleaved ? "interleaved" : "gates then ups", dtype ? widen(o16.get()) : widen(o32.get()), want,
                  dtype ? kBf16 : 1e-5, 1e-6);
    }
  return ok;
}

bool gemm_generic() {
  Rng rng(4);
  bool ok = true;
  const int n = 33, k = 50;
  for (int m : {3, 20}) {            // the small tile (a decode step) and the large one
    const std::vector<float> a = normals(rng, static_cast<size_t>(m) * k), w = normals(rng, static_cast<size_t>(n) * k);
    const std::vector<float> before = normals(rng, static_cast<size_t>(m) * n);
    {   // float x float -> float, and added into a float output
      Dev<float> da(a), dw(w), out(static_cast<size_t>(m) * n), acc(before);
      RUN(bc4g_gemm_generic(da.p, 0, dw.p, 0, out.p, 0, 0, m, n, k, kStream));
      RUN(bc4g_gemm_generic(da.p, 0, dw.p, 0, acc.p, 0, 1, m, n, k, kStream));
      const std::vector<double> want = plain::gemm(widen(a), widen(w), m, n, k);
      ok &= close("float product", widen(out.get()), want, 1e-5, 1e-5);
      std::vector<double> sum = want;
      for (size_t i = 0; i < sum.size(); ++i) sum[i] += before[i];
      ok &= close("float product added", widen(acc.get()), sum, 1e-5, 1e-5);
    }
    {   // bfloat16 x bfloat16 -> float
      Dev<bf16> da(as_bf16(a)), dw(as_bf16(w));
      Dev<float> out(static_cast<size_t>(m) * n);
      RUN(bc4g_gemm_generic(da.p, 1, dw.p, 1, out.p, 0, 0, m, n, k, kStream));
      ok &= close("bfloat16 product", widen(out.get()), plain::gemm(widen(as_bf16(a)), widen(as_bf16(w)), m, n, k), 1e-5, 1e-5);
    }
  }
  return ok;
}

bool gemm_skinny() {
  Rng rng(5);
  bool ok = true;
  const int n = 48, k = 104;        // k no multiple of a 32-wide step: the packed weight ends in zeros
  const std::vector<bf16> w = as_bf16(normals(rng, static_cast<size_t>(n) * k, 0.5f));
  Dev<bf16> packed(pack_weight(w, n, k));
  for (int m : {1, 9, 33, 64}) {
    const std::vector<bf16> x = as_bf16(normals(rng, static_cast<size_t>(m) * k));
    const std::vector<float> before = normals(rng, static_cast<size_t>(m) * n);
    const std::vector<double> want = plain::gemm(widen(x), widen(w), m, n, k);
    Dev<bf16> dx(x), o16(static_cast<size_t>(m) * n), act(static_cast<size_t>(m) * n / 2);
    Dev<float> o32(static_cast<size_t>(m) * n), acc(before);
    RUN(bc4g_gemm_skinny(dx.p, packed.p, o16.p, 0, m, n, k, kStream));
    RUN(bc4g_gemm_skinny(dx.p, packed.p, o32.p, 1, m, n, k, kStream));
    RUN(bc4g_gemm_skinny(dx.p, packed.p, acc.p, 2, m, n, k, kStream));
    RUN(bc4g_gemm_skinny(dx.p, packed.p, act.p, 3, m, n, k, kStream));
    ok &= close("bfloat16 out", widen(o16.get()), want, kBf16, 1e-2);
    ok &= close("float out", widen(o32.get()), want, 1e-4, 1e-4);
    std::vector<double> sum = want, gated;
    for (size_t i = 0; i < sum.size(); ++i) sum[i] += before[i];
    ok &= close("added to a float stream", widen(acc.get()), sum, 1e-4, 1e-4);
    for (int r = 0; r < m; ++r)           // every 16 rows of w: eight gate rows, then the eight up rows of the same outputs
      for (int i = 0; i < n / 2; ++i) {
        const size_t g = static_cast<size_t>(r) * n + (i / 8) * 16 + i % 8;
        gated.push_back(plain::swiglu(want[g], want[g + 8]));
      }
    ok &= close("SwiGLU", widen(act.get()), gated, kBf16, 1e-2);
  }
  return ok;
}

bool gemm_skinny_norms() {
  // The RMSNorm fused into the product, and the norm that the adding product before prepares for it.
  Rng rng(6);
  bool ok = true;
  const int m = 7, hidden = 64, n = 80;
  const float eps = 1e-5f;
  const std::vector<float> stream = normals(rng, static_cast<size_t>(m + 2) * hidden, 2.0f);
  std::vector<float> g = normals(rng, hidden, 0.2f);
  for (float& v : g) v += 1.0f;
  const std::vector<bf16> w = as_bf16(normals(rng, static_cast<size_t>(n) * hidden, 0.3f));
  const std::vector<int32_t> rows = {8, 1, 0, 5, 4, 3, 2};
  Dev<bf16> packed(pack_weight(w, n, hidden));
  Dev<float> dstream(stream), dg(g), out(static_cast<size_t>(m) * n);
  Dev<int32_t> drows(rows);
  RUN(bc4g_gemm_skinny_normed(dstream.p, drows.p, dg.p, 0, eps, packed.p, out.p, 1, m, n, hidden, kStream));
  std::vector<double> normed;
  for (int r = 0; r < m; ++r) {
    const std::vector<double> y = plain::rmsnorm(take(widen(stream), static_cast<size_t>(rows[r]) * hidden, hidden), widen(g), eps);
    normed.insert(normed.end(), y.begin(), y.end());
  }
  // (the kernel rounds x * g to bfloat16 before the matrix cores: a bfloat16's rounding over a sum of `hidden` terms)
  ok &= close("norm fused", widen(out.get()), plain::gemm(normed, widen(w), m, n, hidden), 2e-2, 2e-2 * std::sqrt(static_cast<double>(hidden)) * 0.3);

  // residual += x w1^T, the norm after it prepared; then the product that finishes that norm
  const int k1 = 96, n2 = 48;
  const std::vector<bf16> x = as_bf16(normals(rng, static_cast<size_t>(m) * k1));
  const std::vector<bf16> w1 = as_bf16(normals(rng, static_cast<size_t>(hidden) * k1, 0.3f));
  const std::vector<bf16> w2 = as_bf16(normals(rng, static_cast<size_t>(n2) * hidden, 0.3f));
  const std::vector<float> residual = normals(rng, static_cast<size_t>(m) * hidden, 2.0f);
  Dev<bf16> dx(x), p1(pack_weight(w1, hidden, k1)), p2(pack_weight(w2, n2, hidden)), emit_x(static_cast<size_t>(m) * hidden);
  Dev<float> dres(residual), ssq(static_cast<size_t>((hidden + 15) / 16) * m), y(static_cast<size_t>(m) * n2);
  RUN(bc4g_gemm_skinny_emit(dx.p, p1.p, dres.p, dg.p, 0, emit_x.p, ssq.p, m, m, hidden, k1, kStream));
  RUN(bc4g_gemm_skinny_prenormed(emit_x.p, ssq.p, (hidden + 15) / 16, m, eps, p2.p, y.p, 1, m, n2, hidden, kStream));
  std::vector<double> after = plain::gemm(widen(x), widen(w1), m, hidden, k1);
  for (size_t i = 0; i < after.size(); ++i) after[i] += residual[i];
  ok &= close("stream after the adding product", widen(dres.get()), after, 1e-4, 1e-4);
  std::vector<double> normed2;
  for (int r = 0; r < m; ++r) {
    const std::vector<double> row = plain::rmsnorm(take(after, static_cast<size_t>(r) * hidden, hidden), widen(g), eps);
    normed2.insert(normed2.end(), row.begin(), row.end());
  }
  ok &= close("norm prepared by the product before", widen(y.get()), plain::gemm(normed2, widen(w2), m, n2, hidden), 2e-2,
              2e-2 * std::sqrt(static_cast<double>(hidden)) * 0.3);
  // ... and the tiled SwiGLU product that finishes the same prepared norm (every 16 rows of its weight: eight gate
  // rows, then the eight up rows of the same outputs)
  const int n3 = 96;
  const std::vector<bf16> w3 = as_bf16(normals(rng, static_cast<size_t>(n3) * hidden, 0.3f));
  Dev<bf16> p3(pack_weight(w3, n3, hidden)), act(static_cast<size_t>(m) * n3 / 2);
  RUN(bc4g_gemm_mfma_swiglu_scaled(emit_x.p, ssq.p, (hidden + 15) / 16, m, eps, p3.p, 1, act.p, m, n3, hidden, kStream));
  const std::vector<double> gu = plain::gemm(normed2, widen(w3), m, n3, hidden);
  std::vector<double> gated;
  for (int r = 0; r < m; ++r)
    for (int i = 0; i < n3 / 2; ++i) {
      const size_t at = static_cast<size_t>(r) * n3 + (i / 8) * 16 + i % 8;
      gated.push_back(plain::swiglu(gu[at], gu[at + 8]));
    }
  ok &= close("SwiGLU over the prepared norm", widen(act.get()), gated, 3e-2, 3e-2 * std::sqrt(static_cast<double>(hidden)) * 0.3);
  return ok;
}

bool gemm_mfma() {
  Rng rng(7);
  bool ok = true;
  const int m = 150, n = 192, k = 128;
  const std::vector<bf16> a = as_bf16(normals(rng, static_cast<size_t>(m) * k)), w = as_bf16(normals(rng, static_cast<size_t>(n) * k, 0.5f));
  const std::vector<float> before = normals(rng, static_cast<size_t>(m) * n);
  const std::vector<double> want = plain::gemm(widen(a), widen(w), m, n, k);
  Dev<bf16> da(a), rows(w), packed(pack_weight(w, n, k));
  for (int w_packed = 0; w_packed < 2; ++w_packed) {       // the weight by rows (tiles staged through registers) and packed (straight into LDS)
    const void* dw = w_packed ? packed.p : rows.p;
    Dev<bf16> o16(static_cast<size_t>(m) * n), act(static_cast<size_t>(m) * n / 2);
    Dev<float> o32(static_cast<size_t>(m) * n), acc(before);
    RUN(bc4g_gemm_mfma(da.p, dw, w_packed, o16.p, 0, m, n, k, kStream));
    RUN(bc4g_gemm_mfma(da.p, dw, w_packed, o32.p, 1, m, n, k, kStream));
    RUN(bc4g_gemm_mfma(da.p, dw, w_packed, acc.p, 2, m, n, k, kStream));
    RUN(bc4g_gemm_mfma(da.p, dw, w_packed, act.p, 3, m, n, k, kStream));
    ok &= close("bfloat16 out", widen(o16.get()), want, kBf16, 1e-2);
    ok &= close("float out", widen(o32.get()), want, 1e-4, 1e-4);
    std::vector<double> sum = want, gated;
    for (size_t i = 0; i < sum.size(); ++i) sum[i] += before[i];
    ok &= close("added to a float stream", widen(acc.get()), sum, 1e-4, 1e-4);
    for (int r = 0; r < m; ++r)
      for (int i = 0; i < n / 2; ++i) {
        const size_t g = static_cast<size_t>(r) * n + (i / 8) * 16 + i % 8;
        gated.push_back(plain::swiglu(want[g], want[g + 8]));
      }
    ok &= close("SwiGLU", widen(act.get()), gated, kBf16, 1e-2);
  }
  // k cut into parts over workgroups, and the kernel that adds the parts to the stream and norms it
  const int rows_few = 20, width = 128, depth = 256, parts = 2;
  const float eps = 1e-5f;
  const std::vector<bf16> x = as_bf16(normals(rng, static_cast<size_t>(rows_few) * depth)), wo = as_bf16(normals(rng, static_cast<size_t>(width) * depth, 0.3f));
  const std::vector<float> residual = normals(rng, static_cast<size_t>(rows_few) * width, 2.0f);
  std::vector<float> g = normals(rng, width, 0.2f);
  for (float& v : g) v += 1.0f;
  Dev<bf16> dx(x), pw(pack_weight(wo, width, depth)), normed(static_cast<size_t>(rows_few) * width);
  Dev<float> dparts(static_cast<size_t>(parts) * rows_few * width), dres(residual), dg(g);
  RUN(bc4g_gemm_mfma_parts(dx.p, pw.p, 1, dparts.p, rows_few, width, depth, parts, kStream));
  RUN(bc4g_rmsnorm_sum(dres.p, dparts.p, parts, dg.p, 0, normed.p, 1, rows_few, width, eps, kStream));
  std::vector<double> after = plain::gemm(widen(x), widen(wo), rows_few, width, depth), y;
  for (size_t i = 0; i < after.size(); ++i) after[i] += residual[i];
  ok &= close("stream after the parts were added", widen(dres.get()), after, 1e-4, 1e-4);
  for (int r = 0; r < rows_few; ++r) {
    const std::vector<double> row = plain::rmsnorm(take(after, static_cast<size_t>(r) * width, width), widen(g), eps);
    y.insert(y.end(), row.begin(), row.end());
  }
  ok &= close("its norm", widen(normed.get()), y, kBf16, 1e-3);
  return ok;
}

// A step of some requests over a paged cache: which rows, which positions, where their keys and values go.
struct Paged {
  int n_seqs, page, pages_per_seq, num_pages;
  std::vector<int32_t> table;                     // [n_seqs][pages_per_seq], pages handed out of order
  Paged(int seqs, int page_tokens, int longest, Rng& rng)
      : n_seqs(seqs), page(page_tokens), pages_per_seq((longest + page_tokens - 1) / page_tokens) {
    num_pages = n_seqs * pages_per_seq + 3;
    std::vector<int32_t> free_pages(num_pages);
    for (int i = 0; i < num_pages; ++i) free_pages[i] = i;
    for (int i = num_pages - 1; i > 0; --i) std::swap(free_pages[i], free_pages[rng.below(i + 1)]);
    table.assign(free_pages.begin(), free_pages.begin() + n_seqs * pages_per_seq);
  }
  int32_t slot(int seq, int pos) const { return table[seq * pages_per_seq + pos / page] * page + pos % page; }
};

// Every row's attention by the twin: rows (request, position) with queries q [row][nh][d] (not yet rotated);
// keys and values of every request and position kv[seq][pos] = (k [nkv][d], v [nkv][d]), keys not yet rotated.
std::vector<double> twin_attention(const std::vector<std::pair<int, int>>& rows, const std::vector<std::vector<double>>& q,
                                   const std::vector<std::vector<std::vector<double>>>& keys,
                                   const std::vector<std::vector<std::vector<double>>>& values, int nh, int nkv, int d,
                                   double theta, int window, bool round_bf16) {
  auto rounded = [&](double v) { return round_bf16 ? static_cast<double>(from_bf16(to_bf16(static_cast<float>(v)))) : v; };
  std::vector<std::vector<std::vector<double>>> turned = keys;       // the keys as the cache holds them: rotated
  for (auto& seq : turned)
    for (size_t pos = 0; pos < seq.size(); ++pos)
      for (int h = 0; h < nkv; ++h) {
        plain::rope(&seq[pos][static_cast<size_t>(h) * d], d, static_cast<int>(pos), theta);
        for (int c = 0; c < d; ++c) seq[pos][static_cast<size_t>(h) * d + c] = rounded(seq[pos][static_cast<size_t>(h) * d + c]);
      }
  std::vector<double> out;
  for (size_t r = 0; r < rows.size(); ++r) {
    const int seq = rows[r].first, pos = rows[r].second;
    const int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    for (int h = 0; h < nh; ++h) {
      std::vector<double> qh(q[r].begin() + static_cast<size_t>(h) * d, q[r].begin() + static_cast<size_t>(h + 1) * d);
      plain::rope(qh.data(), d, pos, theta);
      for (double& v : qh) v = rounded(v);
      const int kvh = h / (nh / nkv);
      std::vector<const double*> kp, vp;
      for (int j = 0; j <= pos; ++j) {
        kp.push_back(&turned[seq][j][static_cast<size_t>(kvh) * d]);
        vp.push_back(&values[seq][j][static_cast<size_t>(kvh) * d]);
      }
      const std::vector<double> o = plain::attend(qh.data(), kp, vp, d, lo, pos, 1.0 / std::sqrt(static_cast<double>(d)));
      out.insert(out.end(), o.begin(), o.end());
    }
  }
  return out;
}

bool attention_generic() {
  // float32, the plain cache layout, a head size that is no multiple of 16: two requests' whole prompts in one step
  Rng rng(8);
  const int nh = 4, nkv = 2, d = 24, page = 8, width = (nh + 2 * nkv) * d;
  const float theta = 10000.0f;
  const std::vector<int> lengths = {19, 11};
  Paged paged(2, page, 19, rng);
  std::vector<std::pair<int, int>> rows;
  for (int s = 0; s < 2; ++s)
    for (int p = 0; p < lengths[s]; ++p) rows.push_back({s, p});
  const int t = static_cast<int>(rows.size());
  const std::vector<float> qkv = normals(rng, static_cast<size_t>(t) * width);
  std::vector<int32_t> positions, slots, row_seq;
  std::vector<std::vector<double>> q(t);
  std::vector<std::vector<std::vector<double>>> keys(2), values(2);
  for (int r = 0; r < t; ++r) {
    positions.push_back(rows[r].second);
    slots.push_back(paged.slot(rows[r].first, rows[r].second));
    row_seq.push_back(rows[r].first);
    const double* row = nullptr;
    const std::vector<double> wide = widen(std::vector<float>(qkv.begin() + static_cast<size_t>(r) * width, qkv.begin() + static_cast<size_t>(r + 1) * width));
    row = wide.data();
    q[r].assign(row, row + nh * d);
    keys[rows[r].first].push_back(std::vector<double>(row + nh * d, row + (nh + nkv) * d));
    values[rows[r].first].push_back(std::vector<double>(row + (nh + nkv) * d, row + width));
  }
  const size_t cache = static_cast<size_t>(paged.num_pages) * nkv * page * d;
  bool ok = true;
  for (int window : {0, 5}) {
    Dev<float> dq(qkv), kc(cache), vc(cache), out(static_cast<size_t>(t) * nh * d);
    Dev<int32_t> dpos(positions), dslots(slots), dseq(row_seq), dtable(paged.table);
    RUN(bc4g_rope_kv_write(dq.p, 0, dpos.p, dslots.p, kc.p, vc.p, t, nh, nkv, d, d, theta, page, paged.num_pages, 1, 0, kStream));
    RUN(bc4g_attention_generic(dq.p, width, out.p, 0, kc.p, vc.p, dtable.p, paged.pages_per_seq, dseq.p, dpos.p, t, nh, nkv, d,
                               page, paged.num_pages, window, 1.0f / std::sqrt(static_cast<float>(d)), kStream));
    ok &= close(window ? "a window of five keys" : "all keys", widen(out.get()),
                twin_attention(rows, q, keys, values, nh, nkv, d, theta, window, false), 1e-4, 1e-5);
  }
  return ok;
}

bool attention_mfma() {
  // bfloat16, the cache in the matrix-core kernel's order (its writers put it there): a step of prompt portions on
  // top of what earlier steps cached, then a step of one decoded token a request
  Rng rng(9);
  const int nh = 8, nkv = 2, d = 64, page = 16, width = (nh + 2 * nkv) * d;
  const float theta = 10000.0f;
  const std::vector<int> cached = {37, 0}, fresh = {9, 21};
  Paged paged(2, page, 37 + 9 + 1, rng);
  const size_t cache = static_cast<size_t>(paged.num_pages) * nkv * page * d;
  Dev<bf16> kc(cache), vc(cache);
  Dev<int32_t> dtable(paged.table);
  std::vector<std::vector<std::vector<double>>> keys(2), values(2);
  bool ok = true;
  // rows of a step: (request, position); the kernel is given the step as the engine describes it
  auto step = [&](const std::vector<std::pair<int, int>>& rows, const std::vector<int32_t>& seq_start,
                  const std::vector<int32_t>& seq_ctx, int form, bool attend, const char* what) -> bool {
    const int t = static_cast<int>(rows.size());
    const std::vector<bf16> qkv = as_bf16(normals(rng, static_cast<size_t>(t) * width));
    std::vector<int32_t> positions, slots, row_seq;
    std::vector<std::vector<double>> q(t);
    for (int r = 0; r < t; ++r) {
      positions.push_back(rows[r].second);
      slots.push_back(paged.slot(rows[r].first, rows[r].second));
      row_seq.push_back(rows[r].first);
      const std::vector<double> wide = widen(std::vector<bf16>(qkv.begin() + static_cast<size_t>(r) * width, qkv.begin() + static_cast<size_t>(r + 1) * width));
      q[r].assign(wide.begin(), wide.begin() + nh * d);
      keys[rows[r].first].push_back(std::vector<double>(wide.begin() + nh * d, wide.begin() + (nh + nkv) * d));
      values[rows[r].first].push_back(std::vector<double>(wide.begin() + (nh + nkv) * d, wide.end()));
    }
    Dev<bf16> dq(qkv), out(static_cast<size_t>(t) * nh * d);
    Dev<int32_t> dpos(positions), dslots(slots), dseq(row_seq), dstart(seq_start), dctx(seq_ctx);
    RUN(bc4g_rope_kv_write(dq.p, 1, dpos.p, dslots.p, kc.p, vc.p, t, nh, nkv, d, d, theta, page, paged.num_pages, 1, 0, kStream));
    if (!attend) return true;
    const int tokens_per_tile = 16 / (nh / nkv);        // a 16-row tile: these tokens times the query heads of a key/value head
    std::vector<int32_t> tile_start = {0};
    for (size_t s = 0; s + 1 < seq_start.size(); ++s)
      tile_start.push_back(tile_start.back() + (seq_start[s + 1] - seq_start[s] + tokens_per_tile - 1) / tokens_per_tile);
    Dev<int32_t> dtiles(tile_start);
    RUN(bc4g_attention_mfma(dq.p, width, out.p, nullptr, nullptr, kc.p, vc.p, dtable.p, paged.pages_per_seq, dstart.p, dctx.p,
                            dtiles.p, 2, tile_start.back(), t, nh, nkv, d, page, 0, 1.0f / std::sqrt(static_cast<float>(d)),
                            tokens_per_tile, 1, form, 1, nullptr, 0, nullptr, form == 1 ? 1 : 0, dseq.p, kStream));
    return close(what, widen(out.get()), twin_attention(rows, q, keys, values, nh, nkv, d, theta, 0, true), 3e-2, 3e-2);
  };
  std::vector<std::pair<int, int>> rows;
  for (int p = 0; p < cached[0]; ++p) rows.push_back({0, p});
  ok &= step(rows, {0, cached[0], cached[0]}, {0, 0}, 0, false, "");                       // what an earlier step cached
  rows.clear();
  for (int s = 0; s < 2; ++s)
    for (int p = 0; p < fresh[s]; ++p) rows.push_back({s, cached[s] + p});
  ok &= step(rows, {0, fresh[0], fresh[0] + fresh[1]}, {cached[0], cached[1]}, 0, true, "prompt portions");
  rows = {{0, cached[0] + fresh[0]}, {1, cached[1] + fresh[1]}};
  ok &= step(rows, {0, 1, 2}, {cached[0] + fresh[0], cached[1] + fresh[1]}, 1, true, "one decoded token a request");
  return ok;
}

bool qkv_fused() {
  // The q|k|v product with rotation and cache write in its epilogue -- the tiled kernel for a step of prompt
  // portions, the weight-streaming one for a step of decoded tokens -- checked through what attention then makes of
  // the queries it left and the cache it wrote.  Every head's rows of the weight come in blocks of sixteen: eight
  // dimensions, then their rotation partners; queries, keys, values and so the outputs live in that order.
  Rng rng(11);
  const int nh = 4, nkv = 2, d = 32, page = 16, hidden = 128, n = (nh + 2 * nkv) * d;
  const float theta = 10000.0f;
  std::vector<int> order(d);                          // place j of a head holds dimension order[j]
  for (int b = 0; b < d / 16; ++b)
    for (int t = 0; t < 16; ++t) order[16 * b + t] = t < 8 ? 8 * b + t : d / 2 + 8 * b + (t - 8);
  const std::vector<bf16> w = as_bf16(normals(rng, static_cast<size_t>(n) * hidden, 0.2f));     // rows: q heads, k heads, v heads
  std::vector<bf16> reordered(w.size());
  for (int head = 0; head < nh + 2 * nkv; ++head)
    for (int j = 0; j < d; ++j)
      std::copy(w.begin() + (static_cast<size_t>(head) * d + order[j]) * hidden, w.begin() + (static_cast<size_t>(head) * d + order[j] + 1) * hidden,
                reordered.begin() + (static_cast<size_t>(head) * d + j) * hidden);
  Dev<bf16> packed(pack_weight(reordered, n, hidden));
  const std::vector<int> fresh = {40, 23};
  Paged paged(2, page, 41, rng);
  const size_t cache = static_cast<size_t>(paged.num_pages) * nkv * page * d;
  Dev<bf16> kc(cache), vc(cache);
  Dev<int32_t> dtable(paged.table);
  std::vector<std::vector<std::vector<double>>> keys(2), values(2);
  auto step = [&](const std::vector<std::pair<int, int>>& rows, const std::vector<int32_t>& seq_start,
                  const std::vector<int32_t>& seq_ctx, bool tiled, const char* what) -> bool {
    const int t = static_cast<int>(rows.size());
    const std::vector<bf16> x = as_bf16(normals(rng, static_cast<size_t>(t) * hidden));
    const std::vector<double> product = plain::gemm(widen(x), widen(w), t, n, hidden);
    std::vector<int32_t> positions, slots, row_seq;
    std::vector<std::vector<double>> q(t);
    for (int r = 0; r < t; ++r) {
      positions.push_back(rows[r].second);
      slots.push_back(paged.slot(rows[r].first, rows[r].second));
      row_seq.push_back(rows[r].first);
      const double* row = &product[static_cast<size_t>(r) * n];
      q[r].assign(row, row + nh * d);
      keys[rows[r].first].push_back(std::vector<double>(row + nh * d, row + (nh + nkv) * d));
      std::vector<double> v(row + (nh + nkv) * d, row + n);
      for (double& e : v) e = from_bf16(to_bf16(static_cast<float>(e)));           // as the cache holds it
      values[rows[r].first].push_back(v);
    }
    Dev<bf16> dx(x), dq(static_cast<size_t>(t) * nh * d), out(static_cast<size_t>(t) * nh * d);
    Dev<int32_t> dpos(positions), dslots(slots), dseq(row_seq), dstart(seq_start), dctx(seq_ctx);
    if (tiled) {
      Dev<float> table(static_cast<size_t>(t) * d);                                 // [t][d / 2][2]: cosine and sine
      RUN(bc4g_rope_table(dpos.p, table.p, t, d, theta, kStream));
      RUN(bc4g_gemm_mfma_qkv(dx.p, packed.p, 1, dq.p, table.p, dslots.p, kc.p, vc.p, t, n, hidden, nh, nkv, d, page, 1, kStream));
    } else {
      RUN(bc4g_gemm_skinny_qkv(dx.p, nullptr, 0, 0.0f, nullptr, 0, 0, packed.p, dq.p, dpos.p, dslots.p, kc.p, vc.p, t, hidden,
                               nh, nkv, d, d, theta, page, 1, kStream));
    }
    const int tokens_per_tile = 16 / (nh / nkv);
    std::vector<int32_t> tile_start = {0};
    for (size_t s = 0; s + 1 < seq_start.size(); ++s)
      tile_start.push_back(tile_start.back() + (seq_start[s + 1] - seq_start[s] + tokens_per_tile - 1) / tokens_per_tile);
    Dev<int32_t> dtiles(tile_start);
    RUN(bc4g_attention_mfma(dq.p, nh * d, out.p, nullptr, nullptr, kc.p, vc.p, dtable.p, paged.pages_per_seq, dstart.p, dctx.p,
                            dtiles.p, 2, tile_start.back(), t, nh, nkv, d, page, 0, 1.0f / std::sqrt(static_cast<float>(d)),
                            tokens_per_tile, 1, tiled ? 0 : 1, 1, nullptr, 0, nullptr, tiled ? 0 : 1, dseq.p, kStream));
    const std::vector<double> straight = twin_attention(rows, q, keys, values, nh, nkv, d, theta, 0, true);
    std::vector<double> want(straight.size());
    for (size_t head = 0; head < straight.size() / d; ++head)
      for (int j = 0; j < d; ++j) want[head * d + j] = straight[head * d + order[j]];
    return close(what, widen(out.get()), want, 3e-2, 3e-2);
  };
  bool ok = true;
  std::vector<std::pair<int, int>> rows;
  for (int s = 0; s < 2; ++s)
    for (int p = 0; p < fresh[s]; ++p) rows.push_back({s, p});
  ok &= step(rows, {0, fresh[0], fresh[0] + fresh[1]}, {0, 0}, true, "prompt portions through the tiled product");
  rows = {{0, fresh[0]}, {1, fresh[1]}};
  ok &= step(rows, {0, 1, 2}, {fresh[0], fresh[1]}, false, "decoded tokens through the weight-streaming product");
  return ok;
}

bool argmax() {
  const int n = 3, vocab = 1000;
  std::vector<float> logits(static_cast<size_t>(n) * vocab, -1.0f);
  logits[7] = logits[500] = logits[999] = 5.0f;          // equal maxima: the lowest index
  logits[vocab + 999] = 2.0f;                             // the maximum in the last place
  for (int i = 0; i < vocab; ++i) logits[2 * vocab + i] = static_cast<float>(i % 613);
  Dev<float> dl(logits), part_v(static_cast<size_t>(n) * 64);
  Dev<int32_t> out(n), part_i(static_cast<size_t>(n) * 64);
  RUN(bc4g_argmax(dl.p, out.p, part_v.p, part_i.p, n, vocab, kStream));
  const std::vector<int32_t> got = out.get();
  bool ok = true;
  for (int r = 0; r < n; ++r) {
    const int want = plain::argmax(std::vector<float>(logits.begin() + static_cast<size_t>(r) * vocab, logits.begin() + static_cast<size_t>(r + 1) * vocab));
    if (got[r] != want) {
      std::printf("  row %d: %d, the twin says %d\n", r, got[r], want);
      ok = false;
    }
  }
  return ok;
}

bool sampling() {
  // the draw without limits (in the order of the ids) and with them (in the order of the weights), both against the
  // twin's walk; logits in steps of a quarter so that many tokens share a weight and the order of the ids decides
  Rng rng(10);
  const int n = 12, vocab = 1003;
  std::vector<float> logits(static_cast<size_t>(n) * vocab);
  for (float& v : logits) v = std::round(rng.normal(2.0f) * 4.0f) / 4.0f;
  std::vector<float> temps(n);
  std::vector<double> us(n), ps(n);
  std::vector<int32_t> ks(n), all_rows(n);
  for (int r = 0; r < n; ++r) {
    temps[r] = r % 4 == 3 ? 0.0f : 0.6f + 0.2f * static_cast<float>(r % 3);
    us[r] = r == 0 ? 0.0 : r == 1 ? 1.0 - 1.0 / 9007199254740992.0 : rng.uniform();
    ks[r] = (r % 3 == 0) ? 0 : (r % 3 == 1 ? 5 : 40);
    ps[r] = (r % 2 == 0) ? 0.9 : (ks[r] ? 1.0 : 0.5);
    all_rows[r] = r;
  }
  Dev<float> dl(logits), dt(temps);
  Dev<double> du(us), dp(ps);
  Dev<int32_t> dk(ks), out(n);
  bool ok = true;
  RUN(bc4g_sample(dl.p, dt.p, du.p, out.p, n, vocab, kStream));
  std::vector<int32_t> got = out.get();
  for (int r = 0; r < n; ++r) {
    const std::vector<float> row(logits.begin() + static_cast<size_t>(r) * vocab, logits.begin() + static_cast<size_t>(r + 1) * vocab);
    const int want = temps[r] > 0.0f ? plain::sample(row, temps[r], 0, 1.0, us[r]) : plain::argmax(row);
    if (got[r] != want) {
      std::printf("  without limits, row %d: %d, the twin says %d\n", r, got[r], want);
      ok = false;
    }
  }
  // with limits: only the rows that have a temperature, into their places of the output
  std::vector<int32_t> rows;
  std::vector<float> t2;
  std::vector<double> u2, p2;
  std::vector<int32_t> k2;
  for (int r = 0; r < n; ++r)
    if (temps[r] > 0.0f) rows.push_back(r), t2.push_back(temps[r]), u2.push_back(us[r]), p2.push_back(ps[r]), k2.push_back(ks[r]);
  Dev<int32_t> drows(rows), dk2(k2), out2(std::vector<int32_t>(n, -7));
  Dev<float> dt2(t2);
  Dev<double> du2(u2), dp2(p2);
  RUN(bc4g_sample_filtered(dl.p, drows.p, dt2.p, du2.p, dk2.p, dp2.p, out2.p, static_cast<int>(rows.size()), vocab, kStream));
  got = out2.get();
  for (size_t i = 0; i < rows.size(); ++i) {
    const int r = rows[i];
    const std::vector<float> row(logits.begin() + static_cast<size_t>(r) * vocab, logits.begin() + static_cast<size_t>(r + 1) * vocab);
    const int want = plain::sample(row, t2[i], k2[i], p2[i], u2[i]);
    if (got[r] != want) {
      std::printf("  top-k %d top-p %g, row %d: %d, the twin says %d\n", k2[i], p2[i], r, got[r], want);
      ok = false;
    }
  }
  for (int r = 0; r < n; ++r)
    if (!(temps[r] > 0.0f) && got[r] != -7) {
      std::printf("  row %d was not the kernel's to write\n", r);
      ok = false;
    }
  return ok;
}

const std::vector<std::pair<std::string, std::function<bool()>>>& tests() {
  static const std::vector<std::pair<std::string, std::function<bool()>>> all = {
      {"embed", embed},
      {"rmsnorm", rmsnorm},
      {"swiglu", swiglu},
      {"gemm_generic", gemm_generic},
      {"gemm_skinny", gemm_skinny},
      {"gemm_skinny_norms", gemm_skinny_norms},
      {"gemm_mfma", gemm_mfma},
      {"attention_generic", attention_generic},
      {"attention_mfma", attention_mfma},
      {"qkv_fused", qkv_fused},
      {"argmax", argmax},
      {"sampling", sampling},
  };
  return all;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc == 2 && std::strcmp(argv[1], "--list") == 0) {
    for (const auto& t : tests()) std::printf("%s\n", t.first.c_str());
    return 0;
  }
  int device_count = 0;
  if (hipGetDeviceCount(&device_count) != hipSuccess || device_count == 0) {
    std::printf("no GPU is visible: the kernels have no other implementation to run\n");
    return 2;
  }
  int failed = 0, ran = 0;
  for (const auto& t : tests()) {
    bool wanted = argc < 2;
    for (int i = 1; i < argc; ++i) wanted |= t.first == argv[i];
    if (!wanted) continue;
    ++ran;
    std::printf("%s ...\n", t.first.c_str());
    std::fflush(stdout);
    const bool ok = t.second();
    HIP_OK(hipDeviceSynchronize());
    std::printf("%s: %s\n", ok ? "PASS" : "FAIL", t.first.c_str());
    std::fflush(stdout);
    failed += ok ? 0 : 1;
  }
  if (ran == 0) {
    std::printf("no test of that name; --list names them\n");
    return 2;
  }
  return failed ? 1 : 0;
}
