// What the twin tests share: device buffers, a random generator, bfloat16 on the host, the packed order
// of a streamed weight, and the comparison that names the worst element.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../kernels/api.h"

#define HIP_OK(call)                                                                         \
  do {                                                                                       \
    hipError_t e_ = (call);                                                                  \
    if (e_ != hipSuccess) {                                                                  \
      std::printf("%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_));      \
      std::exit(2);                                                                          \
    }                                                                                        \
  } while (0)

// A kernel entry point that must succeed.
#define RUN(call)                                                                    \
  do {                                                                               \
    if ((call) != 0) {                                                               \
      std::printf("  %s refused: %s\n", #call, bc4g_last_error());                   \
      return false;                                                                  \
    }                                                                                \
  } while (0)

namespace twin {

typedef uint16_t bf16;

inline bf16 to_bf16(float f) {      // round to nearest, ties to even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<bf16>(u >> 16);
}
inline float from_bf16(bf16 b) {
  const uint32_t u = static_cast<uint32_t>(b) << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

struct Rng {       // splitmix64; normal() by Box-Muller
  uint64_t s;
  explicit Rng(uint64_t seed) : s(seed) {}
  uint64_t next() {
    uint64_t z = (s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
  }
  double uniform() { return static_cast<double>(next() >> 11) * (1.0 / 9007199254740992.0); }
  float normal(float scale = 1.0f) {
    const double a = uniform(), b = uniform();
    return scale * static_cast<float>(std::sqrt(-2.0 * std::log(a + 1e-300)) * std::cos(6.283185307179586 * b));
  }
  int below(int n) { return static_cast<int>(next() % static_cast<uint64_t>(n)); }
};

inline std::vector<float> normals(Rng& rng, size_t n, float scale = 1.0f) {
  std::vector<float> v(n);
  for (float& x : v) x = rng.normal(scale);
  return v;
}
inline std::vector<bf16> as_bf16(const std::vector<float>& v) {
  std::vector<bf16> out(v.size());
  for (size_t i = 0; i < v.size(); ++i) out[i] = to_bf16(v[i]);
  return out;
}
inline std::vector<double> widen(const std::vector<bf16>& v) {
  std::vector<double> out(v.size());
  for (size_t i = 0; i < v.size(); ++i) out[i] = from_bf16(v[i]);
  return out;
}
inline std::vector<double> widen(const std::vector<float>& v) { return std::vector<double>(v.begin(), v.end()); }

// Device memory that lives as long as the object.
template <typename T>
struct Dev {
  T* p = nullptr;
  size_t n = 0;
  explicit Dev(size_t count) : n(count) {
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&p), (n ? n : 1) * sizeof(T)));
    HIP_OK(hipMemset(p, 0, (n ? n : 1) * sizeof(T)));
  }
  explicit Dev(const std::vector<T>& host) : Dev(host.size()) { put(host); }
  Dev(const Dev&) = delete;
  Dev& operator=(const Dev&) = delete;
  ~Dev() { (void)hipFree(p); }
  void put(const std::vector<T>& host) { HIP_OK(hipMemcpy(p, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice)); }
  std::vector<T> get() const {
    HIP_OK(hipDeviceSynchronize());
    std::vector<T> host(n);
    HIP_OK(hipMemcpy(host.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
    return host;
  }
};

// A [n, k] weight in the order the weight-streaming kernel reads: [ceil(n/16)][ceil(k/32)][64 lanes][8], lane l of
// a k-step holding row l % 16 of the block and k 8 * (l / 16) .. + 7 of the step; zeros past n and k.
inline std::vector<bf16> pack_weight(const std::vector<bf16>& w, int n, int k) {
  const int nb = (n + 15) / 16, ks = (k + 31) / 32;
  std::vector<bf16> out(static_cast<size_t>(nb) * ks * 64 * 8, 0);
  for (int b = 0; b < nb; ++b)
    for (int s = 0; s < ks; ++s)
      for (int l = 0; l < 64; ++l)
        for (int e = 0; e < 8; ++e) {
          const int row = b * 16 + l % 16, col = s * 32 + 8 * (l / 16) + e;
          if (row < n && col < k) out[((static_cast<size_t>(b) * ks + s) * 64 + l) * 8 + e] = w[static_cast<size_t>(row) * k + col];
        }
  return out;
}

// |got - want| <= atol + rtol |want| everywhere; names the worst place otherwise.
inline bool close(const char* what, const std::vector<double>& got, const std::vector<double>& want, double rtol, double atol) {
  if (got.size() != want.size()) {
    std::printf("  %s: %zu values, %zu expected\n", what, got.size(), want.size());
    return false;
  }
  double worst = 0.0;
  size_t at = 0;
  for (size_t i = 0; i < got.size(); ++i) {
    const double over = std::fabs(got[i] - want[i]) - (atol + rtol * std::fabs(want[i]));
    if (!(over <= worst) || std::isnan(got[i])) {
      if (std::isnan(got[i])) {
        std::printf("  %s: element %zu is not a number\n", what, i);
        return false;
      }
      worst = over, at = i;
    }
  }
  if (worst > 0.0) {
    std::printf("  %s: element %zu is %.9g, the twin says %.9g\n", what, at, got[at], want[at]);
    return false;
  }
  return true;
}

}  // namespace twin
