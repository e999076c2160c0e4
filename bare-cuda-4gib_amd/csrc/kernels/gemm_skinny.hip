// out[m, n] = sum_k x[m, k] * w[n, k] for few rows m (a decode step: m <= 64), bfloat16 weights.
//
// The weights are read once, straight from memory into matrix-core registers: a workgroup owns
// 16 output columns n (16 rows of w) and all of k; its 8 waves split k between them, each wave
// feeding 16x16x32 MFMAs with w as the A operand (16-byte loads, rows of w are contiguous in k)
// and x as the B operand.  Loads run one batch of k-steps ahead of the MFMAs that use them.  The
// waves' partial sums meet in LDS and are added in wave order, so a result does not depend on
// the number of rows or on timing.
//
// What comes in (XMODE):
//   plain    x is bfloat16 [m, k], read from cache as the B operand
//   normed   x is the float residual stream (rows taken through `rows` if given) and RMSNorm is
//            fused (up to 16 rows): while the first weights are already on their way, the
//            workgroup writes bf16(x * g) into LDS and sums x^2 per row; the MFMAs read their B
//            operand from LDS, and the row's rsqrt(mean(x^2) + eps) -- a factor common to the
//            whole row -- multiplies the finished sum.
// What goes out (EPI): bfloat16 or float stored, float added into the residual stream, or, when
// w holds gate rows followed by up rows, SwiGLU of the pair of sums.
#include <math.h>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
constexpr int kRedPad = 17;
constexpr int kStagePad = 8;     // bf16 elements appended to each staged row of x

enum Epilogue : int { kStoreBf16 = 0, kStoreF32 = 1, kAccumF32 = 2, kSwigluBf16 = 3 };
enum XMode : int { kPlain = 0, kNormedG16 = 1, kNormedG32 = 2 };   // norm scale g in bfloat16 / float

struct SkinnyArgs {
  const void* x;            // bf16 [m, k], or float [*, k] in the normed modes
  const int32_t* rows;      // normed modes: row m of the product reads x[rows[m]] (null: x[m])
  const void* g;            // normed modes: RMSNorm scale [k]
  const bf16_t* w;          // [n, k]
  void* out;
  int m, n, k, n_out;
  int m_stage;              // normed modes: rows of x staged in LDS (m rounded up to 4)
  float eps;
};

__device__ inline uint32_t pack2(float a, float b) {
  return static_cast<uint32_t>(bf16_bits_from_float(a)) | (static_cast<uint32_t>(bf16_bits_from_float(b)) << 16);
}

template <int MT, int EPI, int XMODE, int U>
__global__ __launch_bounds__(kThreads) void gemm_skinny_kernel(const SkinnyArgs a) {
  constexpr int kSets = (EPI == kSwigluBf16) ? 2 : 1;   // gate and up rows
  constexpr bool kNormed = XMODE != kPlain;
  static_assert(!kNormed || MT == 1, "the fused norm handles one tile of rows");
  __shared__ float red[kWaves][kSets][MT][16][kRedPad];
  __shared__ float ssq_row[16];
  extern __shared__ __align__(16) unsigned char stage_raw[];   // normed: bf16 [m_stage][k + kStagePad]
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int col = lane % 16, grp = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int k = a.k, m = a.m;

  const int chunk = ((k + kWaves * 32 - 1) / (kWaves * 32)) * 32;
  const int k_begin = wave * chunk;
  const int k_end = min(k, k_begin + chunk);

  floatx4 acc[kSets][MT];
#pragma unroll
  for (int s = 0; s < kSets; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[s][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int wrow = n0 + col;                           // this lane's row of w (output column)
  const bool wrow_ok = wrow < a.n_out;
  const bf16_t* wptr[kSets];
#pragma unroll
  for (int s = 0; s < kSets; ++s) wptr[s] = a.w + (static_cast<long>(wrow) + static_cast<long>(s) * a.n_out) * k;

  // where this lane's B operand comes from
  const bf16_t* xptr[MT];
  bool xrow_ok[MT];
  const int stage_stride = k + kStagePad;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = t * 16 + col;
    xrow_ok[t] = row < m;
    if constexpr (kNormed) {
      xptr[t] = reinterpret_cast<const bf16_t*>(stage_raw) + static_cast<long>(min(row, a.m_stage - 1)) * stage_stride;
    } else {
      xptr[t] = static_cast<const bf16_t*>(a.x) + static_cast<long>(row) * k;
    }
  }

  struct Batch {
    uint4 w[kSets][U];
    uint4 x[kNormed ? 1 : MT][kNormed ? 1 : U];
  };
  auto load = [&](Batch& b, int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + 32 * u + 8 * grp;
      const bool ok = kk < k_end;
#pragma unroll
      for (int s = 0; s < kSets; ++s) b.w[s][u] = (ok && wrow_ok) ? load16(wptr[s] + kk) : zero16();
      if constexpr (!kNormed) {
#pragma unroll
        for (int t = 0; t < MT; ++t) b.x[t][u] = (ok && xrow_ok[t]) ? load16(xptr[t] + kk) : zero16();
      }
    }
  };
  auto compute = [&](const Batch& b, int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        uint4 xb;
        if constexpr (kNormed) {
          const int kk = k0 + 32 * u + 8 * grp;
          xb = kk < k_end ? *reinterpret_cast<const uint4*>(xptr[t] + kk) : zero16();
        } else {
          xb = b.x[t][u];
        }
#pragma unroll
        for (int s = 0; s < kSets; ++s) acc[s][t] = mfma_16x16x32(b.w[s][u], xb, acc[s][t]);
      }
    }
  };

  constexpr int kStep = 32 * U;
  Batch cur, nxt;
  if (k_begin < k_end) load(cur, k_begin);   // the first weights are on their way

  if constexpr (kNormed) {
    // stage bf16(x * g) for every row: 32 threads walk one row, 8 elements each per pass
    bf16_t* stage = reinterpret_cast<bf16_t*>(stage_raw);
    const int srow0 = threadIdx.x / 32, sl = threadIdx.x % 32;
    for (int row = srow0; row < a.m_stage; row += kThreads / 32) {
      float ss = 0.f;
      if (row < m) {
        const long src = a.rows ? a.rows[row] : row;
        const float* xr = static_cast<const float*>(a.x) + src * k;
        for (int kk = sl * 8; kk < k; kk += 256) {
          const uint4 x0 = load16(xr + kk), x1 = load16(xr + kk + 4);
          float xv[8] = {__uint_as_float(x0.x), __uint_as_float(x0.y), __uint_as_float(x0.z), __uint_as_float(x0.w),
                         __uint_as_float(x1.x), __uint_as_float(x1.y), __uint_as_float(x1.z), __uint_as_float(x1.w)};
          float gv[8];
          if constexpr (XMODE == kNormedG16) {
            const uint4 g0 = load16(static_cast<const bf16_t*>(a.g) + kk);
            const uint32_t gr[4] = {g0.x, g0.y, g0.z, g0.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              gv[2 * i] = __uint_as_float(gr[i] << 16);
              gv[2 * i + 1] = __uint_as_float(gr[i] & 0xffff0000u);
            }
          } else {
            const uint4 g0 = load16(static_cast<const float*>(a.g) + kk), g1 = load16(static_cast<const float*>(a.g) + kk + 4);
            const uint32_t gr[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) gv[i] = __uint_as_float(gr[i]);
          }
#pragma unroll
          for (int i = 0; i < 8; ++i) ss += xv[i] * xv[i];
          *reinterpret_cast<uint4*>(stage + static_cast<long>(row) * stage_stride + kk) =
              make_uint4(pack2(xv[0] * gv[0], xv[1] * gv[1]), pack2(xv[2] * gv[2], xv[3] * gv[3]),
                         pack2(xv[4] * gv[4], xv[5] * gv[5]), pack2(xv[6] * gv[6], xv[7] * gv[7]));
        }
      } else {
        for (int kk = sl * 8; kk < k; kk += 256)
          *reinterpret_cast<uint4*>(stage + static_cast<long>(row) * stage_stride + kk) = zero16();
      }
#pragma unroll
      for (int off = 16; off > 0; off >>= 1) ss += __shfl_xor(ss, off, kWave);   // the row's 32 threads
      if (sl == 0 && row < 16) ssq_row[row] = ss;
    }
    __syncthreads();
  }

  for (int k0 = k_begin; k0 < k_end; k0 += kStep) {
    const bool more = k0 + kStep < k_end;
    if (more) load(nxt, k0 + kStep);
    compute(cur, k0);
    if (more) cur = nxt;
  }

  // acc[s][t][r] is the partial sum for output column n0 + 4*grp + r and row t*16 + col
#pragma unroll
  for (int s = 0; s < kSets; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][s][t][4 * grp + r][col] = acc[s][t][r];
  __syncthreads();

  for (int idx = threadIdx.x; idx < MT * 256; idx += kThreads) {
    const int nl = idx % 16, row = idx / 16;
    const int gn = n0 + nl;
    if (row >= m || gn >= a.n_out) continue;
    float sum[kSets];
#pragma unroll
    for (int s = 0; s < kSets; ++s) {
      float v = 0.f;
#pragma unroll
      for (int wv = 0; wv < kWaves; ++wv) v += red[wv][s][row / 16][nl][row % 16];
      sum[s] = v;
    }
    if constexpr (kNormed) {
      const float scale = 1.0f / sqrtf(ssq_row[row] / static_cast<float>(k) + a.eps);
#pragma unroll
      for (int s = 0; s < kSets; ++s) sum[s] *= scale;
    }
    const long o = static_cast<long>(row) * a.n_out + gn;
    if constexpr (EPI == kStoreBf16) {
      static_cast<bf16_t*>(a.out)[o] = from_float<bf16_t>(sum[0]);
    } else if constexpr (EPI == kStoreF32) {
      static_cast<float*>(a.out)[o] = sum[0];
    } else if constexpr (EPI == kAccumF32) {
      static_cast<float*>(a.out)[o] += sum[0];
    } else {
      const float gt = sum[0], up = sum[kSets - 1];
      static_cast<bf16_t*>(a.out)[o] = from_float<bf16_t>((gt / (1.0f + expf(-gt))) * up);
    }
  }
}

constexpr int kMaxStageBytes = 96 * 1024;

template <int EPI, int XMODE>
int launch(const SkinnyArgs& a, hipStream_t s) {
  const int mt = (a.m + 15) / 16;
  dim3 grid((a.n_out + 15) / 16), block(kThreads);
  if constexpr (XMODE != kPlain) {
    if (mt != 1) return fail("gemm_skinny: the fused norm takes at most 16 rows, got %d", a.m);
    const size_t stage = static_cast<size_t>(a.m_stage) * (a.k + kStagePad) * 2;
    if (stage > kMaxStageBytes) return fail("gemm_skinny: %d rows of k=%d do not fit the staging buffer", a.m, a.k);
    auto kernel = gemm_skinny_kernel<1, EPI, XMODE, (EPI == kSwigluBf16 ? 4 : 8)>;
    static bool raised = false;   // per instantiation: allow more than the default dynamic LDS
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kMaxStageBytes) != hipSuccess)
        return fail("gemm_skinny: cannot raise the dynamic LDS limit");
      raised = true;
    }
    kernel<<<grid, block, stage, s>>>(a);
  } else {
    switch (mt) {
      case 1: gemm_skinny_kernel<1, EPI, XMODE, 4><<<grid, block, 0, s>>>(a); break;
      case 2: gemm_skinny_kernel<2, EPI, XMODE, 4><<<grid, block, 0, s>>>(a); break;
      case 3: gemm_skinny_kernel<3, EPI, XMODE, 2><<<grid, block, 0, s>>>(a); break;
      case 4: gemm_skinny_kernel<4, EPI, XMODE, 2><<<grid, block, 0, s>>>(a); break;
      default: return fail("gemm_skinny: M=%d is beyond 64 rows", a.m);
    }
  }
  return check_launch("gemm_skinny");
}

template <int XMODE>
int launch_epilogue(SkinnyArgs& a, int epilogue, hipStream_t s) {
  a.n_out = a.n;
  switch (epilogue) {
    case kStoreBf16: return launch<kStoreBf16, XMODE>(a, s);
    case kStoreF32: return launch<kStoreF32, XMODE>(a, s);
    case kAccumF32: return launch<kAccumF32, XMODE>(a, s);
    case kSwigluBf16: a.n_out = a.n / 2; return launch<kSwigluBf16, XMODE>(a, s);
    default: return fail("gemm_skinny: unknown epilogue %d", epilogue);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_gemm_skinny(const void* x, const void* w, void* out, int epilogue, int m, int n, int k,
                                void* stream) {
  BC4G_REQUIRE(m >= 0 && m <= 64, "gemm_skinny: M=%d must be at most 64", m);
  BC4G_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny: K=%d must be a positive multiple of 8 (N=%d)", k, n);
  BC4G_REQUIRE(epilogue != kSwigluBf16 || n % 2 == 0, "gemm_skinny: SwiGLU needs gate and up rows, N=%d is odd", n);
  if (m == 0) return 0;
  SkinnyArgs a{x, nullptr, nullptr, static_cast<const bf16_t*>(w), out, m, n, k, n, 0, 0.f};
  return launch_epilogue<kPlain>(a, epilogue, static_cast<hipStream_t>(stream));
}

extern "C" int bc4g_gemm_skinny_normed_max_k(int m) {
  const int m_stage = ((m + 3) / 4) * 4;
  return m_stage > 0 ? kMaxStageBytes / (2 * m_stage) - kStagePad : 0;
}

extern "C" int bc4g_gemm_skinny_normed(const float* x, const int32_t* rows, const void* g, int g_dtype,
                                       float eps, const void* w, void* out, int epilogue, int m, int n, int k,
                                       void* stream) {
  BC4G_REQUIRE(m >= 0 && m <= 16, "gemm_skinny_normed: M=%d must be at most 16", m);
  BC4G_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny_normed: K=%d must be a positive multiple of 8 (N=%d)", k, n);
  BC4G_REQUIRE(epilogue != kSwigluBf16 || n % 2 == 0, "gemm_skinny_normed: SwiGLU needs gate and up rows, N=%d is odd", n);
  BC4G_REQUIRE(epilogue != kAccumF32, "gemm_skinny_normed: adding into the stream it reads is not supported");
  if (m == 0) return 0;
  SkinnyArgs a{x, rows, g, static_cast<const bf16_t*>(w), out, m, n, k, n, ((m + 3) / 4) * 4, eps};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (g_dtype == kBF16) return launch_epilogue<kNormedG16>(a, epilogue, s);
  if (g_dtype == kF32) return launch_epilogue<kNormedG32>(a, epilogue, s);
  return fail("gemm_skinny_normed: unknown norm scale dtype %d", g_dtype);
}
