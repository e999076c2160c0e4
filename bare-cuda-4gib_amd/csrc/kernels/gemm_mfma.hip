// out[m, n] (+)= sum_k a[m, k] * w[n, k], bfloat16 operands, float accumulation on the matrix
// cores: the product of prompt portions (many rows).
//
// A workgroup of 4 waves computes a 128 x 128 tile of the output in k-steps of 64.  Both operands
// are contiguous in k, so a tile of each is staged through LDS as [128 rows][64 k] with rows padded
// to 144 bytes (which makes the 16-byte fragment reads of 8 consecutive lanes cover all banks), in
// two buffers: while the waves feed 32x32x16 MFMAs from one, the next k-step's global loads are in
// flight (two k-steps ahead, in registers) and the one after the current is written to the other.  Each wave owns a 64 x 64 quarter (2 x 2 MFMA blocks).
// Rows and columns beyond the matrix are read as zero and not stored; k must be a multiple of 8.
// Every output element is accumulated over k in ascending order, whatever the number of rows.
//
// Workgroups are numbered so that those sharing a tile of w run on the same XCD (workgroups are
// dealt to the 8 XCDs in turn, each with an L2 of its own).
#include <math.h>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kLdsStride = kBK + 8;   // elements; 144 bytes
constexpr int kXcds = 8;

// kSwigluBf16: every 16 rows of w are eight gate rows and the eight up rows of the same outputs;
// out [m, n / 2] = silu(gate) * up.  A gate and its up lie eight lanes apart in the MFMA result.
enum Epilogue : int { kStoreBf16 = 0, kStoreF32 = 1, kAccumF32 = 2, kSwigluBf16 = 3 };

struct Tile {
  bf16_t a[kBM][kLdsStride];
  bf16_t w[kBN][kLdsStride];
};

template <int EPI>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                        void* __restrict__ out, int m, int n, int k,
                                                        int m_blocks, int n_blocks) {
  __shared__ Tile tiles[2];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / 2, wn = wave % 2;   // this wave's 64 x 64 quarter

  // XCD-aware numbering: consecutive logical ids stay on one XCD; m runs fastest so that
  // neighbours share a tile of w.
  const int total = m_blocks * n_blocks;
  int logical = blockIdx.x;
  if (total % kXcds == 0) logical = (blockIdx.x % kXcds) * (total / kXcds) + blockIdx.x / kXcds;
  const int bm = logical % m_blocks, bn = logical / m_blocks;
  const long m0 = static_cast<long>(bm) * kBM, n0 = static_cast<long>(bn) * kBN;

  // global -> LDS: a tile is 128 rows x 8 segments of 16 bytes; thread t moves segment t%8 of rows t/8 + 32 i.
  // Two register sets hold the k-steps that are on their way from memory (two steps ahead of the
  // MFMAs); LDS holds the step being multiplied and the next one.
  const int seg = tid % 8, lrow = tid / 8;
  struct Staged {
    uint4 a[4], w[4];
  };
  auto load_tiles = [&](Staged& r, int kt) {
    const int kk = kt * kBK + seg * 8;
    const bool k_ok = kk < k;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const long gm = m0 + lrow + 32 * i, gn = n0 + lrow + 32 * i;
      r.a[i] = (k_ok && gm < m) ? load16(a + gm * k + kk) : zero16();
      r.w[i] = (k_ok && gn < n) ? load16(w + gn * k + kk) : zero16();
    }
  };
  auto store_tiles = [&](const Staged& r, int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<uint4*>(&tiles[buf].a[lrow + 32 * i][seg * 8]) = r.a[i];
      *reinterpret_cast<uint4*>(&tiles[buf].w[lrow + 32 * i][seg * 8]) = r.w[i];
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frow = lane % 32, fk = (lane / 32) * 8;
  auto multiply = [&](int buf) {
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      uint4 fa[2], fw[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = *reinterpret_cast<const uint4*>(&tiles[buf].a[wm * 64 + i * 32 + frow][ks * 16 + fk]);
        fw[i] = *reinterpret_cast<const uint4*>(&tiles[buf].w[wn * 64 + i * 32 + frow][ks * 16 + fk]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma_32x32x16(fa[i], fw[j], acc[i][j]);
    }
  };

  const int nk = (k + kBK - 1) / kBK;
  Staged r0, r1;
  load_tiles(r0, 0);
  if (nk > 1) load_tiles(r1, 1);
  store_tiles(r0, 0);
  if (nk > 2) load_tiles(r0, 2);
  __syncthreads();
  for (int kt = 0; kt < nk; kt += 2) {
    multiply(0);                                  // k-step kt
    if (kt + 1 < nk) store_tiles(r1, 1);
    if (kt + 3 < nk) load_tiles(r1, kt + 3);
    __syncthreads();
    if (kt + 1 < nk) multiply(1);                 // k-step kt + 1
    if (kt + 2 < nk) store_tiles(r0, 0);
    if (kt + 4 < nk) load_tiles(r0, kt + 4);
    __syncthreads();
  }

  // acc[i][j][r]: row m0 + wm*64 + i*32 + 8*(r/4) + 4*(lane/32) + r%4, column n0 + wn*64 + j*32 + lane%32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const long gn = n0 + wn * 64 + j * 32 + lane % 32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const long gm = m0 + wm * 64 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        if constexpr (EPI == kSwigluBf16) {
          const float mine = acc[i][j][r];
          const float other = __shfl_xor(mine, 8, kWave);          // every lane takes part
          if ((lane & 8) == 0 && gm < m && gn < n) {
            const long oc = (gn / 16) * 8 + gn % 8;
            static_cast<bf16_t*>(out)[gm * (n / 2) + oc] = from_float<bf16_t>((mine / (1.0f + expf(-mine))) * other);
          }
          continue;
        }
        if (gm >= m || gn >= n) continue;
        const long o = gm * n + gn;
        if constexpr (EPI == kStoreBf16) static_cast<bf16_t*>(out)[o] = from_float<bf16_t>(acc[i][j][r]);
        else if constexpr (EPI == kStoreF32) static_cast<float*>(out)[o] = acc[i][j][r];
        else static_cast<float*>(out)[o] += acc[i][j][r];
      }
    }
}

template <int EPI>
void launch_tiled(const bf16_t* ap, const bf16_t* wp, void* out, int m, int n, int k, long m_blocks, long n_blocks,
                  hipStream_t s) {
  dim3 grid(static_cast<unsigned>(m_blocks * n_blocks)), block(256);
  gemm_mfma_kernel<EPI><<<grid, block, 0, s>>>(ap, wp, out, m, n, k, m_blocks, n_blocks);
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_gemm_mfma(const void* a, const void* w, void* out, int epilogue, int m, int n, int k,
                              void* stream) {
  BC4G_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 8 == 0, "gemm_mfma: K=%d must be a positive multiple of 8 (M=%d N=%d)",
               k, m, n);
  if (m == 0) return 0;
  const long m_blocks = (m + kBM - 1) / kBM, n_blocks = (n + kBN - 1) / kBN;
  BC4G_REQUIRE(m_blocks * n_blocks <= 2147483647L, "gemm_mfma: too many tiles");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bf16_t* ap = static_cast<const bf16_t*>(a);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  switch (epilogue) {
    case kStoreBf16: launch_tiled<kStoreBf16>(ap, wp, out, m, n, k, m_blocks, n_blocks, s); break;
    case kStoreF32: launch_tiled<kStoreF32>(ap, wp, out, m, n, k, m_blocks, n_blocks, s); break;
    case kAccumF32: launch_tiled<kAccumF32>(ap, wp, out, m, n, k, m_blocks, n_blocks, s); break;
    case kSwigluBf16:
      BC4G_REQUIRE(n % 16 == 0, "gemm_mfma: SwiGLU needs blocks of eight gate and eight up rows, N=%d is no multiple of 16", n);
      launch_tiled<kSwigluBf16>(ap, wp, out, m, n, k, m_blocks, n_blocks, s);
      break;
    default: return fail("gemm_mfma: unknown epilogue %d", epilogue);
  }
  return check_launch("gemm_mfma");
}
