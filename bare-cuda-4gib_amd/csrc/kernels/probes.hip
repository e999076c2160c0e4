// What this GPU delivers to a kernel that does nothing else: memory bandwidth for a kernel that only
// reads, and the rate of back-to-back matrix-core instructions.  The benchmark programs state their
// results against the published peaks and against these.
#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

// Every workgroup reads its share of the buffer in 16-byte pieces, sixteen loads of a thread in flight.
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ p, long pieces, float* sink) {
  const long stride = static_cast<long>(gridDim.x) * blockDim.x;
  long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 15 * stride < pieces; i += 16 * stride) {
    uint4 v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = p[i + j * stride];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  for (; i < pieces; i += stride) acc ^= p[i].x;
  if (acc == 0x12345678u) sink[0] = 1.f;      // (keeps the loads alive; never true for the data the host fills in)
}

// Eight independent chains of 32x32x16 bfloat16 MFMAs per wave (2 x 4 blocks from two and four fragments, two slices
// of k), nothing else in the loop.  The operands come from memory, 12 fragments of 256 lanes x 16 bytes: what the
// matrix cores sustain depends on them -- the chip lowers its clock with the power that toggling operands draw (zeros
// and ones run at 2.1-2.2 GHz, normally distributed values at 1.7).
__global__ __launch_bounds__(256) void probe_mfma_kernel(const uint4* operands, int iters, float* sink) {
  uint4 a[2][2], b[4][2];
  for (int i = 0; i < 2; ++i)
    for (int s = 0; s < 2; ++s) a[i][s] = operands[(i * 2 + s) * 256 + threadIdx.x];
  for (int j = 0; j < 4; ++j)
    for (int s = 0; s < 2; ++s) b[j][s] = operands[(4 + j * 2 + s) * 256 + threadIdx.x];
  floatx16 c[2][4] = {};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) c[i][j] = mfma_32x32x16(a[i][s], b[j][s], c[i][j]);
  }
  float total = 0.f;
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 4; ++j) total += c[i][j][threadIdx.x % 16];
  sink[blockIdx.x * 256 + threadIdx.x] = total;
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_probe_read(const void* p, long bytes, float* sink, int workgroups, void* stream) {
  BC4G_REQUIRE(p && sink && bytes >= 16 && workgroups > 0, "probe_read: a buffer of at least 16 bytes, a sink and a grid are needed");
  probe_read_kernel<<<workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const uint4*>(p), bytes / 16, sink);
  return check_launch("probe_read");
}

// operands: 12 * 256 * 16 bytes of bfloat16; sink: float [workgroups * 256].  Operations of one launch:
// workgroups * 4 waves * iters * 16 * 2 * 32 * 32 * 16.
extern "C" int bc4g_probe_mfma(const void* operands, int iters, float* sink, int workgroups, void* stream) {
  BC4G_REQUIRE(operands && sink && iters > 0 && workgroups > 0, "probe_mfma: operands, a sink, a count and a grid are needed");
  probe_mfma_kernel<<<workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const uint4*>(operands), iters, sink);
  return check_launch("probe_mfma");
}
