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

// Four independent chains of 32x32x16 bfloat16 MFMAs per wave, nothing else in the loop.
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* sink) {
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = static_cast<__bf16>(threadIdx.x * 0.001f + i);
    b[i] = static_cast<__bf16>(i * 0.5f);
  }
  floatx16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int it = 0; it < iters; ++it) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
  }
  sink[blockIdx.x * 256 + threadIdx.x] = c0[0] + c1[1] + c2[2] + c3[3];
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_probe_read(const void* p, long bytes, float* sink, int workgroups, void* stream) {
  BC4G_REQUIRE(p && sink && bytes >= 16 && workgroups > 0, "probe_read: a buffer of at least 16 bytes, a sink and a grid are needed");
  probe_read_kernel<<<workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const uint4*>(p), bytes / 16, sink);
  return check_launch("probe_read");
}

// sink: float [workgroups * 256].  Operations of one launch: workgroups * 4 waves * iters * 4 * 2 * 32 * 32 * 16.
extern "C" int bc4g_probe_mfma(int iters, float* sink, int workgroups, void* stream) {
  BC4G_REQUIRE(sink && iters > 0 && workgroups > 0, "probe_mfma: a sink, a count and a grid are needed");
  probe_mfma_kernel<<<workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(iters, sink);
  return check_launch("probe_mfma");
}
