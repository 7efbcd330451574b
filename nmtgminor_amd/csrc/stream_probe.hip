// Streaming probes for gfx950: what one launch of the simplest possible kernel reaches on this HBM for the three access
// mixes the library's bandwidth-bound kernels have (one stream in and one out; two in and one out; read only). They exist
// to be timed: the figures are the practical ceiling that the roofline fractions of layer norm, dropout + add, softmax
// and the loss kernels are read against. No counterpart in the reference.
//
// Shape of every probe: 16 bytes per lane and access, four accesses of a lane in flight before the first use (as the
// library's elementwise kernels do), the grid covers the buffer exactly once.
#include "common.hip.h"

namespace nmtg {
namespace {

constexpr int SP_THREADS = 256;
constexpr int SP_UNROLL = 4;   // 16-byte accesses per lane

// mode 0: out = a;  mode 1: out = a + b (fp32 lanes);  mode 2: out[block] = sum over the block's chunk of a (read only)
template <int MODE>
__global__ __launch_bounds__(SP_THREADS) void stream_probe_kernel(const float4* __restrict__ a, const float4* __restrict__ b,
                                                                  float4* __restrict__ out, float* __restrict__ sums, int64_t n16) {
  __shared__ float part[SP_THREADS / 64];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (SP_THREADS * SP_UNROLL) + threadIdx.x;
  float4 va[SP_UNROLL], vb[SP_UNROLL];
#pragma unroll
  for (int u = 0; u < SP_UNROLL; ++u) {
    const int64_t i = base + static_cast<int64_t>(u) * SP_THREADS;
    va[u] = i < n16 ? a[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    if constexpr (MODE == 1) vb[u] = i < n16 ? b[i] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  if constexpr (MODE == 2) {
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < SP_UNROLL; ++u) s += (va[u].x + va[u].y) + (va[u].z + va[u].w);
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) sums[blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
  } else {
#pragma unroll
    for (int u = 0; u < SP_UNROLL; ++u) {
      const int64_t i = base + static_cast<int64_t>(u) * SP_THREADS;
      if constexpr (MODE == 1) va[u] = make_float4(va[u].x + vb[u].x, va[u].y + vb[u].y, va[u].z + vb[u].z, va[u].w + vb[u].w);
      if (i < n16) out[i] = va[u];
    }
  }
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int64_t nmtg_stream_probe_blocks(int64_t bytes) {
  const int64_t n16 = bytes / 16, per_block = SP_THREADS * SP_UNROLL;
  return (n16 + per_block - 1) / per_block;
}

extern "C" int nmtg_stream_probe(const void* a, const void* b, void* out, int64_t bytes, int mode, void* stream) {
  NMTG_REQUIRE(mode >= 0 && mode <= 2, "stream_probe: mode %d (0 copy, 1 add, 2 read)", mode);
  NMTG_REQUIRE(bytes >= 0 && bytes % 16 == 0, "stream_probe: %lld bytes, a multiple of 16 required", (long long)bytes);
  if (bytes == 0) return 0;
  NMTG_REQUIRE(a && out && (mode != 1 || b), "stream_probe: null pointer argument");
  NMTG_REQUIRE(aligned16(a) && aligned16(out) && (mode != 1 || aligned16(b)), "stream_probe: 16-byte aligned buffers required");
  const int64_t n16 = bytes / 16, blocks = nmtg_stream_probe_blocks(bytes);
  NMTG_REQUIRE(blocks <= 0x7fffffff, "stream_probe: %lld bytes need more than 2^31 blocks", (long long)bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  TraceScope trace("stream_probe", st);
  const dim3 grid(static_cast<unsigned>(blocks)), block(SP_THREADS);
  const float4* pa = static_cast<const float4*>(a);
  const float4* pb = static_cast<const float4*>(b);
  if (mode == 0) hipLaunchKernelGGL(stream_probe_kernel<0>, grid, block, 0, st, pa, pb, static_cast<float4*>(out), nullptr, n16);
  else if (mode == 1) hipLaunchKernelGGL(stream_probe_kernel<1>, grid, block, 0, st, pa, pb, static_cast<float4*>(out), nullptr, n16);
  else hipLaunchKernelGGL(stream_probe_kernel<2>, grid, block, 0, st, pa, pb, nullptr, static_cast<float*>(out), n16);
  NMTG_CHECK_LAUNCH("stream_probe");
  return 0;
}
