// Host stand-in for <hip/hip_runtime.h>: just enough of the HIP vocabulary to compile this library's elementwise
// kernels as ordinary C++ and run them on the CPU, one fiber per lane, in lockstep at every wavefront shuffle and
// block barrier (tests/hostsim/hostsim.cpp). Test infrastructure only; nothing in the product includes it.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <functional>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))

struct dim3 {
  unsigned x, y, z;
  constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct alignas(16) uint4 { uint32_t x, y, z, w; };
struct alignas(8) uint2 { uint32_t x, y; };
struct alignas(16) float4 { float x, y, z, w; };
struct alignas(8) float2 { float x, y; };
static inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{x, y, z, w}; }
static inline uint2 make_uint2(uint32_t x, uint32_t y) { return uint2{x, y}; }
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
static inline float2 make_float2(float x, float y) { return float2{x, y}; }

using std::max;
using std::min;

typedef void* hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0 };
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 1 };

namespace hostsim {
struct Index { unsigned x, y, z; };
// block-by-block, lane-by-lane execution of `body` (the kernel call with its arguments bound)
void launch(dim3 grid, dim3 block, size_t dynamic_lds_bytes, const std::function<void()>& body);
uint64_t shfl_xor_bits(uint64_t bits, int mask);
void sync_block();
int compute_units();     // HOSTSIM_CUS (default 4): small, so that grid-stride loops take several trips
extern unsigned char* dynamic_lds;   // at least dynamic_lds_bytes of the current launch
}  // namespace hostsim

extern hostsim::Index threadIdx, blockIdx;
extern dim3 blockDim, gridDim;

static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "host simulation"; }
static inline hipError_t hipGetDevice(int* dev) { *dev = 0; return hipSuccess; }
static inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = hostsim::compute_units(); return hipSuccess; }

#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
  ::hostsim::launch((grid), (block), (lds), [=]() { kernel(__VA_ARGS__); })

template <typename T>
static inline T __shfl_xor(T v, int mask, int width = 64) {
  static_assert(sizeof(T) <= 8, "shuffle of at most 64 bits");
  (void)width;
  uint64_t bits = 0;
  std::memcpy(&bits, &v, sizeof(T));
  bits = hostsim::shfl_xor_bits(bits, mask);
  T out;
  std::memcpy(&out, &bits, sizeof(T));
  return out;
}
static inline void __syncthreads() { hostsim::sync_block(); }

static inline uint32_t __umulhi(uint32_t a, uint32_t b) { return static_cast<uint32_t>((static_cast<uint64_t>(a) * b) >> 32); }
static inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
static inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
static inline float rsqrtf(float v) { return 1.0f / std::sqrt(v); }
static inline float __builtin_amdgcn_exp2f(float v) { return std::exp2(v); }
static inline float __builtin_amdgcn_rcpf(float v) { return 1.0f / v; }
static inline void __builtin_amdgcn_sched_barrier(int) {}
