// Host stand-in for <hip/hip_runtime.h>: just enough of the HIP vocabulary to compile this library's elementwise
// kernels as ordinary C++ and run them on the CPU, one fiber per lane, in lockstep at every wavefront shuffle and
// block barrier (tests/hostsim/hostsim.cpp). Test infrastructure only; nothing in the product includes it.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <functional>

#include "hip_fp16.h"

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
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };

namespace hostsim {
struct Index { unsigned x, y, z; };
// block-by-block, lane-by-lane execution of `body` (the kernel call with its arguments bound)
void launch(dim3 grid, dim3 block, size_t dynamic_lds_bytes, const std::function<void()>& body);
// Wavefront-wide operation: every lane of the wavefront calls this with the same resolver; once all have arrived the
// resolver runs once over the lanes' payloads (payloads[l] belongs to lane l), then every lane continues.
typedef void (*Resolver)(void** payloads, int lanes);
void wave_collective(Resolver resolver, void* payload);
[[noreturn]] void fail(const char* what);
unsigned lane_id();
uint64_t shfl_xor_bits(uint64_t bits, int mask);
uint64_t gather_bits(uint64_t bits, int source_lane);   // every lane names the lane whose value it reads
void sync_block();
// direct global -> LDS transfers (asynchronous; see hostsim.cpp for the two timing models)
void dma_issue(const void* src, uint32_t lds_offset, int bytes);
void dma_wait(int may_stay_outstanding);
uint32_t lds_offset_of(uint32_t low_address_bits);   // LDS byte offset from the low 32 bits of a pointer into LDS
int compute_units();     // HOSTSIM_CUS (default 4): small, so that grid-stride loops take several trips
extern unsigned char* dynamic_lds;   // at least dynamic_lds_bytes of the current launch
}  // namespace hostsim

extern hostsim::Index threadIdx, blockIdx;
extern dim3 blockDim, gridDim;

// cycle counters (tuning aids of the kernels): no clock on the host
static inline long long clock64() { return 0; }
static inline long long wall_clock64() { return 0; }
static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "host simulation"; }
static inline hipError_t hipGetDevice(int* dev) { *dev = 0; return hipSuccess; }
static inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = hostsim::compute_units(); return hipSuccess; }

#define HIP_SYMBOL(x) x
template <typename T>
static inline hipError_t hipGetSymbolAddress(void** p, const T& symbol) { *p = const_cast<void*>(static_cast<const void*>(&symbol)); return hipSuccess; }
static inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }

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

// DPP lane exchange (all rows and banks enabled): the controls the kernels use
static inline int __builtin_amdgcn_update_dpp(int, int src, int ctrl, int, int, bool) {
  const int lane = static_cast<int>(hostsim::lane_id());
  int from;
  if (ctrl < 0x100) from = (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);   // quad_perm
  else if (ctrl == 0x141) from = (lane & ~7) | (7 - (lane & 7));              // row_half_mirror
  else if (ctrl == 0x140) from = (lane & ~15) | (15 - (lane & 15));           // row_mirror
  else hostsim::fail("DPP control not modelled");
  return static_cast<int>(hostsim::gather_bits(static_cast<uint32_t>(src), from));
}
static inline int __builtin_amdgcn_readlane(int v, int lane) { return static_cast<int>(hostsim::gather_bits(static_cast<uint32_t>(v), lane)); }

// v_permlane32_swap_b32: lanes 32..63 of the first operand change places with lanes 0..31 of the second; returns both
typedef unsigned int hostsim_u32x2 __attribute__((ext_vector_type(2)));
static inline hostsim_u32x2 __builtin_amdgcn_permlane32_swap(unsigned int vdst, unsigned int vsrc, bool, bool) {
  const int lane = static_cast<int>(hostsim::lane_id());
  const unsigned int other_dst = static_cast<unsigned int>(hostsim::gather_bits(vdst, lane ^ 32));
  const unsigned int other_src = static_cast<unsigned int>(hostsim::gather_bits(vsrc, lane ^ 32));
  return lane < 32 ? hostsim_u32x2{vdst, other_dst} : hostsim_u32x2{other_src, vsrc};
}

// v_dot2c_f32_f16 / v_dot2c_f32_bf16: acc + a[0] b[0] + a[1] b[1] in fp32
typedef _Float16 hostsim_half2 __attribute__((ext_vector_type(2)));
typedef __bf16 hostsim_bf16x2 __attribute__((ext_vector_type(2)));
static inline float __builtin_amdgcn_fdot2(hostsim_half2 a, hostsim_half2 b, float acc, bool) {
  return acc + static_cast<float>(a[0]) * static_cast<float>(b[0]) + static_cast<float>(a[1]) * static_cast<float>(b[1]);
}
static inline float __builtin_amdgcn_fdot2_f32_bf16(hostsim_bf16x2 a, hostsim_bf16x2 b, float acc, bool) {
  return acc + static_cast<float>(a[0]) * static_cast<float>(b[0]) + static_cast<float>(a[1]) * static_cast<float>(b[1]);
}

// Wavefront barrier: every lane arrives before any continues (the lanes run as fibers, so this is what makes one
// lane's earlier LDS writes visible to the others); the fences around it only constrain the device compiler.
static inline void hostsim_no_resolver(void**, int) {}
static inline void __builtin_amdgcn_wave_barrier() { hostsim::wave_collective(hostsim_no_resolver, nullptr); }
#define __builtin_amdgcn_fence(order, scope) ((void)0)

// a wavefront-uniform 64-bit mask as a per-lane predicate (the operand form of v_cndmask)
static inline bool __builtin_amdgcn_inverse_ballot_w64(uint64_t mask) { return ((mask >> hostsim::lane_id()) & 1u) != 0; }

// v_cmp into a wavefront-wide mask: bit l is lane l's predicate
static inline uint64_t __builtin_amdgcn_ballot_w64(bool pred) {
  uint64_t mask = 0;
  for (int l = 0; l < 64; ++l) mask |= (hostsim::gather_bits(pred ? 1 : 0, l) & 1u) << l;
  return mask;
}

static inline uint32_t __umulhi(uint32_t a, uint32_t b) { return static_cast<uint32_t>((static_cast<uint64_t>(a) * b) >> 32); }
static inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
static inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
static inline float rsqrtf(float v) { return 1.0f / std::sqrt(v); }
static inline float __builtin_amdgcn_exp2f(float v) { return std::exp2(v); }
static inline float __builtin_amdgcn_rcpf(float v) { return 1.0f / v; }
static inline void __builtin_amdgcn_sched_barrier(int) {}
static inline void __builtin_amdgcn_sched_group_barrier(int, int, int) {}
static inline float __builtin_amdgcn_fmed3f(float a, float b, float c) { return std::fmax(std::fmin(a, b), std::fmin(std::fmax(a, b), c)); }
static inline float __builtin_amdgcn_fractf(float v) { return v - std::floor(v); }

// ---------------------------------------------------------------------------------------------------------------
// gfx950 instructions the GEMM kernels use, by their compiler-builtin names (unknown to an x86 compiler, so free).
// ---------------------------------------------------------------------------------------------------------------
static inline uint32_t __builtin_amdgcn_readfirstlane(uint32_t v) { return v; }   // only used on wavefront-uniform values
static inline int __builtin_amdgcn_readfirstlane(int v) { return v; }

// v_perm_b32: byte i of the result is byte sel[i] of the eight bytes {src1 (0..3), src0 (4..7)}; 0x0c selects 0x00
static inline uint32_t __builtin_amdgcn_perm(uint32_t src0, uint32_t src1, uint32_t sel) {
  const uint64_t both = (static_cast<uint64_t>(src0) << 32) | src1;
  uint32_t out = 0;
  for (int i = 0; i < 4; ++i) {
    const uint32_t s = (sel >> (8 * i)) & 0xffu;
    uint32_t byte;
    if (s < 8) byte = static_cast<uint32_t>(both >> (8 * s)) & 0xffu;
    else if (s == 0x0c) byte = 0;
    else hostsim::fail("v_perm_b32 selector outside the forms this stand-in implements");
    out |= byte << (8 * i);
  }
  return out;
}

// s_waitcnt: only the vmcnt field matters here (bits 3:0 and 15:14 of the gfx9 encoding)
static inline void __builtin_amdgcn_s_waitcnt(int imm) { hostsim::dma_wait((imm & 15) | (((imm >> 14) & 3) << 4)); }

// global_load_lds_dwordx4 through the compiler builtin: lane l moves `bytes` from its own global address to LDS address
// (wavefront-uniform base) + l * bytes
static inline void __builtin_amdgcn_global_load_lds(const __attribute__((address_space(1))) void* src,
                                                    __attribute__((address_space(3))) void* lds_base, int bytes, int offset, int) {
  const uint32_t low = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_base)) + static_cast<uint32_t>(offset);
  hostsim::dma_issue(reinterpret_cast<const void*>(reinterpret_cast<uintptr_t>(src)), hostsim::lds_offset_of(low) + hostsim::lane_id() * bytes, bytes);
}

// ds_read_b64_tr_b16: within a group of 16 lanes, lane i receives element (i & 3) of the four 16-bit elements that
// lane 4 e + (i >> 2) addressed, for e = 0..3
typedef short hostsim_short4 __attribute__((ext_vector_type(4)));
namespace hostsim {
struct TrRead { const unsigned char* addr; short out[4]; };
void resolve_tr_read(void** payloads, int lanes);
}  // namespace hostsim
static inline hostsim_short4 __builtin_amdgcn_ds_read_tr16_b64_v4i16(__attribute__((address_space(3))) hostsim_short4* p) {
  hostsim::TrRead r;
  r.addr = reinterpret_cast<const unsigned char*>(reinterpret_cast<uintptr_t>(p));
  hostsim::wave_collective(hostsim::resolve_tr_read, &r);
  return hostsim_short4{r.out[0], r.out[1], r.out[2], r.out[3]};
}

// v_mfma_f32_32x32x16_{f16,bf16}: D[i][j] = C[i][j] + sum_k A[i][k] B[k][j], 32 x 32 x 16. Lane l holds
// A[l & 31][8 (l >> 5) + t] and B[8 (l >> 5) + t][l & 31] for t = 0..7, and D[8 (r / 4) + 4 (l >> 5) + r % 4][l & 31]
// in accumulator register r = 0..15.
typedef float hostsim_float16 __attribute__((ext_vector_type(16)));
namespace hostsim {
struct Mfma { const uint16_t* a; const uint16_t* b; float* c; };
void resolve_mfma_f16(void** payloads, int lanes);
void resolve_mfma_bf16(void** payloads, int lanes);
template <bool BF16, typename V>
static inline hostsim_float16 mfma(V a, V b, hostsim_float16 c) {
  uint16_t av[8], bv[8];
  float cv[16];
  std::memcpy(av, &a, 16);
  std::memcpy(bv, &b, 16);
  std::memcpy(cv, &c, 64);
  Mfma m{av, bv, cv};
  wave_collective(BF16 ? resolve_mfma_bf16 : resolve_mfma_f16, &m);
  hostsim_float16 d;
  std::memcpy(&d, cv, 64);
  return d;
}
}  // namespace hostsim
namespace hostsim {
struct MfmaF32 { float a, b; float* c; };
void resolve_mfma_f32(void** payloads, int lanes);
}  // namespace hostsim
static inline hostsim_float16 __builtin_amdgcn_mfma_f32_32x32x2f32(float a, float b, hostsim_float16 c, int, int, int) {
  float cv[16];
  std::memcpy(cv, &c, 64);
  hostsim::MfmaF32 m{a, b, cv};
  hostsim::wave_collective(hostsim::resolve_mfma_f32, &m);
  hostsim_float16 d;
  std::memcpy(&d, cv, 64);
  return d;
}
typedef _Float16 hostsim_half8 __attribute__((ext_vector_type(8)));
typedef __bf16 hostsim_bf16x8 __attribute__((ext_vector_type(8)));
static inline hostsim_float16 __builtin_amdgcn_mfma_f32_32x32x16_f16(hostsim_half8 a, hostsim_half8 b, hostsim_float16 c, int, int, int) {
  return hostsim::mfma<false>(a, b, c);
}
static inline hostsim_float16 __builtin_amdgcn_mfma_f32_32x32x16_bf16(hostsim_bf16x8 a, hostsim_bf16x8 b, hostsim_float16 c, int, int, int) {
  return hostsim::mfma<true>(a, b, c);
}
