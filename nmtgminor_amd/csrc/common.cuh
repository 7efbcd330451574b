// Shared device/host helpers for the gfx950 (MI355X, CDNA4) kernels of this library.
// Everything here assumes 64-lane wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <string>
#include <cstdio>
#include <cstdarg>

#include "../../include/nmtg_hip.h"

namespace nmtg {

// ---------------------------------------------------------------------------------------------
// Error plumbing: every extern "C" entry point returns an int status and leaves a message that
// nmtg_last_error() hands back. Nothing in the library aborts the process.
// ---------------------------------------------------------------------------------------------
std::string& last_error_slot();
int fail(int code, const char* fmt, ...);

#define NMTG_REQUIRE(cond, ...)                                        \
  do {                                                                 \
    if (!(cond)) return ::nmtg::fail(NMTG_ERR_INVALID, __VA_ARGS__);   \
  } while (0)

#define NMTG_CHECK_LAUNCH(what)                                                            \
  do {                                                                                     \
    hipError_t e_ = hipGetLastError();                                                     \
    if (e_ != hipSuccess)                                                                  \
      return ::nmtg::fail(NMTG_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e_)); \
  } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

int num_cus();  // compute units of the current device (cached per device)

constexpr int kWave = 64;

// ---------------------------------------------------------------------------------------------
// Element types. Storage types are raw 16-bit patterns for half / bfloat16 so that vector loads
// are plain integer loads; conversion is explicit.
// ---------------------------------------------------------------------------------------------
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };

template <typename T> struct elem;
template <> struct elem<float> {
  static constexpr int dtype = NMTG_F32;
  static __device__ __forceinline__ float to_float(float v) { return v; }
  static __device__ __forceinline__ float from_float(float v) { return v; }
};
template <> struct elem<f16_t> {
  static constexpr int dtype = NMTG_F16;
  static __device__ __forceinline__ float to_float(f16_t v) {
    return __half2float(__ushort_as_half(v.bits));
  }
  static __device__ __forceinline__ f16_t from_float(float v) {
    f16_t r; r.bits = __half_as_ushort(__float2half_rn(v)); return r;
  }
};
template <> struct elem<bf16_t> {
  static constexpr int dtype = NMTG_BF16;
  static __device__ __forceinline__ float to_float(bf16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v.bits) << 16);
  }
  // round-to-nearest-even, NaN kept quiet
  static __device__ __forceinline__ bf16_t from_float(float v) {
    uint32_t u = __float_as_uint(v);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) { r.bits = static_cast<uint16_t>((u >> 16) | 0x40u); return r; }
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = static_cast<uint16_t>(u >> 16);
    return r;
  }
};

// A pack of N elements of T moved with the widest loads/stores its byte size allows.
template <typename T, int N> struct alignas(sizeof(T) * N >= 16 ? 16 : sizeof(T) * N) pack {
  T v[N];
};

template <typename T, int N>
__device__ __forceinline__ void load_pack(const T* __restrict__ p, float (&out)[N]) {
  constexpr int BYTES = sizeof(T) * N;
  if constexpr (BYTES % 16 == 0) {
    constexpr int NV = BYTES / 16;
    constexpr int PER = 16 / sizeof(T);
    const uint4* q = reinterpret_cast<const uint4*>(p);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      uint4 raw = q[i];
      const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
      for (int j = 0; j < PER; ++j) out[i * PER + j] = elem<T>::to_float(e[j]);
    }
  } else if constexpr (BYTES == 8) {
    uint2 raw = *reinterpret_cast<const uint2*>(p);
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = elem<T>::to_float(e[j]);
  } else if constexpr (BYTES == 4) {
    uint32_t raw = *reinterpret_cast<const uint32_t*>(p);
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = elem<T>::to_float(e[j]);
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = elem<T>::to_float(p[j]);
  }
}

template <typename T, int N>
__device__ __forceinline__ void store_pack(T* __restrict__ p, const float (&in)[N]) {
  constexpr int BYTES = sizeof(T) * N;
  if constexpr (BYTES % 16 == 0) {
    constexpr int NV = BYTES / 16;
    constexpr int PER = 16 / sizeof(T);
    uint4* q = reinterpret_cast<uint4*>(p);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      uint4 raw;
      T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
      for (int j = 0; j < PER; ++j) e[j] = elem<T>::from_float(in[i * PER + j]);
      q[i] = raw;
    }
  } else if constexpr (BYTES == 8) {
    uint2 raw;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int j = 0; j < N; ++j) e[j] = elem<T>::from_float(in[j]);
    *reinterpret_cast<uint2*>(p) = raw;
  } else if constexpr (BYTES == 4) {
    uint32_t raw;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int j = 0; j < N; ++j) e[j] = elem<T>::from_float(in[j]);
    *reinterpret_cast<uint32_t*>(p) = raw;
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) p[j] = elem<T>::from_float(in[j]);
  }
}

// ---------------------------------------------------------------------------------------------
// Wavefront (64 lanes) reductions: butterfly over lanes, every lane ends with the result.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}
__device__ __forceinline__ void wave_sum2(float& a, float& b) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    a += __shfl_xor(a, m, 64);
    b += __shfl_xor(b, m, 64);
  }
}

// Dispatch a runtime dtype code to a template parameter.
#define NMTG_DISPATCH_DTYPE(code, T, ...)                                   \
  switch (code) {                                                           \
    case NMTG_F32: { using T = float; __VA_ARGS__; break; }                 \
    case NMTG_F16: { using T = ::nmtg::f16_t; __VA_ARGS__; break; }         \
    case NMTG_BF16: { using T = ::nmtg::bf16_t; __VA_ARGS__; break; }       \
    default: return ::nmtg::fail(NMTG_ERR_INVALID, "unknown dtype code %d", (int)(code)); \
  }

}  // namespace nmtg
