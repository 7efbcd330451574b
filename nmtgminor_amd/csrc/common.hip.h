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
#include <cstdlib>

#include "../../include/nmtg_hip.h"
#include "trace.hip.h"

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

// Diagnostic switches: NAME=0 in the environment selects the plainer of two validated code paths (read on every
// call, so that one process can run both and compare them).
inline bool switched_off(const char* name) {
  const char* e = getenv(name);
  return e != nullptr && e[0] == '0';
}

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
  // round-to-nearest-even in hardware (v_cvt_pk_bf16_f32 on gfx950)
  static __device__ __forceinline__ bf16_t from_float(float v) {
    const __bf16 b = static_cast<__bf16>(v);
    bf16_t r;
    r.bits = __builtin_bit_cast(uint16_t, b);
    return r;
  }
};

// A pack of N elements of T moved with the widest loads/stores its byte size allows.
template <typename T, int N> struct alignas(sizeof(T) * N >= 16 ? 16 : sizeof(T) * N) pack {
  T v[N];
};

// Load without conversion / conversion without load: a kernel that wants several loads in flight issues all its
// load_raw calls first and converts afterwards (a conversion is a use of the loaded registers, and the compiler
// waits for a load at its first use).
template <typename T, int N>
__device__ __forceinline__ pack<T, N> load_raw(const T* __restrict__ p) {
  return *reinterpret_cast<const pack<T, N>*>(p);
}
// Pins a loaded pack in registers at this point of the program: the compiler may otherwise sink a load into the
// branch that holds its only use, where it waits for it alone.
template <typename T, int N>
__device__ __forceinline__ void pin_raw(pack<T, N>& r) {
  constexpr int WORDS = (sizeof(pack<T, N>) + 3) / 4;       // a pack narrower than a word is pinned in one word
  uint32_t w[WORDS] = {};
  __builtin_memcpy(w, &r, sizeof(r));
#pragma unroll
  for (int k = 0; k < WORDS; ++k) asm volatile("" : "+v"(w[k]));
  __builtin_memcpy(&r, w, sizeof(r));
}
template <typename T, int N>
__device__ __forceinline__ void unpack_raw(const pack<T, N>& r, float (&out)[N]) {
#pragma unroll
  for (int j = 0; j < N; ++j) out[j] = elem<T>::to_float(r.v[j]);
}

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
// Wavefront reductions on the DPP lane-exchange modifiers (no LDS traffic, no address arithmetic): four exchange steps
// leave every lane of a 16-lane row with the row's total, then the four row totals are read as scalars. The pairing
// is that of the xor butterfly (1, 2, 4, 8, 16, 32), so the result is the same in every lane, bit for bit.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_f32(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
template <typename Op>
__device__ __forceinline__ float wave_reduce(float v, Op op) {
  v = op(v, dpp_f32<0xB1>(v));    // quad_perm [1, 0, 3, 2]: lane ^ 1
  v = op(v, dpp_f32<0x4E>(v));    // quad_perm [2, 3, 0, 1]: lane ^ 2
  v = op(v, dpp_f32<0x141>(v));   // row_half_mirror: the other quad of each group of 8
  v = op(v, dpp_f32<0x140>(v));   // row_mirror: the other half of each row of 16
  return op(op(lane_f32(v, 0), lane_f32(v, 16)), op(lane_f32(v, 32), lane_f32(v, 48)));
}
__device__ __forceinline__ float wave_sum(float v) {
  return wave_reduce(v, [](float a, float b) { return a + b; });
}
__device__ __forceinline__ float wave_max(float v) {
  return wave_reduce(v, [](float a, float b) { return fmaxf(a, b); });
}
__device__ __forceinline__ void wave_sum2(float& a, float& b) {
  a = wave_sum(a);
  b = wave_sum(b);
}


// acc + a.lo * b.lo + a.hi * b.hi on one register of two 16-bit elements each (v_dot2c_f32_f16 / v_dot2c_f32_bf16): the
// inner step of the bandwidth-bound products (few-row projections, one-row attention), where converting every element
// to fp32 first would cost more instructions than the multiplications.
// Orders a wavefront's LDS writes before its later LDS reads of other lanes' data (and the reverse): the hardware runs
// one wavefront's LDS instructions in order, the fences keep the compiler from moving them.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T> __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc);
template <> __device__ __forceinline__ float dot2<f16_t>(uint32_t a, uint32_t b, float acc) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, a), __builtin_bit_cast(h2, b), acc, false);
}
template <> __device__ __forceinline__ float dot2<bf16_t>(uint32_t a, uint32_t b, float acc) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, a), __builtin_bit_cast(b2, b), acc, false);
}

// ---------------------------------------------------------------------------------------------
// Philox4x32-10 counter-based generator (Salmon et al., SC'11). One call turns a 128-bit
// counter and a 64-bit key into four 32-bit words. Dropout draws u = (word >> 8) * 2^-24 in
// [0, 1) and keeps an element when u < keep_probability.
// ---------------------------------------------------------------------------------------------
struct Philox {
  uint32_t key0, key1;
  __device__ __forceinline__ Philox(uint64_t seed) : key0(static_cast<uint32_t>(seed)), key1(static_cast<uint32_t>(seed >> 32)) {}
  __device__ __forceinline__ uint4 operator()(uint64_t index, uint64_t offset) const {
    uint32_t c0 = static_cast<uint32_t>(offset), c1 = static_cast<uint32_t>(offset >> 32);
    uint32_t c2 = static_cast<uint32_t>(index), c3 = static_cast<uint32_t>(index >> 32);
    uint32_t k0 = key0, k1 = key1;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
      // one 32x32->64 multiply per product (both halves from the same instruction)
      const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * c0, p1 = static_cast<uint64_t>(0xCD9E8D57u) * c2;
      const uint32_t hi0 = static_cast<uint32_t>(p0 >> 32), lo0 = static_cast<uint32_t>(p0);
      const uint32_t hi1 = static_cast<uint32_t>(p1 >> 32), lo1 = static_cast<uint32_t>(p1);
      const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
      c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
      k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    return make_uint4(c0, c1, c2, c3);
  }
};

__device__ __forceinline__ float u01(uint32_t w) { return static_cast<float>(w >> 8) * (1.0f / 16777216.0f); }

// Keep-decisions for N consecutive elements starting at linear element index `first` (first % 4
// == 0 when N >= 4): element i uses word (i % 4) of the Philox block with index i / 4, so the
// mask depends only on (seed, offset, element index), not on the launch shape.
template <int N>
__device__ __forceinline__ void philox_keep(const Philox& gen, uint64_t first, uint64_t offset, float keep_p,
                                            uint8_t (&keep)[N]) {
#ifdef NMTG_NO_PHILOX   // tuning builds only
  for (int i = 0; i < N; ++i) keep[i] = 1;
  return;
#endif
  if constexpr (N >= 4) {
#pragma unroll
    for (int b = 0; b < N / 4; ++b) {
      const uint4 r = gen(first / 4 + b, offset);
      keep[b * 4 + 0] = u01(r.x) < keep_p;
      keep[b * 4 + 1] = u01(r.y) < keep_p;
      keep[b * 4 + 2] = u01(r.z) < keep_p;
      keep[b * 4 + 3] = u01(r.w) < keep_p;
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const uint64_t e = first + i;
      const uint4 r = gen(e / 4, offset);
      const uint32_t w = (e & 3) == 0 ? r.x : (e & 3) == 1 ? r.y : (e & 3) == 2 ? r.z : r.w;
      keep[i] = u01(w) < keep_p;
    }
  }
}

template <int N>
__device__ __forceinline__ void load_bytes(const uint8_t* __restrict__ p, uint8_t (&out)[N]) {
  if constexpr (N == 8) {
    uint2 raw = *reinterpret_cast<const uint2*>(p);
    const uint8_t* e = reinterpret_cast<const uint8_t*>(&raw);
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = e[j];
  } else if constexpr (N == 4) {
    uint32_t raw = *reinterpret_cast<const uint32_t*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = (raw >> (8 * j)) & 0xffu;
  } else if constexpr (N == 2) {
    uint16_t raw = *reinterpret_cast<const uint16_t*>(p);
    out[0] = raw & 0xffu; out[1] = raw >> 8;
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = p[j];
  }
}

template <int N>
__device__ __forceinline__ void store_bytes(uint8_t* __restrict__ p, const uint8_t (&in)[N]) {
  if constexpr (N == 8) {
    uint2 raw;
    uint8_t* e = reinterpret_cast<uint8_t*>(&raw);
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = in[j];
    *reinterpret_cast<uint2*>(p) = raw;
  } else if constexpr (N == 4) {
    uint32_t raw = in[0] | (in[1] << 8) | (in[2] << 16) | (static_cast<uint32_t>(in[3]) << 24);
    *reinterpret_cast<uint32_t*>(p) = raw;
  } else if constexpr (N == 2) {
    *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(in[0] | (in[1] << 8));
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) p[j] = in[j];
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
