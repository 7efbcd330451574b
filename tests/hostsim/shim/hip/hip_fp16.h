// Host stand-in for <hip/hip_fp16.h>: IEEE binary16 <-> float in software (round to nearest even).
#pragma once
#include <cstdint>
#include <cstring>

struct __half { uint16_t bits; };
static inline __half __ushort_as_half(uint16_t b) { return __half{b}; }
static inline uint16_t __half_as_ushort(__half h) { return h.bits; }

static inline float __half2float(__half h) {
  const uint32_t sign = static_cast<uint32_t>(h.bits & 0x8000u) << 16;
  uint32_t exp = (h.bits >> 10) & 0x1fu, man = h.bits & 0x3ffu, out;
  if (exp == 0x1f) out = sign | 0x7f800000u | (man << 13);                 // inf / nan
  else if (exp != 0) out = sign | ((exp + 112u) << 23) | (man << 13);      // normal
  else if (man == 0) out = sign;                                            // zero
  else {                                                                    // subnormal: renormalise
    int e = -1;
    do { man <<= 1; ++e; } while ((man & 0x400u) == 0);
    out = sign | ((112u - e) << 23) | ((man & 0x3ffu) << 13);
  }
  float f; std::memcpy(&f, &out, 4); return f;
}

static inline __half __float2half_rn(float f) {
  uint32_t x; std::memcpy(&x, &f, 4);
  const uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
  const uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return __half{static_cast<uint16_t>(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u | ((ax >> 13) & 0x3ffu) : 0u))};
  if (ax >= 0x477ff000u) return __half{static_cast<uint16_t>(sign | 0x7c00u)};     // rounds to >= 65520 -> inf
  if (ax < 0x33000001u) return __half{sign};                                        // <= 2^-25 -> zero
  int exp = static_cast<int>(ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u;                                      // 24-bit significand
  int shift = exp >= -14 ? 13 : 13 + (-14 - exp);                                   // bits dropped
  uint32_t kept = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) ++kept;
  uint32_t out = exp >= -14 ? ((static_cast<uint32_t>(exp + 15) << 10) + (kept - 0x400u)) : kept;  // carries propagate
  return __half{static_cast<uint16_t>(sign | out)};
}
