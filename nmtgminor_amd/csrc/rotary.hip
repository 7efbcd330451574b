// Rotary position encoding of queries / keys, in place, and its transpose for the backward pass (gfx950).
//
// Stands in for what the reference's attention functions do with PyTorch ops when rotary_pos_enc is set
// (onmt/modules/optimized/self_attention_func.py:25-48 rotate_half / apply_rotary_pos_emb / rotate_backward, applied
// to views of the in-projection output at :178-184 and to their gradients at :467-469;
// onmt/modules/optimized/encdec_attention_func.py:21-34 for the one-operand form):
//   forward : y = x * cos + rotate_half(x) * sin,          rotate_half(x) = cat(-x[D/2:], x[:D/2])
//   backward: dx = g * cos + rotate_backward(sin * g),      rotate_backward(u) = cat(u[D/2:], -u[:D/2])
// cos, sin are [T, D] (the reference's [T, 1, D], broadcast over batch * heads). Element j < D/2 pairs with j + D/2:
//   forward : y_j = x_j c_j - x_{j+h} s_j           y_{j+h} = x_{j+h} c_{j+h} + x_j s_{j+h}
//   backward: dx_j = g_j c_j + g_{j+h} s_{j+h}      dx_{j+h} = g_{j+h} c_{j+h} - g_j s_j
// The operand is addressed as x[t * stride_t + n * stride_n + part * stride_part + j]: the query and key slots of the
// head-interleaved projection [T, B*H, 3, D] are two parts of one launch. One thread owns EPV pairs. Bandwidth bound:
// one read and one write of the rotated slots.
#include "common.hip.h"

namespace nmtg {
namespace {

constexpr int RO_THREADS = 256;

template <typename T, int EPV, bool INVERSE>
__global__ __launch_bounds__(RO_THREADS) void rotary_kernel(T* __restrict__ x, const T* __restrict__ cosv,
                                                            const T* __restrict__ sinv, int64_t items, int n, int half,
                                                            int nparts, int64_t stride_t, int64_t stride_n,
                                                            int64_t stride_part) {
  const int64_t item = static_cast<int64_t>(blockIdx.x) * RO_THREADS + threadIdx.x;
  if (item >= items) return;
  const int per_head = half / EPV;
  const int j = static_cast<int>(item % per_head) * EPV;
  int64_t r = item / per_head;
  const int part = static_cast<int>(r % nparts); r /= nparts;
  const int head = static_cast<int>(r % n);
  const int64_t t = r / n;
  T* p = x + t * stride_t + head * stride_n + part * stride_part + j;
  const T* c = cosv + t * (2 * half) + j;
  const T* s = sinv + t * (2 * half) + j;
  float a[EPV], b[EPV], ca[EPV], cb[EPV], sa[EPV], sb[EPV];
  load_pack<T, EPV>(p, a);
  load_pack<T, EPV>(p + half, b);
  load_pack<T, EPV>(c, ca);
  load_pack<T, EPV>(c + half, cb);
  load_pack<T, EPV>(s, sa);
  load_pack<T, EPV>(s + half, sb);
  float ya[EPV], yb[EPV];
#pragma unroll
  for (int k = 0; k < EPV; ++k) {
    if constexpr (!INVERSE) {
      ya[k] = a[k] * ca[k] - b[k] * sa[k];
      yb[k] = b[k] * cb[k] + a[k] * sb[k];
    } else {
      ya[k] = a[k] * ca[k] + b[k] * sb[k];
      yb[k] = b[k] * cb[k] - a[k] * sa[k];
    }
  }
  store_pack<T, EPV>(p, ya);
  store_pack<T, EPV>(p + half, yb);
}

template <typename T>
int rotary_launch(void* x, const void* cosv, const void* sinv, int64_t t, int64_t n, int64_t d, int64_t nparts,
                  int64_t stride_t, int64_t stride_n, int64_t stride_part, bool inverse, hipStream_t st) {
  constexpr int WIDE = 16 / sizeof(T);
  const int half = static_cast<int>(d / 2);
  const uintptr_t bytes = WIDE * sizeof(T);
  const bool wide = half % WIDE == 0 && stride_t % WIDE == 0 && stride_n % WIDE == 0 && stride_part % WIDE == 0 &&
                    reinterpret_cast<uintptr_t>(x) % bytes == 0 && reinterpret_cast<uintptr_t>(cosv) % bytes == 0 &&
                    reinterpret_cast<uintptr_t>(sinv) % bytes == 0;
  TraceScope trace(inverse ? "rotary_bwd" : "rotary_fwd", st);
#define RO_LAUNCH(EPV, INV)                                                                                          \
  {                                                                                                                  \
    const int64_t items = t * n * nparts * (half / EPV);                                                             \
    const int64_t grid = (items + RO_THREADS - 1) / RO_THREADS;                                                      \
    if (grid > 0x7fffffff) return fail(NMTG_ERR_UNSUPPORTED, "rotary: too many elements for one launch");            \
    hipLaunchKernelGGL((rotary_kernel<T, EPV, INV>), dim3(static_cast<unsigned>(grid)), dim3(RO_THREADS), 0, st,      \
                       static_cast<T*>(x), static_cast<const T*>(cosv), static_cast<const T*>(sinv), items,           \
                       static_cast<int>(n), half, static_cast<int>(nparts), stride_t, stride_n, stride_part);         \
  }
  if (wide) { if (inverse) RO_LAUNCH(WIDE, true) else RO_LAUNCH(WIDE, false) }
  else { if (inverse) RO_LAUNCH(1, true) else RO_LAUNCH(1, false) }
#undef RO_LAUNCH
  return 0;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_rotary(void* x, const void* cos_table, const void* sin_table, int64_t t, int64_t n, int64_t d,
                           int64_t nparts, int64_t stride_t, int64_t stride_n, int64_t stride_part, int inverse,
                           int dtype, void* stream) {
  NMTG_REQUIRE(t >= 0 && n >= 0 && d > 0 && d % 2 == 0 && d <= (1 << 20) && nparts >= 1 && nparts <= 4 && n <= INT32_MAX,
               "rotary: bad shape t=%lld n=%lld d=%lld parts=%lld (the head dimension must be even)", (long long)t,
               (long long)n, (long long)d, (long long)nparts);
  NMTG_REQUIRE(stride_n >= 0 && stride_t >= 0 && stride_part >= 0, "rotary: negative stride");
  // the rotated slots must not overlap: a part holds d elements, a head nparts parts, a position n heads
  NMTG_REQUIRE((nparts == 1 || stride_part >= d) && (n <= 1 || stride_n >= (nparts - 1) * stride_part + d) &&
                   (t <= 1 || stride_t >= (n - 1) * stride_n + (nparts - 1) * stride_part + d),
               "rotary: strides (%lld, %lld, %lld) let the rotated slots overlap", (long long)stride_t, (long long)stride_n,
               (long long)stride_part);
  if (t == 0 || n == 0) return 0;
  NMTG_REQUIRE(x && cos_table && sin_table, "rotary: null pointer argument");
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = rotary_launch<T>(x, cos_table, sin_table, t, n, d, nparts, stride_t, stride_n, stride_part,
                                                      inverse != 0, static_cast<hipStream_t>(stream)));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("rotary");
  return 0;
}
