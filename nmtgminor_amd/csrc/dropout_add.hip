// Dropout + residual add, and its backward (masked scale), for gfx950.
//
// Stands in for fused_dropout_add_cuda.forward / backward of the reference
// (onmt/modules/extensions/dropout_add/fused_dropout_add_cuda_kernel.cu:19-95, kernels
// dropout.h:72-189). out = residual + x * keep / (1 - p), written in place into x; the keep mask
// is one byte per element (1 = keep). The mask either comes from the caller (replay / tests) or
// is drawn here from Philox4x32-10 keyed by (seed, offset, element index).
//
// Bandwidth bound: forward reads x and residual, writes x and 1 B/element of mask; backward
// reads g and the mask, writes dx. Each lane moves 16 bytes per access; the grid covers the
// tensor once (no grid-stride tail) so every CU streams contiguous 4 KiB wavefront chunks.
#include "common.hip.h"

namespace nmtg {
namespace {

constexpr int DA_THREADS = 256;
enum { DA_EVAL = 0, DA_MASK_IN = 1, DA_MASK_RNG = 2 };

template <typename T, int EPV, int MODE>
__global__ __launch_bounds__(DA_THREADS) void dropout_add_fwd_kernel(
    T* __restrict__ x, const T* __restrict__ residual, uint8_t* __restrict__ mask, int64_t n, float keep_p,
    float scale, uint64_t seed, uint64_t offset) {
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * DA_THREADS + threadIdx.x) * EPV;
  if (first >= n) return;
  if (first + EPV <= n) {
    // all loads are issued before the first conversion, so the lane waits for memory once
    pack<T, EPV> rawx = load_raw<T, EPV>(x + first), rawr = load_raw<T, EPV>(residual + first);
    pack<uint8_t, EPV> rawm = {};
    if constexpr (MODE == DA_MASK_IN) rawm = load_raw<uint8_t, EPV>(mask + first);
    pin_raw(rawx); pin_raw(rawr); pin_raw(rawm);
    float xv[EPV], rv[EPV];
    unpack_raw<T, EPV>(rawx, xv);
    unpack_raw<T, EPV>(rawr, rv);
    if constexpr (MODE == DA_EVAL) {
#pragma unroll
      for (int j = 0; j < EPV; ++j) xv[j] += rv[j];
    } else {
      uint8_t keep[EPV];
      if constexpr (MODE == DA_MASK_IN) {
#pragma unroll
        for (int j = 0; j < EPV; ++j) keep[j] = rawm.v[j];
      } else {
        philox_keep<EPV>(Philox(seed), static_cast<uint64_t>(first), offset, keep_p, keep);
        store_bytes<EPV>(mask + first, keep);
      }
#pragma unroll
      for (int j = 0; j < EPV; ++j) xv[j] = rv[j] + (keep[j] ? xv[j] * scale : 0.f);
    }
    store_pack<T, EPV>(x + first, xv);
  } else {  // ragged tail: scalar
    for (int64_t e = first; e < n; ++e) {
      float xv = elem<T>::to_float(x[e]);
      const float rv = elem<T>::to_float(residual[e]);
      if constexpr (MODE == DA_EVAL) {
        xv += rv;
      } else {
        uint8_t keep[1];
        if constexpr (MODE == DA_MASK_IN) keep[0] = mask[e];
        else { philox_keep<1>(Philox(seed), static_cast<uint64_t>(e), offset, keep_p, keep); mask[e] = keep[0]; }
        xv = rv + (keep[0] ? xv * scale : 0.f);
      }
      x[e] = elem<T>::from_float(xv);
    }
  }
}

template <typename T, int EPV>
__global__ __launch_bounds__(DA_THREADS) void masked_scale_kernel(
    const T* __restrict__ g, const uint8_t* __restrict__ mask, T* __restrict__ dx, int64_t n, float scale) {
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * DA_THREADS + threadIdx.x) * EPV;
  if (first >= n) return;
  if (first + EPV <= n) {
    float gv[EPV];
    uint8_t keep[EPV];
    load_pack<T, EPV>(g + first, gv);
    load_bytes<EPV>(mask + first, keep);
#pragma unroll
    for (int j = 0; j < EPV; ++j) gv[j] = keep[j] ? gv[j] * scale : 0.f;
    store_pack<T, EPV>(dx + first, gv);
  } else {
    for (int64_t e = first; e < n; ++e)
      dx[e] = elem<T>::from_float(mask[e] ? elem<T>::to_float(g[e]) * scale : 0.f);
  }
}

template <typename T>
int dropout_add_fwd_launch(void* x, const void* residual, uint8_t* mask, int64_t n, float p, int mode,
                           uint64_t seed, uint64_t offset, hipStream_t st) {
  const float keep_p = 1.f - p, scale = 1.f / (1.f - p);
  T* X = static_cast<T*>(x);
  const T* R = static_cast<const T*>(residual);
  constexpr int WIDE = 16 / sizeof(T);
  TraceScope trace("dropout_add_fwd", st);
  const bool wide = aligned16(x) && aligned16(residual) && (mode == DA_EVAL || aligned8(mask));
#define DA_LAUNCH(EPV, MODE)                                                                         \
  {                                                                                                  \
    const int64_t per_block = static_cast<int64_t>(DA_THREADS) * EPV;                                \
    const int64_t grid = (n + per_block - 1) / per_block;                                            \
    hipLaunchKernelGGL((dropout_add_fwd_kernel<T, EPV, MODE>), dim3(static_cast<unsigned>(grid)),    \
                       dim3(DA_THREADS), 0, st, X, R, mask, n, keep_p, scale, seed, offset);         \
  }
  if (wide) {
    if (mode == DA_EVAL) DA_LAUNCH(WIDE, DA_EVAL)
    else if (mode == DA_MASK_IN) DA_LAUNCH(WIDE, DA_MASK_IN)
    else DA_LAUNCH(WIDE, DA_MASK_RNG)
  } else {
    if (mode == DA_EVAL) DA_LAUNCH(1, DA_EVAL)
    else if (mode == DA_MASK_IN) DA_LAUNCH(1, DA_MASK_IN)
    else DA_LAUNCH(1, DA_MASK_RNG)
  }
#undef DA_LAUNCH
  return 0;
}

template <typename T>
int masked_scale_launch(const void* g, const uint8_t* mask, void* dx, int64_t n, float p, hipStream_t st) {
  const float scale = 1.f / (1.f - p);
  constexpr int WIDE = 16 / sizeof(T);
  const bool wide = aligned16(g) && aligned16(dx) && aligned8(mask);
  TraceScope trace("dropout_add_bwd", st);
  if (wide) {
    const int64_t per_block = static_cast<int64_t>(DA_THREADS) * WIDE;
    hipLaunchKernelGGL((masked_scale_kernel<T, WIDE>), dim3(static_cast<unsigned>((n + per_block - 1) / per_block)),
                       dim3(DA_THREADS), 0, st, static_cast<const T*>(g), mask, static_cast<T*>(dx), n, scale);
  } else {
    hipLaunchKernelGGL((masked_scale_kernel<T, 1>), dim3(static_cast<unsigned>((n + DA_THREADS - 1) / DA_THREADS)),
                       dim3(DA_THREADS), 0, st, static_cast<const T*>(g), mask, static_cast<T*>(dx), n, scale);
  }
  return 0;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_dropout_add_fwd(void* x, const void* residual, uint8_t* mask, int64_t n, float p,
                                    int mask_mode, uint64_t seed, uint64_t offset, int dtype, void* stream) {
  NMTG_REQUIRE(n >= 0 && n < (int64_t(1) << 40), "dropout_add_fwd: bad element count %lld", (long long)n);
  NMTG_REQUIRE(mask_mode >= DA_EVAL && mask_mode <= DA_MASK_RNG, "dropout_add_fwd: bad mask_mode %d", mask_mode);
  if (n == 0) return 0;
  NMTG_REQUIRE(x && residual, "dropout_add_fwd: null pointer argument");
  if (mask_mode != DA_EVAL) {
    NMTG_REQUIRE(mask != nullptr, "dropout_add_fwd: mask buffer required when dropout is applied");
    NMTG_REQUIRE(p >= 0.f && p < 1.f, "dropout_add_fwd: dropout probability %f outside [0, 1)", p);
  }
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = dropout_add_fwd_launch<T>(x, residual, mask, n, p, mask_mode, seed, offset,
                                                                static_cast<hipStream_t>(stream)));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("dropout_add_fwd");
  return 0;
}

extern "C" int nmtg_dropout_add_bwd(const void* grad_out, const uint8_t* mask, void* grad_x, int64_t n, float p,
                                    int dtype, void* stream) {
  NMTG_REQUIRE(n >= 0 && n < (int64_t(1) << 40), "dropout_add_bwd: bad element count %lld", (long long)n);
  if (n == 0) return 0;
  NMTG_REQUIRE(grad_out && mask && grad_x, "dropout_add_bwd: null pointer argument");
  NMTG_REQUIRE(p >= 0.f && p < 1.f, "dropout_add_bwd: dropout probability %f outside [0, 1)", p);
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = masked_scale_launch<T>(grad_out, mask, grad_x, n, p, static_cast<hipStream_t>(stream)));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("dropout_add_bwd");
  return 0;
}
