// Gated feed-forward activation with dropout, forward and backward, for gfx950.
//
// The gated branch of the reference's PositionWiseFeedForward (onmt/modules/optimized/feed_forward.py:188-200), which
// runs there as PyTorch ops: the first projection yields [rows, 2 * inner]; with a = its first half and b = its second,
//     y = act(a) * b                     for relu / gelu / silu / agelu          (:190-192)
//     y = a * sigmoid(b)                 for the 'sigmoid' activation (F.glu)    (:57-58, :194)
// followed by dropout: independent per element (F.dropout, :199) or one mask row shared by all time steps
// ("variational", onmt/modules/dropout.py:32-48: a [1, batch, inner] mask over a [time, batch, inner] tensor).
//
// Bandwidth bound: the forward reads 2 * inner and writes inner elements per row (+ 1 byte of mask per output when the
// mask is drawn here), the backward reads 3 * inner and writes 2 * inner. Each lane moves 16 bytes per access.
#include "gemm.hip.h"

namespace nmtg {
namespace {

constexpr int GLU_THREADS = 256;
constexpr int GLU_SIGMOID = 5;   // activation code of the F.glu form, beside the nmtg_act codes

struct GluArgs {
  const void* x;       // [rows, 2 * inner], row pitch ld_x
  void* y;             // forward: [rows, inner] dense
  const void* g;       // backward: gradient of y, [rows, inner] dense
  void* dx;            // backward: [rows, 2 * inner], row pitch ld_dx
  uint8_t* mask;       // keep flags [mask_rows, inner]; row m of x uses mask row m % mask_rows
  int64_t ld_x, ld_dx, rows, mask_rows;
  int inner;
  int mode;            // 0 no dropout, 1 read the mask, 2 draw it (dense: mask_rows == rows) and store it
  float keep_p, scale;
  uint64_t seed, offset;
};

__device__ __forceinline__ float sigmoidf_fast(float v) { return fast_rcp(1.f + fast_exp2(v * -1.4426950408889634f)); }

template <int ACT>
__device__ __forceinline__ float glu_value(float a, float b) {
  if constexpr (ACT == GLU_SIGMOID) return a * sigmoidf_fast(b);
  else return act_apply<ACT>(a, nullptr) * b;
}
template <int ACT>
__device__ __forceinline__ void glu_grads(float a, float b, float gy, float& da, float& db) {
  if constexpr (ACT == GLU_SIGMOID) {
    const float s = sigmoidf_fast(b);
    da = gy * s;
    db = gy * a * s * (1.f - s);
  } else {
    da = gy * act_grad<ACT>(a, nullptr) * b;
    db = gy * act_apply<ACT>(a, nullptr);
  }
}

template <typename F>
__device__ __forceinline__ void dispatch_glu(int act, F&& f) {
  switch (act) {
    case NMTG_ACT_RELU: f(std::integral_constant<int, NMTG_ACT_RELU>{}); break;
    case NMTG_ACT_GELU: f(std::integral_constant<int, NMTG_ACT_GELU>{}); break;
    case NMTG_ACT_SILU: f(std::integral_constant<int, NMTG_ACT_SILU>{}); break;
    case NMTG_ACT_AGELU: f(std::integral_constant<int, NMTG_ACT_AGELU>{}); break;
    case GLU_SIGMOID: f(std::integral_constant<int, GLU_SIGMOID>{}); break;
    default: f(std::integral_constant<int, NMTG_ACT_NONE>{}); break;
  }
}

// One lane per EPV consecutive outputs of one row.
template <typename T, int EPV, bool BWD>
__global__ __launch_bounds__(GLU_THREADS) void glu_kernel(GluArgs p, int act) {
  const int per_row = p.inner / EPV;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * GLU_THREADS + threadIdx.x;
  if (item >= p.rows * per_row) return;
  const int64_t m = item / per_row;
  const int j = static_cast<int>(item % per_row) * EPV;
  const T* xr = static_cast<const T*>(p.x) + m * p.ld_x + j;
  pack<T, EPV> ra = load_raw<T, EPV>(xr), rb = load_raw<T, EPV>(xr + p.inner), rg = {};
  if constexpr (BWD) rg = load_raw<T, EPV>(static_cast<const T*>(p.g) + m * p.inner + j);
  uint8_t keep[EPV];
  const int64_t mrow = p.mask_rows == p.rows ? m : m % p.mask_rows;
  uint8_t* mk = p.mask + mrow * p.inner + j;
  if (p.mode == 1) {
    load_bytes<EPV>(mk, keep);
  } else if (p.mode == 2 && !BWD) {
    const uint64_t first = static_cast<uint64_t>(m) * p.inner + j;
    if constexpr (EPV >= 4) {
      philox_keep<EPV>(Philox(p.seed), first, p.offset, p.keep_p, keep);     // first is a multiple of 4 on this path
    } else {
#pragma unroll
      for (int e = 0; e < EPV; ++e) {
        uint8_t one[1];
        philox_keep<1>(Philox(p.seed), first + e, p.offset, p.keep_p, one);
        keep[e] = one[0];
      }
    }
    store_bytes<EPV>(mk, keep);
  } else {
#pragma unroll
    for (int e = 0; e < EPV; ++e) keep[e] = 1;
  }
  float a[EPV], b[EPV], g[EPV];
  unpack_raw<T, EPV>(ra, a);
  unpack_raw<T, EPV>(rb, b);
  if constexpr (BWD) unpack_raw<T, EPV>(rg, g);
  dispatch_glu(act, [&](auto tag) {
    constexpr int ACT = decltype(tag)::value;
    if constexpr (!BWD) {
      float y[EPV];
#pragma unroll
      for (int e = 0; e < EPV; ++e) y[e] = keep[e] ? glu_value<ACT>(a[e], b[e]) * p.scale : 0.f;
      store_pack<T, EPV>(static_cast<T*>(p.y) + m * p.inner + j, y);
    } else {
      float da[EPV], db[EPV];
#pragma unroll
      for (int e = 0; e < EPV; ++e) glu_grads<ACT>(a[e], b[e], keep[e] ? g[e] * p.scale : 0.f, da[e], db[e]);
      T* dr = static_cast<T*>(p.dx) + m * p.ld_dx + j;
      store_pack<T, EPV>(dr, da);
      store_pack<T, EPV>(dr + p.inner, db);
    }
  });
}

template <typename T, bool BWD>
int glu_launch(const GluArgs& p, int act, hipStream_t st) {
  constexpr int WIDE = 16 / sizeof(T);
  auto ok = [&](const void* ptr, int64_t ld) { return ptr == nullptr || (reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && ld % WIDE == 0); };
  const bool wide = p.inner % WIDE == 0 && ok(p.x, p.ld_x) && ok(p.y, p.inner) && ok(p.g, p.inner) && ok(p.dx, p.ld_dx) &&
                    (p.mode == 0 || reinterpret_cast<uintptr_t>(p.mask) % WIDE == 0);
  const int epv = wide ? WIDE : 1;
  const int64_t items = p.rows * (p.inner / epv);
  const int64_t grid = (items + GLU_THREADS - 1) / GLU_THREADS;
  if (grid > 0x7fffffff) return fail(NMTG_ERR_UNSUPPORTED, "glu: too many elements for one launch");
  TraceScope trace(BWD ? "glu_bwd" : "glu_fwd", st);
  if (wide) hipLaunchKernelGGL((glu_kernel<T, WIDE, BWD>), dim3(static_cast<unsigned>(grid)), dim3(GLU_THREADS), 0, st, p, act);
  else hipLaunchKernelGGL((glu_kernel<T, 1, BWD>), dim3(static_cast<unsigned>(grid)), dim3(GLU_THREADS), 0, st, p, act);
  return 0;
}

int glu_check(const char* who, int64_t rows, int64_t inner, int64_t ld, int act, int mode, float p, int64_t mask_rows,
              const void* mask) {
  NMTG_REQUIRE(rows >= 0 && inner >= 1 && inner <= (1 << 30) && ld >= 2 * inner, "%s: bad shape rows=%lld inner=%lld pitch=%lld", who,
               (long long)rows, (long long)inner, (long long)ld);
  NMTG_REQUIRE((act >= NMTG_ACT_NONE && act <= NMTG_ACT_AGELU) || act == GLU_SIGMOID, "%s: unknown activation %d", who, act);
  NMTG_REQUIRE(mode >= 0 && mode <= 2, "%s: dropout mode %d", who, mode);
  NMTG_REQUIRE(mode == 0 || (p >= 0.f && p < 1.f), "%s: dropout probability %g outside [0, 1)", who, (double)p);
  NMTG_REQUIRE(mode == 0 || mask != nullptr, "%s: dropout needs a mask buffer", who);
  NMTG_REQUIRE(mode == 0 || (mask_rows >= 1 && (mask_rows == rows || rows % mask_rows == 0)),
               "%s: %lld mask rows do not divide %lld rows", who, (long long)mask_rows, (long long)rows);
  return 0;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_glu_fwd(const void* x, int64_t ld_x, void* y, uint8_t* mask, int64_t mask_rows, int64_t rows, int64_t inner,
                            int act, int dropout_mode, float p, uint64_t seed, uint64_t offset, int dtype, void* stream) {
  if (int rc = glu_check("glu_fwd", rows, inner, ld_x, act, dropout_mode, p, mask_rows, mask)) return rc;
  NMTG_REQUIRE(dropout_mode != 2 || mask_rows == rows, "glu_fwd: a drawn mask has one row per input row");
  if (rows == 0) return 0;
  NMTG_REQUIRE(x && y, "glu_fwd: null pointer argument");
  GluArgs a = {};
  a.x = x; a.y = y; a.mask = mask; a.ld_x = ld_x; a.rows = rows; a.mask_rows = dropout_mode ? mask_rows : rows;
  a.inner = static_cast<int>(inner); a.mode = dropout_mode;
  a.keep_p = 1.f - p; a.scale = dropout_mode ? 1.f / (1.f - p) : 1.f; a.seed = seed; a.offset = offset;
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = (glu_launch<T, false>(a, act, static_cast<hipStream_t>(stream))));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("glu_fwd");
  return 0;
}

extern "C" int nmtg_glu_bwd(const void* grad_y, const void* x, int64_t ld_x, const uint8_t* mask, int64_t mask_rows, void* grad_x,
                            int64_t ld_grad_x, int64_t rows, int64_t inner, int act, int dropout_mode, float p, int dtype,
                            void* stream) {
  if (int rc = glu_check("glu_bwd", rows, inner, ld_x, act, dropout_mode, p, mask_rows, mask)) return rc;
  NMTG_REQUIRE(dropout_mode != 2, "glu_bwd: the backward reads the mask the forward stored (mode 0 or 1)");
  NMTG_REQUIRE(ld_grad_x >= 2 * inner, "glu_bwd: gradient pitch %lld below 2 * inner", (long long)ld_grad_x);
  if (rows == 0) return 0;
  NMTG_REQUIRE(grad_y && x && grad_x, "glu_bwd: null pointer argument");
  GluArgs a = {};
  a.x = x; a.g = grad_y; a.dx = grad_x; a.mask = const_cast<uint8_t*>(mask); a.ld_x = ld_x; a.ld_dx = ld_grad_x; a.rows = rows;
  a.mask_rows = dropout_mode ? mask_rows : rows;
  a.inner = static_cast<int>(inner); a.mode = dropout_mode;
  a.keep_p = 1.f - p; a.scale = dropout_mode ? 1.f / (1.f - p) : 1.f;
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = (glu_launch<T, true>(a, act, static_cast<hipStream_t>(stream))));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("glu_bwd");
  return 0;
}
