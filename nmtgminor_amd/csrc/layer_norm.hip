// LayerNorm forward / backward for gfx950.
//
// Stands in for fast_layer_norm_cuda.ln_fwd / ln_bwd of the reference
// (onmt/modules/extensions/layer_norm/ln_api.cpp:80-249, kernels ln_fwd_kernels.cuh:7-108 and
// ln_bwd_kernels.cuh:5-323). The design is not the reference's: there the hidden size is a
// template constant and rows are spread over 32-lane warps with a per-size launcher registry;
// here a row lives in the registers of WPR 64-lane wavefronts (VPL 16-byte vectors per lane),
// any hidden size is accepted, statistics are two-pass in registers, and the gamma/beta
// gradient is accumulated per lane over a block's rows and written as one partial row per block
// which a second small kernel sums in a fixed order (deterministic).
//
// HBM traffic per row of H elements (the kernels are bandwidth bound):
//   forward : read x, write z, +8 B (mu, rsigma)          -> 2 H elements
//   backward: read dz, x, write dx, +8 B                  -> 3 H elements (+ the [n_part, H]
//             fp32 partials once written and once read)
#include "common.hip.h"
#include <algorithm>

namespace nmtg {
namespace {

constexpr int LN_THREADS = 256;
constexpr int LN_WAVES = LN_THREADS / kWave;

template <typename T> struct ln_vec { static constexpr int EPV = 16 / sizeof(T); };

// Sum over the WPR wavefronts that share a row. WPR == 1: wavefront butterfly only.
template <int WPR>
__device__ __forceinline__ float row_sum(float v, float* smem, int wave) {
  v = wave_sum(v);
  if constexpr (WPR > 1) {
    __syncthreads();  // smem reuse guard
    if ((threadIdx.x & (kWave - 1)) == 0) smem[wave] = v;
    __syncthreads();
    const int base = (wave / WPR) * WPR;
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < WPR; ++i) t += smem[base + i];
    v = t;
  }
  return v;
}

template <int WPR>
__device__ __forceinline__ void row_sum2(float& a, float& b, float* smem, int wave) {
  wave_sum2(a, b);
  if constexpr (WPR > 1) {
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) { smem[wave] = a; smem[LN_WAVES + wave] = b; }
    __syncthreads();
    const int base = (wave / WPR) * WPR;
    float ta = 0.f, tb = 0.f;
#pragma unroll
    for (int i = 0; i < WPR; ++i) { ta += smem[base + i]; tb += smem[LN_WAVES + base + i]; }
    a = ta; b = tb;
  }
}

// ---------------------------------------------------------------------------------------------
// Forward: one row per WPR wavefronts, row held in registers.
// ---------------------------------------------------------------------------------------------
template <typename TI, typename TW, int VPL, int WPR>
__global__ __launch_bounds__(LN_THREADS) void ln_fwd_kernel(
    const TI* __restrict__ x, const TW* __restrict__ gamma, const TW* __restrict__ beta,
    TW* __restrict__ z, float* __restrict__ mu, float* __restrict__ rsigma, int64_t rows, int hidden,
    float eps) {
  constexpr int EPV = ln_vec<TI>::EPV;
  constexpr int RPB = LN_WAVES / WPR;  // rows per block per iteration
  __shared__ float smem[2 * LN_WAVES];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int sub = wave % WPR;  // which slice of the row this wavefront holds
  const float rn = 1.f / static_cast<float>(hidden);
  const int64_t groups = (rows + RPB - 1) / RPB;

  // Loads are issued unconditionally from clamped (always mapped) addresses and ahead of any use: a load inside a
  // branch waits for its own data before the next one is issued, which made a row cost four memory latencies.
  pack<TW, EPV> gr[VPL], br[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = ((sub * VPL + i) * kWave + lane) * EPV;
    const int cc = col < hidden ? col : 0;
    gr[i] = load_raw<TW, EPV>(gamma + cc);
    br[i] = load_raw<TW, EPV>(beta + cc);
  }

  for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
    const int64_t row = g * RPB + wave / WPR;
    const bool row_ok = row < rows;
    const int64_t rowc = row_ok ? row : 0;
    pack<TI, EPV> xr[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      xr[i] = load_raw<TI, EPV>(x + rowc * hidden + (col < hidden ? col : 0));
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) pin_raw(xr[i]);
    float xf[VPL][EPV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      if (row_ok && col < hidden) {
        unpack_raw<TI, EPV>(xr[i], xf[i]);
#pragma unroll
        for (int j = 0; j < EPV; ++j) s += xf[i][j];
      } else {
#pragma unroll
        for (int j = 0; j < EPV; ++j) xf[i][j] = 0.f;
      }
    }
    const float mean = row_sum<WPR>(s, smem, wave) * rn;
    float m2 = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      if (col < hidden) {
#pragma unroll
        for (int j = 0; j < EPV; ++j) { const float d = xf[i][j] - mean; m2 += d * d; }
      }
    }
    m2 = row_sum<WPR>(m2, smem, wave);
    const float rs = rsqrtf(m2 * rn + eps);
    if (row_ok && sub == 0 && lane == 0) { mu[row] = mean; rsigma[row] = rs; }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      if (row_ok && col < hidden) {
        float gf[EPV], bf[EPV], zf[EPV];
        unpack_raw<TW, EPV>(gr[i], gf);
        unpack_raw<TW, EPV>(br[i], bf);
#pragma unroll
        for (int j = 0; j < EPV; ++j) zf[j] = gf[j] * (rs * (xf[i][j] - mean)) + bf[j];
        store_pack<TW, EPV>(z + row * hidden + col, zf);
      }
    }
  }
}

// Fallback for hidden sizes that are not a multiple of the vector width or exceed what the
// register kernel holds: one block per row, three passes over the row (the re-reads hit cache).
template <typename TI, typename TW>
__global__ __launch_bounds__(LN_THREADS) void ln_fwd_generic_kernel(
    const TI* __restrict__ x, const TW* __restrict__ gamma, const TW* __restrict__ beta,
    TW* __restrict__ z, float* __restrict__ mu, float* __restrict__ rsigma, int64_t rows, int hidden,
    float eps) {
  __shared__ float smem[2 * LN_WAVES];
  const int wave = threadIdx.x / kWave;
  const float rn = 1.f / static_cast<float>(hidden);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const TI* xr = x + row * hidden;
    float s = 0.f;
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS) s += elem<TI>::to_float(xr[c]);
    const float mean = row_sum<LN_WAVES>(s, smem, wave) * rn;
    float m2 = 0.f;
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS) {
      const float d = elem<TI>::to_float(xr[c]) - mean;
      m2 += d * d;
    }
    m2 = row_sum<LN_WAVES>(m2, smem, wave);
    const float rs = rsqrtf(m2 * rn + eps);
    if (threadIdx.x == 0) { mu[row] = mean; rsigma[row] = rs; }
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS) {
      const float y = rs * (elem<TI>::to_float(xr[c]) - mean);
      z[row * hidden + c] =
          elem<TW>::from_float(elem<TW>::to_float(gamma[c]) * y + elem<TW>::to_float(beta[c]));
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Backward. MEMEFF: x_or_z holds z and y is rebuilt as (z - beta) / gamma
// (reference ln_bwd_kernels.cuh:91-110); otherwise y = rsigma * (x - mu).
// Each lane keeps running sums of dz and dz*y for its own columns over all rows the block
// visits; the block folds its wavefronts through LDS and writes one partial row.
// ---------------------------------------------------------------------------------------------
template <typename TI, typename TW, int VPL, int WPR, bool MEMEFF>
__global__ __launch_bounds__(LN_THREADS) void ln_bwd_kernel(
    const TW* __restrict__ dz, const TI* __restrict__ x_or_z, const float* __restrict__ mu,
    const float* __restrict__ rsigma, const TW* __restrict__ gamma, const TW* __restrict__ beta,
    TI* __restrict__ dx, float* __restrict__ dgamma_part, float* __restrict__ dbeta_part,
    int64_t rows, int hidden) {
  constexpr int EPV = ln_vec<TI>::EPV;
  constexpr int RPB = LN_WAVES / WPR;
  __shared__ float smem[2 * LN_WAVES];
  extern __shared__ float fold[];  // [RPB-1][2][WPR*VPL*64*EPV] when RPB > 1

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int sub = wave % WPR;
  const float rn = 1.f / static_cast<float>(hidden);
  const int64_t groups = (rows + RPB - 1) / RPB;

  float gf[VPL][EPV], bf[VPL][EPV];
  float dg_acc[VPL][EPV], db_acc[VPL][EPV];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = ((sub * VPL + i) * kWave + lane) * EPV;
    if (col < hidden) {
      load_pack<TW, EPV>(gamma + col, gf[i]);
      if constexpr (MEMEFF) load_pack<TW, EPV>(beta + col, bf[i]);
    } else {
#pragma unroll
      for (int j = 0; j < EPV; ++j) { gf[i][j] = 1.f; bf[i][j] = 0.f; }
    }
#pragma unroll
    for (int j = 0; j < EPV; ++j) { dg_acc[i][j] = 0.f; db_acc[i][j] = 0.f; if (!MEMEFF) bf[i][j] = 0.f; }
  }

  for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
    const int64_t row = g * RPB + wave / WPR;
    const bool row_ok = row < rows;
    float dy[VPL][EPV], y[VPL][EPV];
    // every load of the row first, from clamped addresses (see ln_fwd_kernel)
    const int64_t rowc = row_ok ? row : 0;
    float rs = rsigma[rowc], mean = 0.f;
    if constexpr (!MEMEFF) mean = mu[rowc];
    pack<TW, EPV> dzr[VPL];
    pack<TI, EPV> xr[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      const int cc = col < hidden ? col : 0;
      dzr[i] = load_raw<TW, EPV>(dz + rowc * hidden + cc);
      xr[i] = load_raw<TI, EPV>(x_or_z + rowc * hidden + cc);
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) { pin_raw(dzr[i]); pin_raw(xr[i]); }
    if (!row_ok) { rs = 0.f; mean = 0.f; }
    float sdy = 0.f, sdyy = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      if (row_ok && col < hidden) {
        float dzf[EPV], xf[EPV];
        unpack_raw<TW, EPV>(dzr[i], dzf);
        unpack_raw<TI, EPV>(xr[i], xf);
#pragma unroll
        for (int j = 0; j < EPV; ++j) {
          float yv;
          if constexpr (MEMEFF) yv = (xf[j] - bf[i][j]) / gf[i][j];
          else yv = rs * (xf[j] - mean);
          const float dyv = dzf[j] * gf[i][j];
          sdy += dyv;
          sdyy += dyv * yv;
          dy[i][j] = dyv;
          y[i][j] = yv;
          dg_acc[i][j] += dzf[j] * yv;
          db_acc[i][j] += dzf[j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < EPV; ++j) { dy[i][j] = 0.f; y[i][j] = 0.f; }
      }
    }
    row_sum2<WPR>(sdy, sdyy, smem, wave);
    const float mdy = sdy * rn, mdyy = sdyy * rn;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      if (row_ok && col < hidden) {
        float dxf[EPV];
#pragma unroll
        for (int j = 0; j < EPV; ++j) dxf[j] = rs * (dy[i][j] - (mdyy * y[i][j] + mdy));
        store_pack<TI, EPV>(dx + row * hidden + col, dxf);
      }
    }
  }

  // Fold the RPB row slots of the block (wavefronts that hold the same columns) in a fixed
  // order, then write the block's partial row.
  constexpr int SPAN = WPR * VPL * kWave * EPV;  // padded column span covered by the block
  if constexpr (RPB > 1) {
    const int slot = wave / WPR;
    __syncthreads();
    if (slot > 0) {
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int pc = ((sub * VPL + i) * kWave + lane) * EPV;
#pragma unroll
        for (int j = 0; j < EPV; ++j) {
          fold[((slot - 1) * 2 + 0) * SPAN + pc + j] = dg_acc[i][j];
          fold[((slot - 1) * 2 + 1) * SPAN + pc + j] = db_acc[i][j];
        }
      }
    }
    __syncthreads();
    if (slot == 0) {
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int pc = ((sub * VPL + i) * kWave + lane) * EPV;
#pragma unroll
        for (int s = 0; s < RPB - 1; ++s) {
#pragma unroll
          for (int j = 0; j < EPV; ++j) {
            dg_acc[i][j] += fold[(s * 2 + 0) * SPAN + pc + j];
            db_acc[i][j] += fold[(s * 2 + 1) * SPAN + pc + j];
          }
        }
      }
    }
  }
  if (wave / WPR == 0) {
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = ((sub * VPL + i) * kWave + lane) * EPV;
      if (col < hidden) {
        store_pack<float, EPV>(dgamma_part + static_cast<int64_t>(blockIdx.x) * hidden + col, dg_acc[i]);
        store_pack<float, EPV>(dbeta_part + static_cast<int64_t>(blockIdx.x) * hidden + col, db_acc[i]);
      }
    }
  }
}

// Generic backward: one block per row slot, scalar columns, three passes; partial sums are kept
// per thread for the columns c = threadIdx.x + k*LN_THREADS in the partial buffers themselves.
template <typename TI, typename TW, bool MEMEFF>
__global__ __launch_bounds__(LN_THREADS) void ln_bwd_generic_kernel(
    const TW* __restrict__ dz, const TI* __restrict__ x_or_z, const float* __restrict__ mu,
    const float* __restrict__ rsigma, const TW* __restrict__ gamma, const TW* __restrict__ beta,
    TI* __restrict__ dx, float* __restrict__ dgamma_part, float* __restrict__ dbeta_part,
    int64_t rows, int hidden) {
  __shared__ float smem[2 * LN_WAVES];
  const int wave = threadIdx.x / kWave;
  const float rn = 1.f / static_cast<float>(hidden);
  float* dgp = dgamma_part + static_cast<int64_t>(blockIdx.x) * hidden;
  float* dbp = dbeta_part + static_cast<int64_t>(blockIdx.x) * hidden;
  for (int c = threadIdx.x; c < hidden; c += LN_THREADS) { dgp[c] = 0.f; dbp[c] = 0.f; }
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const float rs = rsigma[row];
    const float mean = MEMEFF ? 0.f : mu[row];
    float sdy = 0.f, sdyy = 0.f;
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS) {
      const float gm = elem<TW>::to_float(gamma[c]);
      const float xv = elem<TI>::to_float(x_or_z[row * hidden + c]);
      const float yv = MEMEFF ? (xv - elem<TW>::to_float(beta[c])) / gm : rs * (xv - mean);
      const float dzv = elem<TW>::to_float(dz[row * hidden + c]);
      const float dyv = dzv * gm;
      sdy += dyv;
      sdyy += dyv * yv;
      dgp[c] += dzv * yv;  // same thread owns column c in every row: no race
      dbp[c] += dzv;
    }
    row_sum2<LN_WAVES>(sdy, sdyy, smem, wave);
    const float mdy = sdy * rn, mdyy = sdyy * rn;
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS) {
      const float gm = elem<TW>::to_float(gamma[c]);
      const float xv = elem<TI>::to_float(x_or_z[row * hidden + c]);
      const float yv = MEMEFF ? (xv - elem<TW>::to_float(beta[c])) / gm : rs * (xv - mean);
      const float dyv = elem<TW>::to_float(dz[row * hidden + c]) * gm;
      dx[row * hidden + c] = elem<TI>::from_float(rs * (dyv - (mdyy * yv + mdy)));
    }
  }
}

// Column sums of the [n_part, hidden] partials, in a fixed order. Block = FIN_CL column lanes
// (CPT columns each) x FIN_GR row groups; a thread walks rows gr, gr + FIN_GR, ... with several
// independent loads in flight, LDS folds the FIN_GR groups in order.
constexpr int FIN_CL = 32, FIN_GR = 32;
template <typename TW, int CPT>
__global__ __launch_bounds__(FIN_CL * FIN_GR) void ln_bwd_finalize_kernel(
    const float* __restrict__ dgamma_part, const float* __restrict__ dbeta_part,
    TW* __restrict__ dgamma, TW* __restrict__ dbeta, int n_part, int hidden) {
  __shared__ float red[FIN_GR][FIN_CL * CPT + 1];
  const float* src = blockIdx.y == 0 ? dgamma_part : dbeta_part;
  TW* dst = blockIdx.y == 0 ? dgamma : dbeta;
  const int cl = threadIdx.x % FIN_CL, gr = threadIdx.x / FIN_CL;
  const int col = (blockIdx.x * FIN_CL + cl) * CPT;
  float s[CPT];
#pragma unroll
  for (int j = 0; j < CPT; ++j) s[j] = 0.f;
  if (col < hidden) {
    // The kernel is a handful of blocks, so what it costs is global-load latency: 16 partial rows
    // are loaded before any of them is added (written as two loops on purpose: with the load and
    // the add in one loop body the compiler waits for each load in turn). Sum order unchanged.
    constexpr int BATCH = 16;
    int p = gr;
    for (; p + (BATCH - 1) * FIN_GR < n_part; p += BATCH * FIN_GR) {
      float v[BATCH][CPT];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) load_pack<float, CPT>(src + static_cast<int64_t>(p + u * FIN_GR) * hidden + col, v[u]);
      __builtin_amdgcn_sched_barrier(0);   // keep every load ahead of the first add
#pragma unroll
      for (int u = 0; u < BATCH; ++u)
#pragma unroll
        for (int j = 0; j < CPT; ++j) s[j] += v[u][j];
    }
    for (; p < n_part; p += FIN_GR) {
      float v[CPT];
      load_pack<float, CPT>(src + static_cast<int64_t>(p) * hidden + col, v);
#pragma unroll
      for (int j = 0; j < CPT; ++j) s[j] += v[j];
    }
  }
#pragma unroll
  for (int j = 0; j < CPT; ++j) red[gr][cl * CPT + j] = s[j];
  __syncthreads();
  for (int c = threadIdx.x; c < FIN_CL * CPT; c += FIN_CL * FIN_GR) {
    const int out_col = blockIdx.x * FIN_CL * CPT + c;
    if (out_col < hidden) {
      float t = 0.f;
#pragma unroll
      for (int k = 0; k < FIN_GR; ++k) t += red[k][c];
      dst[out_col] = elem<TW>::from_float(t);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Host-side shape planning.
// ---------------------------------------------------------------------------------------------
struct LnPlan {
  bool vectorised;
  int vpl, wpr;
};

template <typename TI>
LnPlan ln_plan(int64_t hidden, int max_vpl) {
  constexpr int EPV = ln_vec<TI>::EPV;
  LnPlan p{false, 0, 0};
  if (hidden % EPV != 0) return p;
  const int64_t vecs = hidden / EPV;
  for (int wpr = 1; wpr <= LN_WAVES; wpr *= 2) {
    for (int vpl = 1; vpl <= max_vpl; vpl *= 2) {
      if (static_cast<int64_t>(wpr) * vpl * kWave >= vecs) {
        p.vectorised = true; p.vpl = vpl; p.wpr = wpr;
        return p;
      }
    }
  }
  return p;
}

int ln_grid_limit() { return num_cus() * 8; }  // 8 blocks of 4 wavefronts per CU = full occupancy

template <typename TI, typename TW>
int ln_fwd_launch(const void* x, const void* gamma, const void* beta, void* z, float* mu,
                  float* rsigma, int64_t rows, int64_t hidden, float eps, hipStream_t st) {
  const bool al = aligned16(x) && aligned16(z) && aligned16(gamma) && aligned16(beta);
  LnPlan p = al ? ln_plan<TI>(hidden, 8) : LnPlan{false, 0, 0};
  auto X = static_cast<const TI*>(x);
  auto G = static_cast<const TW*>(gamma);
  auto B = static_cast<const TW*>(beta);
  auto Z = static_cast<TW*>(z);
  const int H = static_cast<int>(hidden);
  TraceScope trace("ln_fwd", st);
  if (!p.vectorised) {
    const int grid = static_cast<int>(std::min<int64_t>(rows, ln_grid_limit()));
    hipLaunchKernelGGL((ln_fwd_generic_kernel<TI, TW>), dim3(grid), dim3(LN_THREADS), 0, st, X, G, B,
                       Z, mu, rsigma, rows, H, eps);
    return 0;
  }
  const int rpb = LN_WAVES / p.wpr;
  const int64_t groups = (rows + rpb - 1) / rpb;
  const int grid = static_cast<int>(std::min<int64_t>(groups, ln_grid_limit()));
#define LN_FWD_CASE(V, W)                                                                       \
  if (p.vpl == V && p.wpr == W) {                                                               \
    hipLaunchKernelGGL((ln_fwd_kernel<TI, TW, V, W>), dim3(grid), dim3(LN_THREADS), 0, st, X, G, \
                       B, Z, mu, rsigma, rows, H, eps);                                         \
    return 0;                                                                                   \
  }
  LN_FWD_CASE(1, 1) LN_FWD_CASE(2, 1) LN_FWD_CASE(4, 1) LN_FWD_CASE(8, 1)
  LN_FWD_CASE(8, 2) LN_FWD_CASE(8, 4)
#undef LN_FWD_CASE
  return fail(NMTG_ERR_UNSUPPORTED, "ln_fwd: no kernel for plan vpl=%d wpr=%d", p.vpl, p.wpr);
}

constexpr int LN_BWD_MAX_VPL = 4;

// One partial row per block: few enough blocks that the partials stay a small fraction of the
// traffic, enough to keep every CU busy. Any n_part >= 1 is correct; this is the tuned choice.
int64_t ln_bwd_parts_for(int64_t rows) {
  const int64_t groups = (rows + LN_WAVES - 1) / LN_WAVES;
  const int64_t cap = static_cast<int64_t>(num_cus()) * 2;
  return std::max<int64_t>(1, std::min<int64_t>(groups, cap));
}

template <typename TI, typename TW>
int ln_bwd_launch(const void* dz, const void* x_or_z, const float* mu, const float* rsigma,
                  const void* gamma, const void* beta, void* dx, void* dgamma, void* dbeta,
                  float* dgp, float* dbp, int64_t n_part, int64_t rows, int64_t hidden, bool memeff,
                  hipStream_t st) {
  auto DZ = static_cast<const TW*>(dz);
  auto X = static_cast<const TI*>(x_or_z);
  auto G = static_cast<const TW*>(gamma);
  auto B = static_cast<const TW*>(beta);
  auto DX = static_cast<TI*>(dx);
  const int H = static_cast<int>(hidden);
  const bool al = aligned16(dz) && aligned16(x_or_z) && aligned16(dx) && aligned16(gamma) &&
                  (!memeff || aligned16(beta)) && aligned16(dgp) && aligned16(dbp);
  LnPlan p = ln_plan<TI>(hidden, LN_BWD_MAX_VPL);
  const int grid = static_cast<int>(n_part);
  bool done = false;
  {
  TraceScope trace("ln_bwd", st);
  if (p.vectorised && al) {
    constexpr int EPV = ln_vec<TI>::EPV;
    const int rpb = LN_WAVES / p.wpr;
    const size_t fold_bytes =
        rpb > 1 ? static_cast<size_t>(rpb - 1) * 2 * p.wpr * p.vpl * kWave * EPV * sizeof(float) : 0;
#define LN_BWD_CASE(V, W)                                                                          \
  if (!done && p.vpl == V && p.wpr == W) {                                                         \
    if (memeff)                                                                                    \
      hipLaunchKernelGGL((ln_bwd_kernel<TI, TW, V, W, true>), dim3(grid), dim3(LN_THREADS),        \
                         fold_bytes, st, DZ, X, mu, rsigma, G, B, DX, dgp, dbp, rows, H);          \
    else                                                                                           \
      hipLaunchKernelGGL((ln_bwd_kernel<TI, TW, V, W, false>), dim3(grid), dim3(LN_THREADS),       \
                         fold_bytes, st, DZ, X, mu, rsigma, G, B, DX, dgp, dbp, rows, H);          \
    done = true;                                                                                   \
  }
    LN_BWD_CASE(1, 1) LN_BWD_CASE(2, 1) LN_BWD_CASE(4, 1) LN_BWD_CASE(4, 2) LN_BWD_CASE(4, 4)
#undef LN_BWD_CASE
  }
  if (!done) {
    if (memeff)
      hipLaunchKernelGGL((ln_bwd_generic_kernel<TI, TW, true>), dim3(grid), dim3(LN_THREADS), 0, st,
                         DZ, X, mu, rsigma, G, B, DX, dgp, dbp, rows, H);
    else
      hipLaunchKernelGGL((ln_bwd_generic_kernel<TI, TW, false>), dim3(grid), dim3(LN_THREADS), 0, st,
                         DZ, X, mu, rsigma, G, B, DX, dgp, dbp, rows, H);
  }
  }
  TraceScope trace("ln_bwd_finalize", st);
  if (H % 4 == 0 && aligned16(dgp) && aligned16(dbp)) {
    dim3 fgrid((H + FIN_CL * 4 - 1) / (FIN_CL * 4), 2);
    hipLaunchKernelGGL((ln_bwd_finalize_kernel<TW, 4>), fgrid, dim3(FIN_CL * FIN_GR), 0, st, dgp, dbp,
                       static_cast<TW*>(dgamma), static_cast<TW*>(dbeta), static_cast<int>(n_part), H);
  } else {
    dim3 fgrid((H + FIN_CL - 1) / FIN_CL, 2);
    hipLaunchKernelGGL((ln_bwd_finalize_kernel<TW, 1>), fgrid, dim3(FIN_CL * FIN_GR), 0, st, dgp, dbp,
                       static_cast<TW*>(dgamma), static_cast<TW*>(dbeta), static_cast<int>(n_part), H);
  }
  return 0;
}

// in/weight dtype pairs the reference registers (ln_fwd_cuda_kernel.cu:73-233): same type, or
// 16-bit activations with fp32 weights.
bool ln_pair_ok(int in_dtype, int w_dtype) {
  return in_dtype == w_dtype || (w_dtype == NMTG_F32 && (in_dtype == NMTG_F16 || in_dtype == NMTG_BF16));
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_ln_fwd(const void* x, const void* gamma, const void* beta, void* z, float* mu,
                           float* rsigma, int64_t rows, int64_t hidden, float eps, int in_dtype,
                           int w_dtype, void* stream) {
  NMTG_REQUIRE(rows >= 0 && hidden > 0 && hidden <= (1 << 30), "ln_fwd: bad shape rows=%lld hidden=%lld",
               (long long)rows, (long long)hidden);
  NMTG_REQUIRE(rows == 0 || (x && gamma && beta && z && mu && rsigma), "ln_fwd: null pointer argument");
  NMTG_REQUIRE(eps >= 0.f, "ln_fwd: epsilon must be >= 0");
  NMTG_REQUIRE(ln_pair_ok(in_dtype, w_dtype), "ln_fwd: unsupported dtype pair in=%d weight=%d", in_dtype, w_dtype);
  if (rows == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc = 0;
  if (in_dtype == w_dtype) {
    NMTG_DISPATCH_DTYPE(in_dtype, T, rc = (ln_fwd_launch<T, T>(x, gamma, beta, z, mu, rsigma, rows, hidden, eps, st)));
  } else if (in_dtype == NMTG_F16) {
    rc = ln_fwd_launch<f16_t, float>(x, gamma, beta, z, mu, rsigma, rows, hidden, eps, st);
  } else {
    rc = ln_fwd_launch<bf16_t, float>(x, gamma, beta, z, mu, rsigma, rows, hidden, eps, st);
  }
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("ln_fwd");
  return 0;
}

extern "C" int64_t nmtg_ln_bwd_parts(int64_t rows, int64_t hidden) {
  if (rows <= 0 || hidden <= 0) return 1;
  return ln_bwd_parts_for(rows);
}

extern "C" int nmtg_ln_bwd(const void* dz, const void* x_or_z, const float* mu, const float* rsigma,
                           const void* gamma, const void* beta, void* dx, void* dgamma, void* dbeta,
                           float* dgamma_part, float* dbeta_part, int64_t n_part, int64_t rows,
                           int64_t hidden, int memory_efficient, int in_dtype, int w_dtype,
                           void* stream) {
  NMTG_REQUIRE(gamma && dgamma && dbeta && dgamma_part && dbeta_part, "ln_bwd: null pointer argument");
  NMTG_REQUIRE(rows == 0 || (dz && x_or_z && rsigma && dx), "ln_bwd: null pointer argument");
  NMTG_REQUIRE(rows == 0 || (memory_efficient ? beta != nullptr : mu != nullptr),
               "ln_bwd: %s is required", memory_efficient ? "beta (memory_efficient)" : "mu");
  NMTG_REQUIRE(rows >= 0 && hidden > 0 && hidden <= (1 << 30), "ln_bwd: bad shape rows=%lld hidden=%lld",
               (long long)rows, (long long)hidden);
  NMTG_REQUIRE(ln_pair_ok(in_dtype, w_dtype), "ln_bwd: unsupported dtype pair in=%d weight=%d", in_dtype, w_dtype);
  NMTG_REQUIRE(n_part >= 1 && n_part <= (1 << 20), "ln_bwd: n_part=%lld out of range", (long long)n_part);
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc = 0;
  const bool me = memory_efficient != 0;
  if (in_dtype == w_dtype) {
    NMTG_DISPATCH_DTYPE(in_dtype, T, rc = (ln_bwd_launch<T, T>(dz, x_or_z, mu, rsigma, gamma, beta, dx, dgamma, dbeta,
                                                               dgamma_part, dbeta_part, n_part, rows, hidden, me, st)));
  } else if (in_dtype == NMTG_F16) {
    rc = ln_bwd_launch<f16_t, float>(dz, x_or_z, mu, rsigma, gamma, beta, dx, dgamma, dbeta, dgamma_part,
                                     dbeta_part, n_part, rows, hidden, me, st);
  } else {
    rc = ln_bwd_launch<bf16_t, float>(dz, x_or_z, mu, rsigma, gamma, beta, dx, dgamma, dbeta, dgamma_part,
                                      dbeta_part, n_part, rows, hidden, me, st);
  }
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("ln_bwd");
  return 0;
}
