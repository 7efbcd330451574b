// C[m][n] = alpha * sum_k X[m][k] W[n][k] (+ bias[n]) for at most 32 rows m: the projections of a decoding step
// (one new position of a few dozen hypotheses against a [1024 x 1024] weight), which the reference runs as cuBLASLt
// calls like any other linear layer (onmt/modules/extensions/mlp_blaslt/linear.cpp:142-144).
//
// With so few rows the product is a read of W: 2 MB of weight against 64 KB of activations, and a 128 x 128 output
// tile leaves all but eight compute units idle while each of those walks the whole reduction. What counts is the
// latency of one block, so the reduction is spread over the wavefronts of a block instead: a block owns 32 output
// columns and all (at most 32) rows, its eight wavefronts each take an eighth of k, load their slices of X and W
// straight into matrix-core operand layout (a lane's 16 bytes of its row: no LDS staging, every load of a 128-k chunk in
// flight at once), run v_mfma_f32_32x32x16 over them, and leave their 32 x 32 partial sums in LDS, where the block adds
// the eight of them up in a fixed order. A [1024 x 1024] weight is 32 blocks of one load latency each.
#include "gemm.hip.h"

namespace nmtg {
namespace {

constexpr int SK_ROWS = 32, SK_COLS = 32, SK_WAVES = 8, SK_THREADS = 64 * SK_WAVES, SK_CHUNK = 128;

template <typename T>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(const GemmArgs g) {
  __shared__ float part[SK_WAVES][16][64];               // partial tiles in accumulator layout
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = static_cast<int>(blockIdx.x) * SK_COLS;
  const T* X = static_cast<const T*>(g.A);
  const T* W = static_cast<const T*>(g.B);
  // this wavefront's share of k: whole 16-k steps, dealt out in chunks of 128 so that the loads in flight stay bounded
  const int steps = (g.K + 15) / 16, per = (steps + SK_WAVES - 1) / SK_WAVES;
  const int k_begin = wave * per * 16, k_end = min(g.K, (wave + 1) * per * 16);
  const int m = lane & 31, n = n0 + (lane & 31);
  const T* xrow = X + static_cast<int64_t>(m) * g.lda + 8 * half;
  const T* wrow = W + static_cast<int64_t>(n) * g.ldb + 8 * half;
  acc16_t acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  for (int k0 = k_begin; k0 < k_end; k0 += SK_CHUNK) {
    uint4 xf[SK_CHUNK / 16], wf[SK_CHUNK / 16];
#pragma unroll
    for (int s = 0; s < SK_CHUNK / 16; ++s) {
      const int k = k0 + 16 * s + 8 * half;               // K is a multiple of 8: a lane's 8 elements are all in or all out
      const bool in = k < k_end;
      xf[s] = in && m < g.M ? *reinterpret_cast<const uint4*>(xrow + k0 + 16 * s) : make_uint4(0, 0, 0, 0);
      wf[s] = in && n < g.N ? *reinterpret_cast<const uint4*>(wrow + k0 + 16 * s) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int s = 0; s < SK_CHUNK / 16; ++s) mfma<T>::run(xf[s], wf[s], acc);   // acc[r], lane (j, half): row 8 (r / 4) + 4 half + r % 4, column j
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) part[wave][r][lane] = acc[r];
  __syncthreads();
  // 1024 outputs, two per thread; the eight partial sums are added in wavefront order
  for (int o = tid; o < 16 * 64; o += SK_THREADS) {
    const int r = o >> 6, l = o & 63;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < SK_WAVES; ++w) v += part[w][r][l];
    const int row = 8 * (r / 4) + 4 * (l >> 5) + r % 4, col = n0 + (l & 31);
    if (row < g.M && col < g.N) {
      v *= g.alpha;
      if (g.bias != nullptr) v += elem<T>::to_float(static_cast<const T*>(g.bias)[col]);
      static_cast<T*>(g.C)[static_cast<int64_t>(row) * g.ldc + col] = elem<T>::from_float(v);
    }
  }
}

}  // namespace

// Eligibility: row-major X and W (the NT layout), plain epilogue, one batch, 16-byte aligned rows. NMTG_GEMM_SKINNY=0
// sends these calls to the tiled kernels instead.
bool gemm_skinny_ok(int dtype, int layout, int epi, const GemmArgs& a) {
  if (switched_off("NMTG_GEMM_SKINNY")) return false;
  return (dtype == NMTG_F16 || dtype == NMTG_BF16) && layout == LAYOUT_NT && epi == EPI_PLAIN && a.batch == 1 && a.M >= 1 &&
         a.M <= SK_ROWS && a.N >= 64 && a.K >= 8 && a.K % 8 == 0 && a.lda % 8 == 0 && a.ldb % 8 == 0 && aligned16(a.A) &&
         aligned16(a.B);
}

int gemm_skinny_run(int dtype, const GemmArgs& a, hipStream_t st) {
  const unsigned grid = static_cast<unsigned>((a.N + SK_COLS - 1) / SK_COLS);
  TraceScope trace("gemm_nt_skinny", st);
  if (dtype == NMTG_F16) hipLaunchKernelGGL((gemm_skinny_kernel<f16_t>), dim3(grid), dim3(SK_THREADS), 0, st, a);
  else hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t>), dim3(grid), dim3(SK_THREADS), 0, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "gemm: launch failed: %s", hipGetErrorString(e));
  return 0;
}

}  // namespace nmtg
