// C[m][n] = alpha * sum_k X[m][k] W[n][k] (+ bias[n]) for at most 32 rows m: the projections of a decoding step
// (one new position of a few dozen hypotheses against a [1024 x 1024] weight), which the reference runs as cuBLASLt
// calls like any other linear layer (onmt/modules/extensions/mlp_blaslt/linear.cpp:142-144).
//
// With so few rows the product is a read of W: 2 MB of weight against 64 KB of activations, and a 128 x 128 output
// tile leaves all but eight compute units idle while each of those walks the whole reduction. Here every wavefront
// owns one output column: its 64 lanes read the column's weight row with 16-byte loads, 16 elements per lane and
// 1024-element chunk of k, and multiply them with the same k-elements of all 32 activation rows, which the block
// stages in LDS once per chunk (64 KB); 32 wavefront reductions then leave row m's sum in lane m. A block of four
// wavefronts covers four columns, so a [1024 x 1024] weight spreads over 256 blocks.
#include "gemm.cuh"

namespace nmtg {
namespace {

constexpr int SK_ROWS = 32, SK_CHUNK = 1024, SK_THREADS = 256;

template <typename T>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(const GemmArgs g) {
  extern __shared__ __align__(16) uint8_t lds_raw[];
  T* xs = reinterpret_cast<T*>(lds_raw);                 // [32][SK_CHUNK]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = static_cast<int>(blockIdx.x) * (SK_THREADS / 64) + wave;
  const T* X = static_cast<const T*>(g.A);
  const T* W = static_cast<const T*>(g.B);
  float acc[SK_ROWS];
#pragma unroll
  for (int m = 0; m < SK_ROWS; ++m) acc[m] = 0.f;

  for (int k0 = 0; k0 < g.K; k0 += SK_CHUNK) {
    const int kc = min(SK_CHUNK, g.K - k0);              // a multiple of 8
    // the column's weights of this chunk: lane l holds k0 + 16 l .. + 15 (two 16-byte loads), zeros past the end
    pack<T, 8> wraw[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int k = 16 * lane + 8 * u;
      wraw[u] = pack<T, 8>{};
      if (n < g.N && k < kc) wraw[u] = load_raw<T, 8>(W + static_cast<int64_t>(n) * g.ldb + k0 + k);
    }
    // the chunk of X: all loads in flight before the first LDS store (16 per lane)
    constexpr int PER = SK_ROWS * (SK_CHUNK / 8) / SK_THREADS;
    pack<T, 8> xraw[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      // every block needs the same rows: each starts at another one, so that at any moment the blocks ask the L2 for
      // different lines instead of all for the same
      const int id = (tid + SK_THREADS * (i + static_cast<int>(blockIdx.x))) % (SK_ROWS * (SK_CHUNK / 8));
      const int m = id / (SK_CHUNK / 8), k = 8 * (id % (SK_CHUNK / 8));
      xraw[i] = pack<T, 8>{};
      if (m < g.M && k < kc) xraw[i] = load_raw<T, 8>(X + static_cast<int64_t>(m) * g.lda + k0 + k);
    }
    if (k0 > 0) __syncthreads();                         // the previous chunk has been consumed
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int id = (tid + SK_THREADS * (i + static_cast<int>(blockIdx.x))) % (SK_ROWS * (SK_CHUNK / 8));
      *reinterpret_cast<pack<T, 8>*>(xs + (id / (SK_CHUNK / 8)) * SK_CHUNK + 8 * (id % (SK_CHUNK / 8))) = xraw[i];
    }
    __syncthreads();
    uint32_t wv[8];
    __builtin_memcpy(wv, &wraw[0], 16);
    __builtin_memcpy(wv + 4, &wraw[1], 16);
#pragma unroll
    for (int m = 0; m < SK_ROWS; ++m) {
      const uint4 x0 = *reinterpret_cast<const uint4*>(xs + m * SK_CHUNK + 16 * lane);
      const uint4 x1 = *reinterpret_cast<const uint4*>(xs + m * SK_CHUNK + 16 * lane + 8);
      const uint32_t xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
      float s = acc[m];
#pragma unroll
      for (int e = 0; e < 8; ++e) s = dot2<T>(xv[e], wv[e], s);
      acc[m] = s;
    }
  }
  // row m's sum over the wavefront ends in lane m
  float mine = 0.f;
#pragma unroll
  for (int m = 0; m < SK_ROWS; ++m) {
    const float s = wave_sum(acc[m]);
    if (lane == m) mine = s;
  }
  if (lane < g.M && n < g.N) {
    float v = mine * g.alpha;
    if (g.bias != nullptr) v += elem<T>::to_float(static_cast<const T*>(g.bias)[n]);
    static_cast<T*>(g.C)[static_cast<int64_t>(lane) * g.ldc + n] = elem<T>::from_float(v);
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
  const unsigned grid = static_cast<unsigned>((a.N + SK_THREADS / 64 - 1) / (SK_THREADS / 64));
  const int lds = SK_ROWS * SK_CHUNK * 2;
  TraceScope trace("gemm_nt_skinny", st);
  if (dtype == NMTG_F16) hipLaunchKernelGGL((gemm_skinny_kernel<f16_t>), dim3(grid), dim3(SK_THREADS), lds, st, a);
  else hipLaunchKernelGGL((gemm_skinny_kernel<bf16_t>), dim3(grid), dim3(SK_THREADS), lds, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "gemm: launch failed: %s", hipGetErrorString(e));
  return 0;
}

}  // namespace nmtg
