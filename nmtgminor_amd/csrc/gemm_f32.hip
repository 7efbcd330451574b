// fp32 GEMM on the fp32 matrix cores (v_mfma_f32_32x32x2_f32) with the bias / activation / dropout epilogues of the
// fused MLP: the data type the reference's own MLP tests run in (onmt/modules/mlp/test_mlp_gelu.py:229-307; its
// extension dispatches AT_DISPATCH_FLOATING_TYPES_AND_HALF, onmt/modules/extensions/mlp/mlp_gelu.cpp:104).
//
// One kernel shape: a block of four wavefronts owns a 128 x 128 tile of C, each wavefront 64 x 64 of it as 2 x 2 MFMA
// tiles; K is walked in steps of 16 through two LDS buffers holding the operands k-major ([16 k][128 rows], rows padded
// to 132 floats so that the two halves of a wavefront, which read rows of k and k + 1, hit different banks); the next
// step's global loads are in flight in registers while the current step multiplies. Operands of either orientation
// are read with 16-byte loads when every pointer, pitch and batch stride allows it, element by element (bounds-checked)
// otherwise and at ragged edges. As in the 16-bit kernels the MFMA takes the B tile first, so a lane holds four
// consecutive n of one row m and stores them as one 16-byte vector.
//
// fp32 is the reference's checking precision, not its training precision: this kernel is written to be exact (fp32
// products and sums in the matrix core, no re-association across blocks: no split-K) and simple, not to reach the fp32
// MFMA roof.
#include "gemm.hip.h"

namespace nmtg {
namespace {

constexpr int F32_BM = 128, F32_BN = 128, F32_BK = 16, F32_PITCH = 132, F32_THREADS = 256;

// Four consecutive elements of the contiguous dimension starting at p; element e is valid iff e < nvalid (and the row is).
__device__ __forceinline__ float4 load4_f32(const float* __restrict__ p, int nvalid, bool vec) {
  if (nvalid >= 4 && vec) return *reinterpret_cast<const float4*>(p);
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (nvalid > 0) v.x = p[0];
  if (nvalid > 1) v.y = p[1];
  if (nvalid > 2) v.z = p[2];
  if (nvalid > 3) v.w = p[3];
  return v;
}

// One operand tile [128 rows][16 k] on its way global -> registers -> LDS (k-major).
template <bool KC>
struct StageF32 {
  float4 v[2];
  // base: first element of the operand for this batch; rows r0 .. r0+127 of `rows` rows, k0 .. k0+15 of K
  __device__ __forceinline__ void load(const float* __restrict__ base, int64_t ld, int rows, int r0, int K, int k0, bool vec) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = static_cast<int>(threadIdx.x) + F32_THREADS * i;
      if constexpr (KC) {
        const int row = r0 + id / 4, k = k0 + 4 * (id % 4);
        v[i] = load4_f32(base + static_cast<int64_t>(row < rows ? row : 0) * ld + (k < K ? k : 0), row < rows ? K - k : 0, vec);
      } else {
        const int k = k0 + id / 32, row = r0 + 4 * (id % 32);
        v[i] = load4_f32(base + static_cast<int64_t>(k < K ? k : 0) * ld + (row < rows ? row : 0), k < K ? rows - row : 0, vec);
      }
    }
  }
  __device__ __forceinline__ void store(float (*s)[F32_PITCH]) const {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int id = static_cast<int>(threadIdx.x) + F32_THREADS * i;
      if constexpr (KC) {
        const int row = id / 4, k = 4 * (id % 4);
        s[k + 0][row] = v[i].x;
        s[k + 1][row] = v[i].y;
        s[k + 2][row] = v[i].z;
        s[k + 3][row] = v[i].w;
      } else {
        *reinterpret_cast<float4*>(&s[id / 32][4 * (id % 32)]) = v[i];
      }
    }
  }
};

template <bool A_KC, bool B_KC, int EPI>
__global__ __launch_bounds__(F32_THREADS) void gemm_f32_kernel(const GemmArgs g) {
  __shared__ __align__(16) float sA[2][F32_BK][F32_PITCH];
  __shared__ __align__(16) float sB[2][F32_BK][F32_PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5;
  const int tile_m = static_cast<int>(blockIdx.x) / g.n_tiles, tile_n = static_cast<int>(blockIdx.x) % g.n_tiles, bz = blockIdx.y;
  const int m0 = tile_m * F32_BM, n0 = tile_n * F32_BN;
  const int wm0 = (wave / 2) * 64, wn0 = (wave % 2) * 64;
  const float* A = static_cast<const float*>(g.A) + static_cast<int64_t>(bz) * g.sA;
  const float* B = static_cast<const float*>(g.B) + static_cast<int64_t>(bz) * g.sB;
  const bool vec = g.vec >= 4;

  acc16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  StageF32<A_KC> sa;
  StageF32<B_KC> sb;
  const int steps = (g.K + F32_BK - 1) / F32_BK;
  if (steps > 0) {
    sa.load(A, g.lda, g.M, m0, g.K, 0, vec);
    sb.load(B, g.ldb, g.N, n0, g.K, 0, vec);
    sa.store(sA[0]);
    sb.store(sB[0]);
  }
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) {
      sa.load(A, g.lda, g.M, m0, g.K, (s + 1) * F32_BK, vec);
      sb.load(B, g.ldb, g.N, n0, g.K, (s + 1) * F32_BK, vec);
    }
#pragma unroll
    for (int kk = 0; kk < F32_BK; kk += 2) {
      float fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = sA[buf][kk + half][wm0 + 32 * i + (lane & 31)];
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = sB[buf][kk + half][wn0 + 32 * j + (lane & 31)];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (s + 1 < steps) {
      sa.store(sA[buf ^ 1]);
      sb.store(sB[buf ^ 1]);
    }
    __syncthreads();
  }

  // ---- epilogue: lane (l) register r of tile (i, j) holds C[m][n], m = m0 + wm0 + 32 i + (l & 31),
  //      n = n0 + wn0 + 32 j + 8 (r / 4) + 4 (l >> 5) + r % 4 ----
  float* C = static_cast<float*>(g.C) + static_cast<int64_t>(bz) * g.sC;
  float* AUX = g.aux_out ? static_cast<float*>(g.aux_out) + static_cast<int64_t>(bz) * g.sC : nullptr;
  const float* bias = static_cast<const float*>(g.bias);
  const float* HIN = static_cast<const float*>(g.aux_in);
  auto store4 = [&](float* base, int m, int n, const float (&v)[4]) {
    float* p = base + static_cast<int64_t>(m) * g.ldc + n;
    if (vec && n + 3 < g.N) {
      *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < g.N) p[e] = v[e];
    }
  };
  float csum[2][4][4];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) csum[j][q][e] = 0.f;

  auto body = [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = m0 + wm0 + 32 * i + (lane & 31);
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn0 + 32 * j + 8 * q + 4 * half;
          if (m >= g.M || n >= g.N) continue;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = acc[i][j][4 * q + e] * g.alpha;
            if (EPI != EPI_ACT_BWD && bias != nullptr) v[e] += bias[min(n + e, g.N - 1)];
          }
          if constexpr (EPI == EPI_PLAIN) {
            store4(C, m, n, v);
          } else if constexpr (EPI == EPI_ACT_FWD) {
            if (AUX != nullptr) store4(AUX, m, n, v);
            float a[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = act_apply<ACT>(v[e], nullptr);
            if (g.dmask != nullptr) {
              uint8_t keep[4];
              const uint64_t first = static_cast<uint64_t>(m) * g.N + n;
              uint8_t* mk = const_cast<uint8_t*>(g.dmask) + first;
              if (g.rng) {
                if ((g.N & 3) == 0) {
                  philox_keep<4>(Philox(g.seed), first, g.offset, g.keep_p, keep);
                } else {
#pragma unroll
                  for (int e = 0; e < 4; ++e) {
                    uint8_t one[1];
                    philox_keep<1>(Philox(g.seed), first + e, g.offset, g.keep_p, one);
                    keep[e] = one[0];
                  }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  if (n + e < g.N) mk[e] = keep[e];
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) keep[e] = n + e < g.N ? mk[e] : 0;
              }
#pragma unroll
              for (int e = 0; e < 4; ++e) a[e] *= static_cast<float>(keep[e]) * g.dscale;
            }
            store4(C, m, n, a);
          } else {   // EPI_ACT_BWD
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const bool in = n + e < g.N;
              const float h = in ? HIN[static_cast<int64_t>(m) * g.ld_aux + n + e] : 0.f;
              const float keep = (g.dmask != nullptr && in) ? static_cast<float>(g.dmask[static_cast<int64_t>(m) * g.N + n + e]) : 1.f;
              v[e] *= act_grad<ACT>(h, nullptr) * (keep * g.dscale);
              if (in) csum[j][q][e] += v[e];
            }
            store4(C, m, n, v);
          }
        }
    }
  };
  if constexpr (EPI == EPI_PLAIN) body(std::integral_constant<int, NMTG_ACT_NONE>{});
  else dispatch_act<false>(g.act, 0, body);

  if constexpr (EPI == EPI_ACT_BWD) {
    if (g.colsum_part != nullptr) {
      // column sums over the tile's 128 rows: across the 32 rows of a half-wavefront by lane exchange, then across the
      // two wavefronts that share the columns through LDS (the operand buffers are free now)
      float* red = &sA[0][0][0];   // [2 row halves of the tile][128 columns]
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float s = csum[j][q][e];
#pragma unroll
            for (int d = 1; d < 32; d <<= 1) s += __shfl_xor(s, d);
            if ((lane & 31) == 0) red[(wave / 2) * F32_BN + wn0 + 32 * j + 8 * q + 4 * half + e] = s;
          }
      __syncthreads();
      if (tid < F32_BN && n0 + tid < g.N)
        g.colsum_part[static_cast<int64_t>(tile_m) * g.N + n0 + tid] = red[tid] + red[F32_BN + tid];
    }
  }
}

template <int EPI>
void launch_f32(int layout, const GemmArgs& a, hipStream_t st) {
  const dim3 grid(static_cast<unsigned>(a.m_tiles * a.n_tiles), static_cast<unsigned>(a.batch));
  if (layout == LAYOUT_NT) hipLaunchKernelGGL((gemm_f32_kernel<true, true, EPI>), grid, dim3(F32_THREADS), 0, st, a);
  else if (layout == LAYOUT_NN) hipLaunchKernelGGL((gemm_f32_kernel<true, false, EPI>), grid, dim3(F32_THREADS), 0, st, a);
  else hipLaunchKernelGGL((gemm_f32_kernel<false, false, EPI>), grid, dim3(F32_THREADS), 0, st, a);
}

}  // namespace

// The fp32 branch of gemm_run: same arguments, EPI_PLAIN / EPI_ACT_FWD / EPI_ACT_BWD, never splits K.
int gemm_f32_run(int layout, int epi, GemmArgs a, hipStream_t st, int* m_tiles_out, GemmArgs* planned_out) {
  if (epi != EPI_PLAIN && epi != EPI_ACT_FWD && epi != EPI_ACT_BWD)
    return fail(NMTG_ERR_UNSUPPORTED, "gemm: fp32 has no kernel for epilogue %d (plain, activation forward / backward are built)", epi);
  auto vec4 = [&](const void* p, int64_t ld, int64_t stride) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0 && ld % 4 == 0 && (a.batch <= 1 || stride % 4 == 0);
  };
  bool wide = vec4(a.A, a.lda, a.sA) && vec4(a.B, a.ldb, a.sB) && vec4(a.C, a.ldc, a.sC);
  if (a.aux_out) wide = wide && vec4(a.aux_out, a.ldc, a.sC);
  a.vec = wide ? 4 : 1;
  a.splits = 1;
  a.k_per_split = a.K;
  a.ring = a.act_lut = a.defer_reduce = a.riders_taken = 0;
  a.m_tiles = (a.M + F32_BM - 1) / F32_BM;
  a.n_tiles = (a.N + F32_BN - 1) / F32_BN;
  a.tile_used = -1;
  if (m_tiles_out) *m_tiles_out = a.m_tiles;
  if (static_cast<int64_t>(a.m_tiles) * a.n_tiles > 0x7fffffff || a.batch > 65535)
    return fail(NMTG_ERR_UNSUPPORTED, "gemm: grid too large (tiles %d x %d, batch %d)", a.m_tiles, a.n_tiles, a.batch);
  if (planned_out) *planned_out = a;
  TraceScope trace(epi == EPI_PLAIN ? "gemm_f32_plain" : epi == EPI_ACT_FWD ? "gemm_f32_act_fwd" : "gemm_f32_act_bwd", st);
  if (epi == EPI_PLAIN) launch_f32<EPI_PLAIN>(layout, a, st);
  else if (epi == EPI_ACT_FWD) launch_f32<EPI_ACT_FWD>(layout, a, st);
  else launch_f32<EPI_ACT_BWD>(layout, a, st);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "gemm: launch failed: %s", hipGetErrorString(e));
  return 0;
}

}  // namespace nmtg
