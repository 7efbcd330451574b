// Small fixed-order reduction kernels that follow a GEMM: the sum over split-K partials and the column sums behind
// every bias gradient. They are latency-bound (a few blocks, short dependent chains), so each keeps a batch of loads
// in flight before the first add. Hosts: reduce.hip (column sums), gemm_inst.hip.h (split-K).
#pragma once
#include "common.hip.h"
#include <type_traits>

namespace nmtg {

// Sums the split-K partials (in the accumulator layout the GEMM kernels' split-K epilogue writes, gemm.hip.h), scales, converts to T and
// writes row-major C; fixed summation order.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
__device__ __forceinline__ void splitk_reduce_slot(int64_t idx, const float* __restrict__ ws, T* __restrict__ C, int64_t ldc,
                                                   int M, int N, int m_tiles, int n_tiles, int batch, int64_t sC, int splits,
                                                   float alpha, int c_vec) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int PER_BLK = NW * TM * TN * 4 * 64;  // float4 slots per tile
  const int64_t total = static_cast<int64_t>(batch) * m_tiles * n_tiles * PER_BLK;
  if (idx >= total) return;
  const int lane = idx & 63;
  int64_t t = idx >> 6;
  const int q = t & 3; t >>= 2;
  const int j = t % TN; t /= TN;
  const int i = t % TM; t /= TM;
  const int wave = t % NW; t /= NW;
  const int tile = t % (m_tiles * n_tiles);
  const int bz = t / (m_tiles * n_tiles);
  const int tile_m = tile / n_tiles, tile_n = tile % n_tiles;
  const int m = tile_m * BM + (wave / WAVES_N) * WTM + i * 32 + (lane & 31);
  const int n = tile_n * BN + (wave % WAVES_N) * WTN + j * 32 + q * 8 + (lane >> 5) * 4;
  if (m >= M || n >= N) return;
  const int64_t per_split = static_cast<int64_t>(batch) * m_tiles * n_tiles * PER_BLK;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  const float4* w = reinterpret_cast<const float4*>(ws) + idx;
  int sp = 0;
  for (; sp + 4 <= splits; sp += 4) {   // four partials in flight, summed in split order
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = w[(sp + u) * per_split];
#pragma unroll
    for (int u = 0; u < 4; ++u) { s.x += v[u].x; s.y += v[u].y; s.z += v[u].z; s.w += v[u].w; }
  }
  for (; sp < splits; ++sp) {
    const float4 v = w[sp * per_split];
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  const float v[4] = {s.x * alpha, s.y * alpha, s.z * alpha, s.w * alpha};
  T* dst = C + static_cast<int64_t>(bz) * sC + static_cast<int64_t>(m) * ldc + n;
  if (n + 4 <= N && c_vec >= 4) store_pack<T, 4>(dst, v);
  else for (int e = 0; e < 4 && n + e < N; ++e) dst[e] = elem<T>::from_float(v[e]);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, T* __restrict__ C, int64_t ldc,
                                                            int M, int N, int m_tiles, int n_tiles, int batch,
                                                            int64_t sC, int splits, float alpha, int c_vec) {
  splitk_reduce_slot<T, BM, BN, WAVES_M, WAVES_N>(static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, ws, C, ldc, M, N, m_tiles,
                                                  n_tiles, batch, sC, splits, alpha, c_vec);
}

// Column sums of a row-major [M, N] matrix: partial[mb][n] over row blocks (fp32), fixed order.
// Block = 32 column lanes (8 columns each = one 16-byte load for 16-bit T) x 8 row lanes.
template <typename T, bool VEC>
__device__ __forceinline__ void colsum_partial_block(int bx, int by, const T* __restrict__ X, int64_t ld, int M, int N,
                                                     int rows_per_block, float* __restrict__ part, float* red_lds) {
  constexpr int CPT = VEC ? 8 : 1;
  float (*red)[32 * CPT + 1] = reinterpret_cast<float (*)[32 * CPT + 1]>(red_lds);   // [8][32 * CPT + 1] floats of LDS
  const int cl = threadIdx.x & 31, rl = threadIdx.x >> 5;
  const int n = (bx * 32 + cl) * CPT;
  const int r0 = by * rows_per_block;
  const int r1 = min(M, r0 + rows_per_block);
  float s[CPT];
#pragma unroll
  for (int j = 0; j < CPT; ++j) s[j] = 0.f;
  if (n < N) {
    // Latency-bound (few blocks, short rows): 16 (then 8) rows are loaded before any is added (two loops on
    // purpose, see ln_bwd_finalize_kernel); the sum order is that of the rows.
    int r = r0 + rl;
    auto batched = [&](auto batch_tag) {
      constexpr int BATCH = decltype(batch_tag)::value;
      for (; r + (BATCH - 1) * 8 < r1; r += BATCH * 8) {
        // raw words first, conversion only in the adding loop (a conversion is a use of the load)
        constexpr int NV = (CPT * sizeof(T)) / 16;   // 16-byte vectors per access; 0 in the scalar form
        if constexpr (NV > 0) {
          uint4 raw[BATCH][NV];
#pragma unroll
          for (int u = 0; u < BATCH; ++u)
#pragma unroll
            for (int i = 0; i < NV; ++i)
              raw[u][i] = reinterpret_cast<const uint4*>(X + static_cast<int64_t>(r + u * 8) * ld + n)[i];
          __builtin_amdgcn_sched_barrier(0);   // keep every load ahead of the first add
#pragma unroll
          for (int u = 0; u < BATCH; ++u) {
            const T* e = reinterpret_cast<const T*>(raw[u]);
#pragma unroll
            for (int j = 0; j < CPT; ++j) s[j] += elem<T>::to_float(e[j]);
          }
        } else {
          T raw[BATCH];
#pragma unroll
          for (int u = 0; u < BATCH; ++u) raw[u] = X[static_cast<int64_t>(r + u * 8) * ld + n];
#pragma unroll
          for (int u = 0; u < BATCH; ++u) s[0] += elem<T>::to_float(raw[u]);
        }
      }
    };
    batched(std::integral_constant<int, 16>{});
    batched(std::integral_constant<int, 8>{});
    for (; r < r1; r += 8) {
      float v[CPT];
      load_pack<T, CPT>(X + static_cast<int64_t>(r) * ld + n, v);
#pragma unroll
      for (int j = 0; j < CPT; ++j) s[j] += v[j];
    }
  }
#pragma unroll
  for (int j = 0; j < CPT; ++j) red[rl][cl * CPT + j] = s[j];
  __syncthreads();
  for (int c = threadIdx.x; c < 32 * CPT; c += 256) {
    const int col = bx * 32 * CPT + c;
    if (col < N) {
      float t = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) t += red[k][c];
      part[static_cast<int64_t>(by) * N + col] = t;
    }
  }
  __syncthreads();   // a caller that runs several of these blocks one after the other reuses `red`
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void colsum_partial_kernel(const T* __restrict__ X, int64_t ld, int M, int N,
                                                             int rows_per_block, float* __restrict__ part) {
  __shared__ float red[8 * (32 * (VEC ? 8 : 1) + 1)];
  colsum_partial_block<T, VEC>(blockIdx.x, blockIdx.y, X, ld, M, N, rows_per_block, part, red);
}

// out[n] = T(sum_p part[p][n]) in order p = 0..parts-1; 8 partial rows in flight per thread.
template <typename T>
__device__ __forceinline__ void colsum_final_column(int n, const float* __restrict__ part, int parts, int N, T* __restrict__ out) {
  if (n >= N) return;
  float s = 0.f;
  int p = 0;
  // a few blocks of dependent-latency work: 32, then 8 partial rows in flight per thread
  for (; p + 32 <= parts; p += 32) {
    float v[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) v[j] = part[static_cast<int64_t>(p + j) * N + n];
#pragma unroll
    for (int j = 0; j < 32; ++j) s += v[j];
  }
  for (; p + 8 <= parts; p += 8) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = part[static_cast<int64_t>(p + j) * N + n];
#pragma unroll
    for (int j = 0; j < 8; ++j) s += v[j];
  }
  for (; p < parts; ++p) s += part[static_cast<int64_t>(p) * N + n];
  out[n] = elem<T>::from_float(s);
}

template <typename T>
__global__ __launch_bounds__(256) void colsum_final_kernel(const float* __restrict__ part, int parts, int N,
                                                           T* __restrict__ out) {
  colsum_final_column<T>(blockIdx.x * 256 + threadIdx.x, part, parts, N, out);
}

// ---------------------------------------------------------------------------------------------
// Several of the reductions above in one launch: an operator that ends in a handful of them (the MLP backward: two
// split-K reductions and two bias-gradient sums) queues them as jobs and runs one kernel at its end instead of
// four launches of a few microseconds each. A block finds its job from the block ranges (uniform per block) and
// then does exactly what the stand-alone kernel's block would have done: results are bit-identical.
// ---------------------------------------------------------------------------------------------
enum GemmTile { TILE_L = 0, TILE_M = 1, TILE_S = 2, TILE_R = 3 };

template <int TILE> struct tile_cfg;
template <> struct tile_cfg<TILE_L> { static constexpr int BM = 256, BN = 256, WM = 2, WN = 4; };
template <> struct tile_cfg<TILE_M> { static constexpr int BM = 128, BN = 128, WM = 2, WN = 2; };
template <> struct tile_cfg<TILE_S> { static constexpr int BM = 256, BN = 64, WM = 4, WN = 1; };
template <> struct tile_cfg<TILE_R> { static constexpr int BM = 128, BN = 512, WM = 4, WN = 2; };

enum TailKind { TAIL_SPLITK_M = 1, TAIL_SPLITK_L = 2, TAIL_COLSUM = 3, TAIL_COLSUM_PARTIAL = 4, TAIL_COLSUM_PARTIAL_VEC = 5 };
struct TailJob {
  int kind;
  int first_block;       // the job's blocks are [first_block, next job's first_block)
  const float* src;      // split-K partials / column-sum partial rows
  void* dst;
  int64_t ldc, sC;       // TAIL_COLSUM_PARTIAL*: ldc = row pitch of x
  int M, N, m_tiles, n_tiles, batch, splits, c_vec, parts;
  float alpha;
  const void* x;         // TAIL_COLSUM_PARTIAL*: the matrix whose columns are summed (dst: fp32 partial rows)
  int rows_per_block, col_blocks;
};
constexpr int TAIL_MAX_JOBS = 8;
struct TailArgs {
  int njobs;
  int blocks;            // all jobs together
  TailJob job[TAIL_MAX_JOBS];
};

constexpr int TAIL_LDS_FLOATS = 8 * (32 * 8 + 1);   // what a partial column sum needs

// One block of 256 threads runs block `vb` of the job list: exactly what the stand-alone kernel's block does.
// lds: TAIL_LDS_FLOATS floats of LDS for the block's use.
template <typename T>
__device__ __forceinline__ void tail_block(const TailArgs& a, int vb, float* lds) {
  int j = 0;
  while (j + 1 < a.njobs && vb >= a.job[j + 1].first_block) ++j;
  const TailJob& t = a.job[j];
  const int64_t local = static_cast<int64_t>(vb - t.first_block) * 256 + threadIdx.x;
  if (t.kind == TAIL_COLSUM_PARTIAL || t.kind == TAIL_COLSUM_PARTIAL_VEC) {
    const int lb = vb - t.first_block, bx = lb % t.col_blocks, by = lb / t.col_blocks;
    if (t.kind == TAIL_COLSUM_PARTIAL_VEC) {
      if constexpr (sizeof(T) == 2) colsum_partial_block<T, true>(bx, by, static_cast<const T*>(t.x), t.ldc, t.M, t.N, t.rows_per_block, static_cast<float*>(t.dst), lds);
    } else {
      colsum_partial_block<T, false>(bx, by, static_cast<const T*>(t.x), t.ldc, t.M, t.N, t.rows_per_block, static_cast<float*>(t.dst), lds);
    }
  } else if (t.kind == TAIL_SPLITK_M) {
    using C = tile_cfg<TILE_M>;
    splitk_reduce_slot<T, C::BM, C::BN, C::WM, C::WN>(local, t.src, static_cast<T*>(t.dst), t.ldc, t.M, t.N, t.m_tiles, t.n_tiles,
                                                      t.batch, t.sC, t.splits, t.alpha, t.c_vec);
  } else if (t.kind == TAIL_SPLITK_L) {
    using C = tile_cfg<TILE_L>;
    splitk_reduce_slot<T, C::BM, C::BN, C::WM, C::WN>(local, t.src, static_cast<T*>(t.dst), t.ldc, t.M, t.N, t.m_tiles, t.n_tiles,
                                                      t.batch, t.sC, t.splits, t.alpha, t.c_vec);
  } else if (t.kind == TAIL_COLSUM) {
    colsum_final_column<T>(static_cast<int>(local), t.src, t.parts, t.N, static_cast<T*>(t.dst));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void reduce_tail_kernel(const TailArgs a) {
  __shared__ float lds[TAIL_LDS_FLOATS];
  tail_block<T>(a, static_cast<int>(blockIdx.x), lds);
}

// The same job list run by `nriders` blocks that ride along in another kernel's launch (gemm_ring.hip.h): the blocks
// of the list are dealt out round-robin.
template <typename T>
__device__ __forceinline__ void tail_ride(const TailArgs& a, int rider, int nriders, float* lds) {
  for (int vb = rider; vb < a.blocks; vb += nriders) tail_block<T>(a, vb, lds);
}

// Host side (reduce.hip): a list of jobs of one dtype, launched once.
struct ReduceTail {
  TailArgs args;
  int& blocks;
  ReduceTail() : blocks(args.blocks) { args.njobs = 0; args.blocks = 0; }
  ReduceTail(const ReduceTail&) = delete;
  bool full() const { return args.njobs >= TAIL_MAX_JOBS; }
  bool empty() const { return args.njobs == 0 || args.blocks == 0; }
};
int tail_add_splitk(ReduceTail& t, int tile, const float* ws, void* C, int64_t ldc, int M, int N, int m_tiles, int n_tiles,
                    int batch, int64_t sC, int splits, float alpha, int c_vec);
int tail_add_colsum(ReduceTail& t, const float* part, int parts, int N, void* out);
// the partial phase of a column sum as a job (what colsum_partial_run launches on its own)
int tail_add_colsum_partial(ReduceTail& t, int dtype, const void* X, int64_t ld, int M, int N, float* part);
int tail_launch(const ReduceTail& t, int dtype, hipStream_t st);
// the partial phase of colsum_run alone (its final sum is then queued with tail_add_colsum)
int colsum_partial_run(int dtype, const void* X, int64_t ld, int M, int N, float* part, hipStream_t st);

// bias-gradient style column sums: out[n] = sum_m X[m][n]; part is fp32 scratch of
// colsum_parts(M) * N floats.
int colsum_parts(int M);
int colsum_run(int dtype, const void* X, int64_t ld, int M, int N, float* part, void* out, hipStream_t st);
int colsum_finish(int dtype, const float* part, int parts, int N, void* out, hipStream_t st);

}  // namespace nmtg
