// Column sums out[n] = sum_m X[m][n] (bias gradients): partial sums per row block, then a fixed-order final sum.
#include "reduce.hip.h"
#include <algorithm>

namespace nmtg {
namespace {
int ceil_div(int a, int b) { return (a + b - 1) / b; }
}  // namespace

// row blocks of 64 rows (eight rows per row lane), at most 256 of them: a [8192 x 512] gradient is 256 blocks
int colsum_parts(int M) { return std::max(1, std::min(256, ceil_div(M, 64))); }

int colsum_finish(int dtype, const float* part, int parts, int N, void* out, hipStream_t st) {
  TraceScope trace("colsum_final", st);
  NMTG_DISPATCH_DTYPE(dtype, T,
                      hipLaunchKernelGGL((colsum_final_kernel<T>), dim3(ceil_div(N, 256)), dim3(256), 0, st, part, parts, N,
                                         static_cast<T*>(out)));
  NMTG_CHECK_LAUNCH("colsum_finish");
  return 0;
}

int colsum_partial_run(int dtype, const void* X, int64_t ld, int M, int N, float* part, hipStream_t st) {
  const int parts = colsum_parts(M);
  const int rpb = ceil_div(M, parts);
  {
    TraceScope trace("colsum_partial", st);
    const bool vec = dtype != NMTG_F32 && aligned16(X) && ld % 8 == 0 && N % 8 == 0;
    if (vec) {
      NMTG_DISPATCH_DTYPE(dtype, T,
                          hipLaunchKernelGGL((colsum_partial_kernel<T, true>), dim3(ceil_div(N, 256), parts), dim3(256), 0, st,
                                             static_cast<const T*>(X), ld, M, N, rpb, part));
    } else {
      NMTG_DISPATCH_DTYPE(dtype, T,
                          hipLaunchKernelGGL((colsum_partial_kernel<T, false>), dim3(ceil_div(N, 32), parts), dim3(256), 0, st,
                                             static_cast<const T*>(X), ld, M, N, rpb, part));
    }
  }
  NMTG_CHECK_LAUNCH("colsum");
  return 0;
}

int colsum_run(int dtype, const void* X, int64_t ld, int M, int N, float* part, void* out, hipStream_t st) {
  if (int rc = colsum_partial_run(dtype, X, ld, M, N, part, st)) return rc;
  return colsum_finish(dtype, part, colsum_parts(M), N, out, st);
}

// ---- several reductions in one launch ----
int tail_add_splitk(ReduceTail& t, int tile, const float* ws, void* C, int64_t ldc, int M, int N, int m_tiles, int n_tiles,
                    int batch, int64_t sC, int splits, float alpha, int c_vec) {
  if (t.full() || (tile != TILE_M && tile != TILE_L)) return fail(NMTG_ERR_UNSUPPORTED, "reduce tail: cannot queue this split-K job");
  const int bm = tile == TILE_M ? 128 : 256;
  const int64_t slots = static_cast<int64_t>(batch) * m_tiles * n_tiles * (static_cast<int64_t>(bm) * bm / 4);   // one float4 slot per 4 outputs
  const int64_t blocks = (slots + 255) / 256;
  if (blocks <= 0 || t.blocks + blocks > 0x7fffffff) return fail(NMTG_ERR_UNSUPPORTED, "reduce tail: grid too large");
  TailJob& j = t.args.job[t.args.njobs++];
  j = TailJob{};
  j.kind = tile == TILE_M ? TAIL_SPLITK_M : TAIL_SPLITK_L;
  j.first_block = t.blocks;
  j.src = ws; j.dst = C; j.ldc = ldc; j.sC = sC;
  j.M = M; j.N = N; j.m_tiles = m_tiles; j.n_tiles = n_tiles; j.batch = batch; j.splits = splits; j.c_vec = c_vec;
  j.alpha = alpha;
  t.blocks += static_cast<int>(blocks);
  return 0;
}

int tail_add_colsum(ReduceTail& t, const float* part, int parts, int N, void* out) {
  if (t.full()) return fail(NMTG_ERR_UNSUPPORTED, "reduce tail: too many jobs");
  TailJob& j = t.args.job[t.args.njobs++];
  j = TailJob{};
  j.kind = TAIL_COLSUM;
  j.first_block = t.blocks;
  j.src = part; j.dst = out; j.parts = parts; j.N = N;
  t.blocks += ceil_div(N, 256);
  return 0;
}

int tail_add_colsum_partial(ReduceTail& t, int dtype, const void* X, int64_t ld, int M, int N, float* part) {
  if (t.full()) return fail(NMTG_ERR_UNSUPPORTED, "reduce tail: too many jobs");
  const int parts = colsum_parts(M);
  const bool vec = dtype != NMTG_F32 && aligned16(X) && ld % 8 == 0 && N % 8 == 0;
  TailJob& j = t.args.job[t.args.njobs++];
  j = TailJob{};
  j.kind = vec ? TAIL_COLSUM_PARTIAL_VEC : TAIL_COLSUM_PARTIAL;
  j.first_block = t.blocks;
  j.x = X; j.ldc = ld; j.M = M; j.N = N; j.dst = part;
  j.rows_per_block = ceil_div(M, parts);
  j.col_blocks = ceil_div(N, vec ? 256 : 32);
  t.blocks += j.col_blocks * parts;
  return 0;
}

int tail_launch(const ReduceTail& t, int dtype, hipStream_t st) {
  if (t.args.njobs == 0 || t.blocks == 0) return 0;
  TraceScope trace("reduce_tail", st);
  const TailArgs args = t.args;
  const unsigned blocks = static_cast<unsigned>(args.blocks);
  NMTG_DISPATCH_DTYPE(dtype, T,
                      hipLaunchKernelGGL((reduce_tail_kernel<T>), dim3(blocks), dim3(256), 0, st, args));
  NMTG_CHECK_LAUNCH("reduce_tail");
  return 0;
}

}  // namespace nmtg

using namespace nmtg;

extern "C" int64_t nmtg_colsum_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0 || rows > INT32_MAX || cols > INT32_MAX) return 0;
  return static_cast<int64_t>(colsum_parts(static_cast<int>(rows))) * cols * static_cast<int64_t>(sizeof(float));
}

extern "C" int nmtg_colsum(const void* x, int64_t rows, int64_t cols, int64_t ld, void* out, void* workspace,
                           int64_t workspace_bytes, int dtype, void* stream) {
  NMTG_REQUIRE(rows > 0 && rows <= INT32_MAX && cols >= 0 && cols <= INT32_MAX,
               "colsum: bad sizes (rows %lld, columns %lld); a sum over no rows is the caller's zero fill", (long long)rows,
               (long long)cols);
  NMTG_REQUIRE(ld >= cols, "colsum: row pitch %lld below the number of columns %lld", (long long)ld, (long long)cols);
  if (cols == 0) return 0;
  NMTG_REQUIRE(x && out, "colsum: null pointer argument");
  NMTG_REQUIRE(workspace && workspace_bytes >= nmtg_colsum_workspace_bytes(rows, cols),
               "colsum: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
               (long long)nmtg_colsum_workspace_bytes(rows, cols));
  return colsum_run(dtype, x, ld, static_cast<int>(rows), static_cast<int>(cols), static_cast<float*>(workspace), out,
                    static_cast<hipStream_t>(stream));
}
