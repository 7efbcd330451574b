// Column sums out[n] = sum_m X[m][n] (bias gradients): partial sums per row block, then a fixed-order final sum.
#include "reduce.cuh"
#include <algorithm>

namespace nmtg {
namespace {
int ceil_div(int a, int b) { return (a + b - 1) / b; }
}  // namespace

int colsum_parts(int M) { return std::max(1, std::min(64, ceil_div(M, 128))); }

int colsum_finish(int dtype, const float* part, int parts, int N, void* out, hipStream_t st) {
  TraceScope trace("colsum_final", st);
  NMTG_DISPATCH_DTYPE(dtype, T,
                      hipLaunchKernelGGL((colsum_final_kernel<T>), dim3(ceil_div(N, 256)), dim3(256), 0, st, part, parts, N,
                                         static_cast<T*>(out)));
  NMTG_CHECK_LAUNCH("colsum_finish");
  return 0;
}

int colsum_run(int dtype, const void* X, int64_t ld, int M, int N, float* part, void* out, hipStream_t st) {
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
  return colsum_finish(dtype, part, parts, N, out, st);
}

}  // namespace nmtg
