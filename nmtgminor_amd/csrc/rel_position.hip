// Elementwise pieces of self-attention with relative position encodings (Transformer-XL form) for gfx950.
//
// Stand in for what RelativeSelfAttnFunc of the reference does between its GEMMs with PyTorch ops
// (onmt/modules/optimized/relative_self_attention_func.py): the additions of r_w_bias / r_r_bias to the queries
// (:210-217), RelativeShift.forward on the position scores followed by the cut to len_k and the sum with the content
// scores (:26-50, :246-253), and RelativeShift.backward on the score gradient (:52-76, :621-630).
//
// The shift is pure index arithmetic. The reference pads a zero column in front of bd[b] ([len_q, len_r]), reads the
// padded buffer as [len_r + 1, len_q], drops its first row and reads the remainder as [len_q, len_r]. In flat offsets:
// output element f = i * len_r + j is padded element p = f + len_q, i.e. row i2 = p / (len_r + 1), column
// c = p % (len_r + 1) of the padded matrix: 0 if c == 0, bd[b][i2][c - 1] otherwise. A row of the output is therefore a
// contiguous run of bd with one zero after every len_r elements of it; the run is not aligned with the output row, so
// the shifted operand is read element by element (coalesced across the lanes of a wavefront) while the operand that
// keeps its place moves in 16-byte accesses. All three kernels are bandwidth bound: one read of each operand, one
// write of the result.
#include "common.hip.h"

namespace nmtg {
namespace {

constexpr int RP_THREADS = 256;

// rw_q = q + r_w_bias, rr_q = q + r_r_bias; one thread per EPV consecutive elements of a head row.
template <typename T, int EPV>
__global__ __launch_bounds__(RP_THREADS) void rel_query_bias_kernel(
    const T* __restrict__ q, int64_t ld_q, const T* __restrict__ r_w_bias, const T* __restrict__ r_r_bias,
    T* __restrict__ rw_q, T* __restrict__ rr_q, int64_t rows, int heads, int head_dim) {
  const int per_row = head_dim / EPV;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * RP_THREADS + threadIdx.x;
  if (item >= rows * per_row) return;
  const int64_t r = item / per_row;
  const int d = static_cast<int>(item - r * per_row) * EPV;
  const int h = static_cast<int>(r % heads);
  float qv[EPV], wv[EPV], rv[EPV];
  load_pack<T, EPV>(q + r * ld_q + d, qv);
  load_pack<T, EPV>(r_w_bias + h * head_dim + d, wv);
  load_pack<T, EPV>(r_r_bias + h * head_dim + d, rv);
#pragma unroll
  for (int j = 0; j < EPV; ++j) {
    wv[j] += qv[j];
    rv[j] += qv[j];
  }
  store_pack<T, EPV>(rw_q + r * head_dim + d, wv);
  store_pack<T, EPV>(rr_q + r * head_dim + d, rv);
}

// Indices inside one batch entry fit 32 bits (the entry points check len_q * (len_r + 1) < 2^31), so a thread does two
// 32-bit divisions, one for its place in the output and one for its first source element, and then walks the source:
// consecutive output elements are consecutive padded elements, column c of the padded row advancing to 0 of the next
// row after len_r.

// scores[b][i][j] += shift(bd)[b][i][j]; grid (items of a batch entry, batch), one thread per EPV columns of one row.
template <typename T, int EPV>
__global__ __launch_bounds__(RP_THREADS) void rel_shift_add_kernel(T* __restrict__ scores, const T* __restrict__ bd,
                                                                   uint32_t len_q, uint32_t len_k, uint32_t len_r) {
  const uint32_t per_row = (len_k + EPV - 1) / EPV;
  const uint32_t item = blockIdx.x * RP_THREADS + threadIdx.x;
  if (item >= len_q * per_row) return;
  const uint32_t i = item / per_row, j0 = (item - i * per_row) * EPV;
  const int64_t b = blockIdx.y;
  T* row = scores + (b * len_q + i) * len_k;
  const T* bd_b = bd + b * len_q * len_r;
  const uint32_t p = i * len_r + j0 + len_q;             // first padded element
  uint32_t i2 = p / (len_r + 1), c = p - i2 * (len_r + 1);
  const uint32_t n = min(static_cast<uint32_t>(EPV), len_k - j0);
  float sh[EPV];
#pragma unroll
  for (int u = 0; u < EPV; ++u) {
    sh[u] = (u < n && c != 0) ? elem<T>::to_float(bd_b[i2 * len_r + c - 1]) : 0.f;
    if (++c > len_r) { c = 0; ++i2; }
  }
  if (n == EPV) {
    float v[EPV];
    load_pack<T, EPV>(row + j0, v);
#pragma unroll
    for (int u = 0; u < EPV; ++u) v[u] += sh[u];
    store_pack<T, EPV>(row + j0, v);
  } else {
    for (uint32_t u = 0; u < n; ++u) row[j0 + u] = elem<T>::from_float(elem<T>::to_float(row[j0 + u]) + sh[u]);
  }
}

// grad_bd[b][i2][c - 1] = grad_scores[b][i][j] with i * len_r + j = i2 * (len_r + 1) + c - len_q (0 if that is negative
// or j >= len_k); grid (items of a batch entry, batch), one thread per EPV columns of one row of grad_bd.
template <typename T, int EPV>
__global__ __launch_bounds__(RP_THREADS) void rel_shift_bwd_kernel(const T* __restrict__ grad_scores, T* __restrict__ grad_bd,
                                                                   uint32_t len_q, uint32_t len_k, uint32_t len_r) {
  const uint32_t per_row = (len_r + EPV - 1) / EPV;
  const uint32_t item = blockIdx.x * RP_THREADS + threadIdx.x;
  if (item >= len_q * per_row) return;
  const uint32_t i2 = item / per_row, c0 = (item - i2 * per_row) * EPV;   // column of grad_bd = c - 1
  const int64_t b = blockIdx.y;
  const T* g_b = grad_scores + b * len_q * len_k;
  T* out = grad_bd + (b * len_q + i2) * len_r;
  // flat offset of the first source element in the [len_q, len_r] view of the gradient; negative inside the dropped row
  const int64_t f0 = static_cast<int64_t>(i2) * (len_r + 1) + c0 + 1 - len_q;
  uint32_t i = 0, j = 0;
  if (f0 >= 0) {
    i = static_cast<uint32_t>(f0) / len_r;
    j = static_cast<uint32_t>(f0) - i * len_r;
  }
  const uint32_t n = min(static_cast<uint32_t>(EPV), len_r - c0);
  float v[EPV];
#pragma unroll
  for (int u = 0; u < EPV; ++u) {
    const bool live = u < n && f0 + u >= 0;
    v[u] = (live && j < len_k) ? elem<T>::to_float(g_b[i * len_k + j]) : 0.f;
    if (f0 + u >= 0 && ++j == len_r) { j = 0; ++i; }
  }
  if (n == EPV) {
    store_pack<T, EPV>(out + c0, v);
  } else {
    for (uint32_t u = 0; u < n; ++u) out[c0 + u] = elem<T>::from_float(v[u]);
  }
}

// out[r][c] = a[r][c] + b[r][c] over rows of `cols` elements with their own pitches (out may be a or b); one thread per
// EPV consecutive columns of one row.
template <typename T, int EPV>
__global__ __launch_bounds__(RP_THREADS) void add_rows_kernel(T* out, int64_t ld_out, const T* a, int64_t ld_a,
                                                              const T* b, int64_t ld_b, int64_t rows, int cols) {
  const int per_row = cols / EPV;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * RP_THREADS + threadIdx.x;
  if (item >= rows * per_row) return;
  const int64_t r = item / per_row;
  const int c = static_cast<int>(item - r * per_row) * EPV;
  float av[EPV], bv[EPV];
  load_pack<T, EPV>(a + r * ld_a + c, av);
  load_pack<T, EPV>(b + r * ld_b + c, bv);
#pragma unroll
  for (int j = 0; j < EPV; ++j) av[j] += bv[j];
  store_pack<T, EPV>(out + r * ld_out + c, av);
}

inline bool fits_grid(int64_t items, int64_t batch) {
  return (items + RP_THREADS - 1) / RP_THREADS <= 0x7fffffff && batch <= 65535;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_rel_query_bias(const void* q, int64_t ld_q, const void* r_w_bias, const void* r_r_bias, void* rw_q,
                                   void* rr_q, int64_t rows, int64_t heads, int64_t head_dim, int dtype, void* stream) {
  NMTG_REQUIRE(rows >= 0 && heads > 0 && heads <= 65536 && head_dim > 0 && head_dim <= 65536,
               "rel_query_bias: bad sizes (rows %lld, heads %lld, head_dim %lld)", (long long)rows, (long long)heads,
               (long long)head_dim);
  NMTG_REQUIRE(ld_q >= head_dim, "rel_query_bias: row pitch %lld below head_dim %lld", (long long)ld_q, (long long)head_dim);
  NMTG_REQUIRE(rows * head_dim < (int64_t(1) << 40), "rel_query_bias: too many elements");
  if (rows == 0) return 0;
  NMTG_REQUIRE(q && r_w_bias && r_r_bias && rw_q && rr_q, "rel_query_bias: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  TraceScope trace("rel_query_bias", st);
  NMTG_DISPATCH_DTYPE(
      dtype, T, constexpr int WIDE = 16 / sizeof(T);
      const bool wide = head_dim % WIDE == 0 && ld_q % WIDE == 0 && aligned16(q) && aligned16(r_w_bias) &&
                        aligned16(r_r_bias) && aligned16(rw_q) && aligned16(rr_q);
      const int64_t items = wide ? rows * (head_dim / WIDE) : rows * head_dim;
      const unsigned grid = static_cast<unsigned>((items + RP_THREADS - 1) / RP_THREADS);
      if (wide) hipLaunchKernelGGL((rel_query_bias_kernel<T, WIDE>), dim3(grid), dim3(RP_THREADS), 0, st,
                                   static_cast<const T*>(q), ld_q, static_cast<const T*>(r_w_bias),
                                   static_cast<const T*>(r_r_bias), static_cast<T*>(rw_q), static_cast<T*>(rr_q), rows,
                                   static_cast<int>(heads), static_cast<int>(head_dim));
      else hipLaunchKernelGGL((rel_query_bias_kernel<T, 1>), dim3(grid), dim3(RP_THREADS), 0, st, static_cast<const T*>(q),
                              ld_q, static_cast<const T*>(r_w_bias), static_cast<const T*>(r_r_bias), static_cast<T*>(rw_q),
                              static_cast<T*>(rr_q), rows, static_cast<int>(heads), static_cast<int>(head_dim)));
  NMTG_CHECK_LAUNCH("rel_query_bias");
  return 0;
}

extern "C" int nmtg_rel_shift_add(void* scores, const void* bd, int64_t batch, int64_t len_q, int64_t len_k, int64_t len_r,
                                  int dtype, void* stream) {
  NMTG_REQUIRE(batch >= 0 && len_q >= 0 && len_k >= 0 && len_r >= 0, "rel_shift_add: negative size");
  NMTG_REQUIRE(len_r >= len_k, "rel_shift_add: %lld relative positions for %lld keys (need at least as many)",
               (long long)len_r, (long long)len_k);
  if (batch == 0 || len_q == 0 || len_k == 0) return 0;
  NMTG_REQUIRE(len_q * (len_r + 1) < (int64_t(1) << 31) && fits_grid(len_q * len_k, batch),
               "rel_shift_add: sizes beyond the kernel's 32-bit indices (len_q * (len_r + 1) < 2^31, batch <= 65535)");
  NMTG_REQUIRE(scores && bd, "rel_shift_add: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  TraceScope trace("rel_shift_add", st);
  NMTG_DISPATCH_DTYPE(
      dtype, T, constexpr int WIDE = 16 / sizeof(T);
      const bool wide = len_k % WIDE == 0 && aligned16(scores);
      const int64_t items = len_q * (wide ? len_k / WIDE : len_k);
      const dim3 grid(static_cast<unsigned>((items + RP_THREADS - 1) / RP_THREADS), static_cast<unsigned>(batch));
      if (wide) hipLaunchKernelGGL((rel_shift_add_kernel<T, WIDE>), grid, dim3(RP_THREADS), 0, st, static_cast<T*>(scores),
                                   static_cast<const T*>(bd), static_cast<uint32_t>(len_q), static_cast<uint32_t>(len_k),
                                   static_cast<uint32_t>(len_r));
      else hipLaunchKernelGGL((rel_shift_add_kernel<T, 1>), grid, dim3(RP_THREADS), 0, st, static_cast<T*>(scores),
                              static_cast<const T*>(bd), static_cast<uint32_t>(len_q), static_cast<uint32_t>(len_k),
                              static_cast<uint32_t>(len_r)));
  NMTG_CHECK_LAUNCH("rel_shift_add");
  return 0;
}

extern "C" int nmtg_rel_shift_bwd(const void* grad_scores, void* grad_bd, int64_t batch, int64_t len_q, int64_t len_k,
                                  int64_t len_r, int dtype, void* stream) {
  NMTG_REQUIRE(batch >= 0 && len_q >= 0 && len_k >= 0 && len_r >= 0, "rel_shift_bwd: negative size");
  NMTG_REQUIRE(len_r >= len_k, "rel_shift_bwd: %lld relative positions for %lld keys (need at least as many)",
               (long long)len_r, (long long)len_k);
  if (batch == 0 || len_q == 0 || len_r == 0) return 0;
  NMTG_REQUIRE(len_q * (len_r + 1) < (int64_t(1) << 31) && fits_grid(len_q * len_r, batch),
               "rel_shift_bwd: sizes beyond the kernel's 32-bit indices (len_q * (len_r + 1) < 2^31, batch <= 65535)");
  NMTG_REQUIRE(grad_scores && grad_bd, "rel_shift_bwd: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  TraceScope trace("rel_shift_bwd", st);
  NMTG_DISPATCH_DTYPE(
      dtype, T, constexpr int WIDE = 16 / sizeof(T);
      const bool wide = len_r % WIDE == 0 && aligned16(grad_bd);
      const int64_t items = len_q * (wide ? len_r / WIDE : len_r);
      const dim3 grid(static_cast<unsigned>((items + RP_THREADS - 1) / RP_THREADS), static_cast<unsigned>(batch));
      if (wide) hipLaunchKernelGGL((rel_shift_bwd_kernel<T, WIDE>), grid, dim3(RP_THREADS), 0, st,
                                   static_cast<const T*>(grad_scores), static_cast<T*>(grad_bd), static_cast<uint32_t>(len_q),
                                   static_cast<uint32_t>(len_k), static_cast<uint32_t>(len_r));
      else hipLaunchKernelGGL((rel_shift_bwd_kernel<T, 1>), grid, dim3(RP_THREADS), 0, st,
                              static_cast<const T*>(grad_scores), static_cast<T*>(grad_bd), static_cast<uint32_t>(len_q),
                              static_cast<uint32_t>(len_k), static_cast<uint32_t>(len_r)));
  NMTG_CHECK_LAUNCH("rel_shift_bwd");
  return 0;
}

extern "C" int nmtg_add_rows(void* out, int64_t ld_out, const void* a, int64_t ld_a, const void* b, int64_t ld_b, int64_t rows,
                             int64_t cols, int dtype, void* stream) {
  NMTG_REQUIRE(rows >= 0 && cols >= 0 && cols <= INT32_MAX && rows * cols < (int64_t(1) << 40),
               "add_rows: bad sizes (rows %lld, columns %lld)", (long long)rows, (long long)cols);
  NMTG_REQUIRE(ld_out >= cols && ld_a >= cols && ld_b >= cols, "add_rows: a row pitch is below the number of columns %lld",
               (long long)cols);
  if (rows == 0 || cols == 0) return 0;
  NMTG_REQUIRE(out && a && b, "add_rows: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  TraceScope trace("add_rows", st);
  NMTG_DISPATCH_DTYPE(
      dtype, T, constexpr int WIDE = 16 / sizeof(T);
      const bool wide = cols % WIDE == 0 && ld_out % WIDE == 0 && ld_a % WIDE == 0 && ld_b % WIDE == 0 && aligned16(out) &&
                        aligned16(a) && aligned16(b);
      const int64_t items = wide ? rows * (cols / WIDE) : rows * cols;
      NMTG_REQUIRE((items + RP_THREADS - 1) / RP_THREADS <= 0x7fffffff, "add_rows: too many elements for one launch");
      const unsigned grid = static_cast<unsigned>((items + RP_THREADS - 1) / RP_THREADS);
      if (wide) hipLaunchKernelGGL((add_rows_kernel<T, WIDE>), dim3(grid), dim3(RP_THREADS), 0, st, static_cast<T*>(out), ld_out,
                                   static_cast<const T*>(a), ld_a, static_cast<const T*>(b), ld_b, rows, static_cast<int>(cols));
      else hipLaunchKernelGGL((add_rows_kernel<T, 1>), dim3(grid), dim3(RP_THREADS), 0, st, static_cast<T*>(out), ld_out,
                              static_cast<const T*>(a), ld_a, static_cast<const T*>(b), ld_b, rows, static_cast<int>(cols)));
  NMTG_CHECK_LAUNCH("add_rows");
  return 0;
}
