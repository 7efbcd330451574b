// Masked row softmax with optional inverted dropout, and its backward, for gfx950.
//
// Stands in for the softmax stage of the reference's fused attention
// (onmt/modules/extensions/multihead_attn_blaslt/softmax_apex.h: dispatch_softmax_dropout
// :443-486, dispatch_softmax :1263-1300, dispatch_softmax_dropout_presampled :874-912,
// dispatch_softmax_dropout_backward_recompute :4039-4075, dispatch_softmax_backward_norecompute
// :3467-3500) and for the stand-alone module mask_softmax_dropout_cuda that
// onmt/modules/optimized/attention_softmax.py:32-59 calls.
//
// One 64-lane wavefront owns one row of `cols` keys and keeps it in registers (VPL vectors of
// EPV elements per lane), so every score is read once and every probability written once.
// Masking can be fused: a key-padding mask [batch, cols] (row -> batch = row / (heads*q_len)) or
// a time mask [q_len, cols] (row -> query = row % q_len); masked keys count as -inf. A row whose
// keys are all masked yields zeros (the reference turns the NaN into 0, softmax_apex.h:209-211).
// Dropout: keep mask of one byte per element, read (replay) or drawn from Philox and written.
//
// Bandwidth bound. Per element: forward reads the score (+1 B mask in replay mode), writes the
// result (+1 B mask in RNG mode); backward reads grad, the saved scores or probabilities and the
// mask byte, writes the score gradient.
#include "common.hip.h"

namespace nmtg {
namespace {

constexpr int SM_THREADS = 256;
constexpr int SM_WAVES = SM_THREADS / kWave;
enum { SM_NO_DROPOUT = 0, SM_MASK_IN = 1, SM_MASK_RNG = 2 };
enum { SM_NOMASK = 0, SM_PAD = 1, SM_TIME = 2 };

struct SoftmaxArgs {
  const void* in;          // fwd: scores; bwd: grad wrt the dropped probabilities
  const void* saved;       // bwd: saved scores (recompute) or saved probabilities
  void* out;               // fwd: dropped probabilities; bwd: grad wrt scores
  void* out_softmax;       // fwd: optional pre-dropout probabilities
  uint8_t* dmask;          // dropout keep mask
  const uint8_t* kmask;    // key-padding or time mask (1 = masked)
  int64_t rows;
  int cols;
  int q_len;               // queries per (batch, head)
  int heads;
  int kmask_kind;
  int dropout_mode;
  int from_scores;         // bwd: saved holds scores (1) or probabilities (0)
  float keep_p, scale;
  uint64_t seed, offset;
  // relative-position form (REL kernels): rows = batch * q_len, every row also takes (forward) or feeds (backward) the
  // shifted position term
  const void* bd;          // fwd: position scores [batch, q_len, len_r]
  void* scores_out;        // fwd: the summed scores, [batch, q_len, cols] (may be `in`)
  void* grad_bd;           // bwd: gradient of the position scores [batch, q_len, len_r]
  int len_r;
};

// The relative shift as seen from row i of a [q_len, cols] score matrix (relative_self_attention_func.py:26-50 of the
// reference: a zero column in front of bd [q_len, len_r], the padded buffer read as [len_r + 1, q_len], first row
// dropped). Element j of the row is padded element p = i * len_r + q_len + j, which lies in padded row i2 = p / (len_r + 1)
// at column c = p % (len_r + 1): zero if c == 0, bd[i2][c - 1] otherwise. A row is shorter than a padded row, so it
// crosses at most one padded-row boundary: with i2 and c0 taken for j = 0, element j has c = c0 + j counted from the
// start of padded row i2, c == len_r + 1 is the zero column of the next padded row and anything beyond it lies one
// element earlier in bd than c - 1 says.
struct RelRow {
  uint32_t i;              // the row's query position
  uint32_t c0;             // column of the row's first element inside its padded row
  int64_t first;           // element offset of bd[b][i2][0]
};
__device__ __forceinline__ RelRow rel_row(int64_t row, uint32_t q_len, uint32_t len_r) {   // row < 2^31 (checked at entry)
  const uint32_t b = static_cast<uint32_t>(row) / q_len, i = static_cast<uint32_t>(row) - b * q_len;
  const uint32_t p0 = i * len_r + q_len, i2 = p0 / (len_r + 1);
  return RelRow{i, p0 - i2 * (len_r + 1), (static_cast<int64_t>(b) * q_len + i2) * len_r};
}
// offset from RelRow::first of the bd element behind column c, or -1 for the zero column
__device__ __forceinline__ int rel_source(uint32_t c, uint32_t len_r) {
  if (c == 0 || c == len_r + 1) return -1;
  return static_cast<int>(c) - 1 - (c > len_r + 1 ? 1 : 0);
}

// 32-bit index arithmetic wherever the row count allows it (a 64-bit division is some 140 scalar instructions,
// as much as the rest of a short row's work).
__device__ __forceinline__ const uint8_t* kmask_row(const SoftmaxArgs& a, int64_t row) {
  if (a.kmask_kind == SM_NOMASK) return nullptr;
  const int64_t group = a.kmask_kind == SM_PAD ? static_cast<int64_t>(a.heads) * a.q_len : a.q_len;
  int64_t idx;
  if (a.rows <= 0x7fffffff) {
    const uint32_t r = static_cast<uint32_t>(row), g = static_cast<uint32_t>(group);
    idx = a.kmask_kind == SM_PAD ? r / g : r % g;
  } else {
    idx = a.kmask_kind == SM_PAD ? row / group : row % group;
  }
  return a.kmask + idx * a.cols;
}

// Every kernel below issues all of a row's loads (scores, key mask, dropout mask, gradient) before it uses any of
// them, so that a wavefront waits for memory once per row instead of once per load: with one row per wavefront
// these kernels are bound by that latency, not by bandwidth. Lanes beyond the row's end load from column 0 and
// discard the value.
template <int EPV>
__device__ __forceinline__ int row_col(int i, int lane) { return (i * kWave + lane) * EPV; }

template <typename T, int EPV, int VPL>
__device__ __forceinline__ void row_load(const T* __restrict__ src, int cols, int lane, pack<T, EPV> (&r)[VPL]) {
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = row_col<EPV>(i, lane);
    r[i] = load_raw<T, EPV>(src + (col < cols ? col : 0));
  }
}
template <typename T, int EPV, int VPL>
__device__ __forceinline__ void row_pin(pack<T, EPV> (&r)[VPL]) {
#pragma unroll
  for (int i = 0; i < VPL; ++i) pin_raw(r[i]);
}

// Turns the row's loaded scores into normalised probabilities in v (masked / out-of-range -> -inf before the
// maximum; a row with every key masked gives zeros).
template <typename T, int EPV, int VPL>
__device__ __forceinline__ void row_softmax(const pack<T, EPV> (&rx)[VPL], const pack<uint8_t, EPV> (&rk)[VPL],
                                            bool masked, int cols, int lane, float (&v)[VPL][EPV]) {
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = row_col<EPV>(i, lane);
    if (col < cols) {
      unpack_raw<T, EPV>(rx[i], v[i]);
      if (masked) {
#pragma unroll
        for (int j = 0; j < EPV; ++j) if (rk[i].v[j]) v[i][j] = -INFINITY;
      }
#pragma unroll
      for (int j = 0; j < EPV; ++j) mx = fmaxf(mx, v[i][j]);
    } else {
#pragma unroll
      for (int j = 0; j < EPV; ++j) v[i][j] = -INFINITY;
    }
  }
  mx = wave_max(mx);
  const float base = (mx == -INFINITY) ? 0.f : mx;
  float sum = 0.f;
  constexpr float LOG2E = 1.4426950408889634f;
#pragma unroll
  for (int i = 0; i < VPL; ++i)
#pragma unroll
    for (int j = 0; j < EPV; ++j) { v[i][j] = __builtin_amdgcn_exp2f((v[i][j] - base) * LOG2E); sum += v[i][j]; }   // argument <= 0
  sum = wave_sum(sum);
  const float inv = sum > 0.f ? 1.f / sum : 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i)
#pragma unroll
    for (int j = 0; j < EPV; ++j) v[i][j] *= inv;
}

// A wavefront owns RPW consecutive rows: the loads of all of them are issued before the first is used, so that the
// bytes in flight per wavefront (and with them the bandwidth of a kernel whose wavefronts otherwise wait out one
// memory latency per row) grow RPW-fold; the rows are then normalised and stored one after the other.
// RNG (the keep mask is drawn here from Philox and stored) is a compile-time switch: as a run-time branch the
// generator's ~200 integer instructions per 8 elements were scheduled ahead of the branch and ran in every mode,
// which made the kernel instruction-bound (about 290 vector instructions per 512-key row instead of about 90).
// REL: the scores are the sum of the content term (a.in) and the shifted position term (a.bd); the sum, rounded to T as
// a separate addition would round it, is stored to a.scores_out for the backward and is what the softmax sees. The
// shifted operand is not aligned with the row, so it is read element by element (consecutive lanes, consecutive
// addresses) and turned into the row's register layout through LDS.
template <typename T, int EPV, int VPL, int RPW, bool RNG, bool REL = false>
__global__ __launch_bounds__(SM_THREADS) void softmax_fwd_kernel(SoftmaxArgs a) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * SM_WAVES + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave)) * RPW;
  if (row0 >= a.rows) return;
  const bool mask_in = !RNG && a.dropout_mode == SM_MASK_IN;
  const bool masked = a.kmask_kind != SM_NOMASK;
  pack<T, EPV> rx[RPW][VPL];
  [[maybe_unused]] pack<T, VPL * EPV> rb[REL ? RPW : 1];
  [[maybe_unused]] __shared__ __align__(16) T stage_all[REL ? SM_WAVES * RPW * EPV * VPL * kWave : 1];
  pack<uint8_t, EPV> rk[RPW][VPL] = {}, rd[RPW][VPL] = {};
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int64_t row = min(row0 + r, a.rows - 1);     // rows past the end: loaded again, not used
    row_load<T, EPV, VPL>(static_cast<const T*>(a.in) + row * a.cols, a.cols, lane, rx[r]);
    if (masked) row_load<uint8_t, EPV, VPL>(kmask_row(a, row), a.cols, lane, rk[r]);
    if (mask_in) row_load<uint8_t, EPV, VPL>(a.dmask + row * a.cols, a.cols, lane, rd[r]);
    if constexpr (REL) {
      // lane l takes elements l, 64 + l, ... of the shifted row: consecutive lanes read consecutive addresses
      const RelRow rr = rel_row(row, a.q_len, a.len_r);
      const T* src = static_cast<const T*>(a.bd) + rr.first;
#pragma unroll
      for (int k = 0; k < VPL * EPV; ++k) {
        const int e = k * kWave + lane;
        const int at = e < a.cols ? rel_source(rr.c0 + e, a.len_r) : -1;
        rb[r].v[k] = at >= 0 ? src[at] : elem<T>::from_float(0.f);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) { row_pin(rx[r]); row_pin(rk[r]); row_pin(rd[r]); }
  if constexpr (REL) {
    // through the wavefront's strips of LDS into the layout of the other operands (lane l: elements EPV l ...)
    T* strip = stage_all + (threadIdx.x / kWave) * (RPW * EPV * VPL * kWave);
#pragma unroll
    for (int r = 0; r < RPW; ++r)
#pragma unroll
      for (int k = 0; k < VPL * EPV; ++k) strip[r * (EPV * VPL * kWave) + k * kWave + lane] = rb[r].v[k];
    wave_lds_fence();
  }
  [[maybe_unused]] const Philox gen(a.seed);
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    if (row0 + r >= a.rows) break;
    const int64_t base = (row0 + r) * a.cols;
    if constexpr (REL) {
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int col = row_col<EPV>(i, lane);
        if (col < a.cols) {
          float x[EPV], sh[EPV];
          unpack_raw<T, EPV>(rx[r][i], x);
          load_pack<T, EPV>(stage_all + ((threadIdx.x / kWave) * RPW + r) * (EPV * VPL * kWave) + col, sh);
#pragma unroll
          for (int u = 0; u < EPV; ++u) rx[r][i].v[u] = elem<T>::from_float(x[u] + sh[u]);
          *reinterpret_cast<pack<T, EPV>*>(static_cast<T*>(a.scores_out) + base + col) = rx[r][i];
        }
      }
    }
    float v[VPL][EPV];
    row_softmax<T, EPV, VPL>(rx[r], rk[r], masked, a.cols, lane, v);
    T* out = static_cast<T*>(a.out) + base;
    T* out_sm = a.out_softmax ? static_cast<T*>(a.out_softmax) + base : nullptr;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = row_col<EPV>(i, lane);
      if (col < a.cols) {
        if (out_sm) store_pack<T, EPV>(out_sm + col, v[i]);
        if (a.dropout_mode != SM_NO_DROPOUT) {
          uint8_t keep[EPV];
          if constexpr (RNG) {
            philox_keep<EPV>(gen, static_cast<uint64_t>(base + col), a.offset, a.keep_p, keep);
            store_bytes<EPV>(a.dmask + base + col, keep);
          } else {
#pragma unroll
            for (int j = 0; j < EPV; ++j) keep[j] = rd[r][i].v[j];
          }
#pragma unroll
          for (int j = 0; j < EPV; ++j) v[i][j] = keep[j] ? v[i][j] * a.scale : 0.f;
        }
        store_pack<T, EPV>(out + col, v[i]);
      }
    }
  }
}

// dS = P * (g - sum_k P * g), g = keep * dP / (1 - p).
// REL: the score gradient also leaves through the adjoint of the relative shift (relative_self_attention_func.py:52-76
// of the reference), as grad_bd [batch, q_len, len_r]. Row i of the scores owns the padded elements from its own first
// one up to the next row's first one (row 0 also those in front of it): its len_k gradients, then zeros. The
// destinations are not aligned with the row either, so the row goes through the wavefront's strip of LDS and is
// stored element by element, consecutive lanes to consecutive addresses.
template <typename T, int EPV, int VPL, int RPW, bool REL = false>
__global__ __launch_bounds__(SM_THREADS) void softmax_bwd_kernel(SoftmaxArgs a) {
  [[maybe_unused]] __shared__ __align__(16) T stage_all[REL ? SM_WAVES * EPV * VPL * kWave : 1];
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * SM_WAVES + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave)) * RPW;
  if (row0 >= a.rows) return;
  const bool masked = a.from_scores && a.kmask_kind != SM_NOMASK;
  const bool dropped = a.dropout_mode != SM_NO_DROPOUT;
  pack<T, EPV> rs[RPW][VPL], rg[RPW][VPL];
  pack<uint8_t, EPV> rk[RPW][VPL] = {}, rd[RPW][VPL] = {};
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int64_t row = min(row0 + r, a.rows - 1);
    row_load<T, EPV, VPL>(static_cast<const T*>(a.saved) + row * a.cols, a.cols, lane, rs[r]);
    row_load<T, EPV, VPL>(static_cast<const T*>(a.in) + row * a.cols, a.cols, lane, rg[r]);
    if (masked) row_load<uint8_t, EPV, VPL>(kmask_row(a, row), a.cols, lane, rk[r]);
    if (dropped) row_load<uint8_t, EPV, VPL>(a.dmask + row * a.cols, a.cols, lane, rd[r]);
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) { row_pin(rs[r]); row_pin(rg[r]); row_pin(rk[r]); row_pin(rd[r]); }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    if (row0 + r >= a.rows) break;
    float pr[VPL][EPV], g[VPL][EPV];
    if (a.from_scores) {
      row_softmax<T, EPV, VPL>(rs[r], rk[r], masked, a.cols, lane, pr);
    } else {
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        if (row_col<EPV>(i, lane) < a.cols) unpack_raw<T, EPV>(rs[r][i], pr[i]);
        else {
#pragma unroll
          for (int j = 0; j < EPV; ++j) pr[i][j] = 0.f;
        }
      }
    }
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      if (row_col<EPV>(i, lane) < a.cols) {
        unpack_raw<T, EPV>(rg[r][i], g[i]);
        if (dropped) {
#pragma unroll
          for (int j = 0; j < EPV; ++j) g[i][j] = rd[r][i].v[j] ? g[i][j] * a.scale : 0.f;
        }
#pragma unroll
        for (int j = 0; j < EPV; ++j) dot += pr[i][j] * g[i][j];
      } else {
#pragma unroll
        for (int j = 0; j < EPV; ++j) g[i][j] = 0.f;
      }
    }
    dot = wave_sum(dot);
    T* out = static_cast<T*>(a.out) + (row0 + r) * a.cols;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int col = row_col<EPV>(i, lane);
      if (col < a.cols) {
#pragma unroll
        for (int j = 0; j < EPV; ++j) g[i][j] = pr[i][j] * (g[i][j] - dot);
        store_pack<T, EPV>(out + col, g[i]);
        if constexpr (REL) store_pack<T, EPV>(stage_all + (threadIdx.x / kWave) * (EPV * VPL * kWave) + col, g[i]);
      }
    }
    if constexpr (REL) {
      const T* stage = stage_all + (threadIdx.x / kWave) * (EPV * VPL * kWave);
      const uint32_t len_r = a.len_r, q_len = a.q_len;
      const RelRow rr = rel_row(row0 + r, q_len, len_r);
      T* dst = static_cast<T*>(a.grad_bd) + rr.first;
      wave_lds_fence();                                  // the strip is written and read by different lanes
      for (uint32_t j = lane; j < len_r; j += kWave) {   // the row's gradients, then zeros up to the next row's start
        const int at = rel_source(rr.c0 + j, len_r);
        if (at >= 0) dst[at] = j < static_cast<uint32_t>(a.cols) ? stage[j] : elem<T>::from_float(0.f);
      }
      if (rr.i == 0) {                                   // the padded elements in front of row 0
        T* head = static_cast<T*>(a.grad_bd) + (row0 + r) * static_cast<int64_t>(len_r);
        for (uint32_t p = lane; p < q_len; p += kWave) {
          const uint32_t i2 = p / (len_r + 1);
          if (p != i2 * (len_r + 1)) head[p - i2 - 1] = elem<T>::from_float(0.f);
        }
      }
      wave_lds_fence();                                  // before the next row overwrites the strip
    }
  }
}

// Vector width: the widest of 16 / 8 / 4 / 2-byte accesses that every row start and the masks
// allow, narrowed further for short rows so that all 64 lanes hold data.
template <typename T>
int pick_epv(const SoftmaxArgs& a, bool bwd) {
  constexpr int WIDE = 16 / sizeof(T);
  int epv = WIDE;
  auto ok = [&](int e) {
    if (a.cols % e) return false;
    const uintptr_t bytes = static_cast<uintptr_t>(e) * sizeof(T);
    auto al = [&](const void* p, uintptr_t b) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % b) == 0; };
    if (!al(a.in, bytes) || !al(a.out, bytes) || !al(a.saved, bytes) || !al(a.out_softmax, bytes)) return false;
    if (!al(a.dmask, e) || !al(a.kmask, e)) return false;
    (void)bwd;
    return true;
  };
  while (epv > 1 && !ok(epv)) epv /= 2;
  while (epv > 2 && a.cols < epv * kWave) epv /= 2;  // short rows: spread over more lanes
  return epv;
}

template <typename T>
int softmax_launch(const SoftmaxArgs& a, bool bwd, hipStream_t st) {
  const int epv = pick_epv<T>(a, bwd);
  const int vecs = (a.cols + epv - 1) / epv;
  int vpl = 1;
  while (vpl * kWave < vecs) vpl *= 2;
  // rows per wavefront: as many as keep the raw loads of a wavefront within about 32 registers per operand
  bool done = false;
  const bool rng = !bwd && a.dropout_mode == SM_MASK_RNG;
  TraceScope trace(bwd ? "softmax_dropout_bwd" : "softmax_dropout_fwd", st);
#define SM_CASE(E, V)                                                                                             \
  if (!done && epv == E && vpl == V) {                                                                            \
    constexpr int R = V == 1 ? 4 : V == 2 ? 2 : 1;                                                                \
    const unsigned grid = static_cast<unsigned>((a.rows + SM_WAVES * R - 1) / (SM_WAVES * R));                    \
    if (bwd) hipLaunchKernelGGL((softmax_bwd_kernel<T, E, V, R>), dim3(grid), dim3(SM_THREADS), 0, st, a);        \
    else if (rng) hipLaunchKernelGGL((softmax_fwd_kernel<T, E, V, R, true>), dim3(grid), dim3(SM_THREADS), 0, st, a);  \
    else hipLaunchKernelGGL((softmax_fwd_kernel<T, E, V, R, false>), dim3(grid), dim3(SM_THREADS), 0, st, a);     \
    done = true;                                                                                                  \
  }
  if constexpr (sizeof(T) == 2) { SM_CASE(8, 1) SM_CASE(8, 2) SM_CASE(8, 4) SM_CASE(8, 8) }
  SM_CASE(4, 1) SM_CASE(4, 2) SM_CASE(4, 4) SM_CASE(4, 8) SM_CASE(4, 16)
  SM_CASE(2, 1) SM_CASE(2, 2) SM_CASE(2, 4) SM_CASE(2, 8) SM_CASE(2, 16)
  SM_CASE(1, 1) SM_CASE(1, 2) SM_CASE(1, 4) SM_CASE(1, 8) SM_CASE(1, 16) SM_CASE(1, 32)
#undef SM_CASE
  if (!done)
    return fail(NMTG_ERR_UNSUPPORTED,
                "softmax: row length %d is beyond what one wavefront holds at vector width %d "
                "(limit 4096 keys for aligned 16-bit rows, 2048 otherwise)", a.cols, epv);
  return 0;
}

// The relative-position kernels exist at full vector width only (rows of a multiple of 16 bytes).
template <typename T>
int softmax_rel_launch(const SoftmaxArgs& a, bool bwd, hipStream_t st) {
  constexpr int E = 16 / sizeof(T);
  const int vecs = a.cols / E;
  int vpl = 1;
  while (vpl * kWave < vecs) vpl *= 2;
  const bool rng = !bwd && a.dropout_mode == SM_MASK_RNG;
  TraceScope trace(bwd ? "rel_softmax_dropout_bwd" : "rel_softmax_dropout_fwd", st);
  bool done = false;
#define REL_CASE(V)                                                                                                     \
  if (!done && vpl == V) {                                                                                              \
    constexpr int R = V == 1 ? 4 : V == 2 ? 2 : 1;                                                                      \
    const unsigned grid = static_cast<unsigned>((a.rows + SM_WAVES * R - 1) / (SM_WAVES * R));                          \
    if (bwd) hipLaunchKernelGGL((softmax_bwd_kernel<T, E, V, R, true>), dim3(grid), dim3(SM_THREADS), 0, st, a);        \
    else if (rng) hipLaunchKernelGGL((softmax_fwd_kernel<T, E, V, R, true, true>), dim3(grid), dim3(SM_THREADS), 0, st, a);  \
    else hipLaunchKernelGGL((softmax_fwd_kernel<T, E, V, R, false, true>), dim3(grid), dim3(SM_THREADS), 0, st, a);     \
    done = true;                                                                                                        \
  }
  REL_CASE(1) REL_CASE(2) REL_CASE(4) REL_CASE(8)
#undef REL_CASE
  if (!done) return fail(NMTG_ERR_UNSUPPORTED, "rel_softmax_dropout: %d keys are beyond what one wavefront holds (%d)", a.cols, 8 * kWave * E);
  return 0;
}

int check_rel(const char* who, const void* const* ptrs, int n_ptrs, int64_t batch, int64_t len_q, int64_t len_k, int64_t len_r, int dtype) {
  NMTG_REQUIRE(batch >= 0 && len_q >= 0 && len_k > 0 && len_r >= len_k, "%s: bad shape batch=%lld len_q=%lld len_k=%lld len_r=%lld (len_r >= len_k)",
               who, (long long)batch, (long long)len_q, (long long)len_k, (long long)len_r);
  NMTG_REQUIRE(len_q * (len_r + 1) < (int64_t{1} << 31) && batch * len_q < (int64_t{1} << 31),
               "%s: sizes beyond the kernel's 32-bit indices (len_q * (len_r + 1) and batch * len_q below 2^31)", who);
  const int wide = dtype == NMTG_F32 ? 4 : 8;
  NMTG_REQUIRE(len_k % wide == 0, "%s: len_k = %lld is not a multiple of %d elements (use the separate shift and softmax calls)", who,
               (long long)len_k, wide);
  for (int k = 0; k < n_ptrs; ++k) NMTG_REQUIRE(aligned16(ptrs[k]), "%s: 16-byte aligned tensors required", who);
  return 0;
}

int check_common(const char* who, const SoftmaxArgs& a, float p) {
  NMTG_REQUIRE(a.rows >= 0 && a.cols > 0, "%s: bad shape rows=%lld cols=%d", who, (long long)a.rows, a.cols);
  NMTG_REQUIRE(a.dropout_mode >= SM_NO_DROPOUT && a.dropout_mode <= SM_MASK_RNG, "%s: bad dropout_mode", who);
  NMTG_REQUIRE(a.kmask_kind >= SM_NOMASK && a.kmask_kind <= SM_TIME, "%s: bad mask_kind", who);
  if (a.kmask_kind != SM_NOMASK) {
    NMTG_REQUIRE(a.kmask != nullptr, "%s: mask_kind set but mask pointer is null", who);
    NMTG_REQUIRE(a.q_len > 0 && a.heads > 0, "%s: q_len and heads must be positive with a mask", who);
    NMTG_REQUIRE(a.rows % (static_cast<int64_t>(a.q_len) * (a.kmask_kind == SM_PAD ? a.heads : 1)) == 0,
                 "%s: rows is not a multiple of %s", who, a.kmask_kind == SM_PAD ? "heads*q_len" : "q_len");
  }
  if (a.dropout_mode != SM_NO_DROPOUT) {
    NMTG_REQUIRE(a.dmask != nullptr, "%s: dropout mask buffer required", who);
    NMTG_REQUIRE(p >= 0.f && p < 1.f, "%s: dropout probability %f outside [0, 1)", who, p);
  }
  return 0;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_softmax_dropout_fwd(const void* scores, const uint8_t* key_mask, int mask_kind, void* softmax_out,
                                        void* dropped_out, uint8_t* dropout_mask, int dropout_mode, float p,
                                        uint64_t seed, uint64_t offset, int64_t rows, int64_t cols, int64_t q_len,
                                        int64_t heads, int dtype, void* stream) {
  NMTG_REQUIRE(cols > 0 && cols <= (1 << 20) && q_len <= INT32_MAX && heads <= INT32_MAX,
               "softmax_dropout_fwd: bad shape cols=%lld", (long long)cols);
  SoftmaxArgs a{};
  a.in = scores; a.out = dropped_out; a.out_softmax = softmax_out; a.dmask = dropout_mask; a.kmask = key_mask;
  a.rows = rows; a.cols = static_cast<int>(cols); a.q_len = static_cast<int>(q_len); a.heads = static_cast<int>(heads);
  a.kmask_kind = mask_kind; a.dropout_mode = dropout_mode;
  a.keep_p = 1.f - p; a.scale = 1.f / (1.f - p); a.seed = seed; a.offset = offset;
  if (int rc = check_common("softmax_dropout_fwd", a, p)) return rc;
  if (rows == 0) return 0;
  NMTG_REQUIRE(scores && dropped_out, "softmax_dropout_fwd: null pointer argument");
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = softmax_launch<T>(a, false, static_cast<hipStream_t>(stream)));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("softmax_dropout_fwd");
  return 0;
}

extern "C" int nmtg_softmax_dropout_bwd(const void* grad_dropped, const void* saved, int saved_is_scores,
                                        const uint8_t* key_mask, int mask_kind, const uint8_t* dropout_mask,
                                        int dropout_mode, float p, void* grad_scores, int64_t rows, int64_t cols,
                                        int64_t q_len, int64_t heads, int dtype, void* stream) {
  NMTG_REQUIRE(cols > 0 && cols <= (1 << 20) && q_len <= INT32_MAX && heads <= INT32_MAX,
               "softmax_dropout_bwd: bad shape cols=%lld", (long long)cols);
  NMTG_REQUIRE(dropout_mode != SM_MASK_RNG, "softmax_dropout_bwd: the backward replays a stored mask (mode 0 or 1)");
  SoftmaxArgs a{};
  a.in = grad_dropped; a.saved = saved; a.out = grad_scores; a.dmask = const_cast<uint8_t*>(dropout_mask);
  a.kmask = key_mask; a.rows = rows; a.cols = static_cast<int>(cols); a.q_len = static_cast<int>(q_len);
  a.heads = static_cast<int>(heads); a.kmask_kind = saved_is_scores ? mask_kind : SM_NOMASK;
  a.dropout_mode = dropout_mode; a.from_scores = saved_is_scores ? 1 : 0;
  a.keep_p = 1.f - p; a.scale = 1.f / (1.f - p);
  if (int rc = check_common("softmax_dropout_bwd", a, p)) return rc;
  if (rows == 0) return 0;
  NMTG_REQUIRE(grad_dropped && saved && grad_scores, "softmax_dropout_bwd: null pointer argument");
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = softmax_launch<T>(a, true, static_cast<hipStream_t>(stream)));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("softmax_dropout_bwd");
  return 0;
}


extern "C" int nmtg_rel_softmax_dropout_fwd(void* scores, const void* bd, int64_t len_r, const uint8_t* key_mask, int mask_kind,
                                            void* dropped_out, uint8_t* dropout_mask, int dropout_mode, float p, uint64_t seed,
                                            uint64_t offset, int64_t batch, int64_t len_q, int64_t len_k, int64_t heads, int dtype,
                                            void* stream) {
  const void* ptrs[] = {scores, bd, dropped_out};
  if (int rc = check_rel("rel_softmax_dropout_fwd", ptrs, 3, batch, len_q, len_k, len_r, dtype)) return rc;
  NMTG_REQUIRE(heads >= 0 && heads <= INT32_MAX, "rel_softmax_dropout_fwd: bad heads");
  SoftmaxArgs a{};
  a.in = scores; a.scores_out = scores; a.bd = bd; a.len_r = static_cast<int>(len_r);
  a.out = dropped_out; a.dmask = dropout_mask; a.kmask = key_mask;
  a.rows = batch * len_q; a.cols = static_cast<int>(len_k); a.q_len = static_cast<int>(len_q); a.heads = static_cast<int>(heads);
  a.kmask_kind = mask_kind; a.dropout_mode = dropout_mode;
  a.keep_p = 1.f - p; a.scale = 1.f / (1.f - p); a.seed = seed; a.offset = offset;
  if (a.rows == 0) return 0;
  if (int rc = check_common("rel_softmax_dropout_fwd", a, p)) return rc;
  NMTG_REQUIRE(scores && bd && dropped_out, "rel_softmax_dropout_fwd: null pointer argument");
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = softmax_rel_launch<T>(a, false, static_cast<hipStream_t>(stream)));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("rel_softmax_dropout_fwd");
  return 0;
}

extern "C" int nmtg_rel_softmax_dropout_bwd(const void* grad_dropped, const void* scores, const uint8_t* key_mask, int mask_kind,
                                            const uint8_t* dropout_mask, int dropout_mode, float p, void* grad_scores,
                                            void* grad_bd, int64_t len_r, int64_t batch, int64_t len_q, int64_t len_k,
                                            int64_t heads, int dtype, void* stream) {
  const void* ptrs[] = {grad_dropped, scores, grad_scores, grad_bd};
  if (int rc = check_rel("rel_softmax_dropout_bwd", ptrs, 4, batch, len_q, len_k, len_r, dtype)) return rc;
  NMTG_REQUIRE(heads >= 0 && heads <= INT32_MAX, "rel_softmax_dropout_bwd: bad heads");
  NMTG_REQUIRE(dropout_mode != SM_MASK_RNG, "rel_softmax_dropout_bwd: the backward replays a stored mask (mode 0 or 1)");
  SoftmaxArgs a{};
  a.in = grad_dropped; a.saved = scores; a.out = grad_scores; a.grad_bd = grad_bd; a.len_r = static_cast<int>(len_r);
  a.dmask = const_cast<uint8_t*>(dropout_mask); a.kmask = key_mask;
  a.rows = batch * len_q; a.cols = static_cast<int>(len_k); a.q_len = static_cast<int>(len_q); a.heads = static_cast<int>(heads);
  a.kmask_kind = mask_kind; a.dropout_mode = dropout_mode; a.from_scores = 1;
  a.keep_p = 1.f - p; a.scale = 1.f / (1.f - p);
  if (a.rows == 0) return 0;
  if (int rc = check_common("rel_softmax_dropout_bwd", a, p)) return rc;
  NMTG_REQUIRE(grad_dropped && scores && grad_scores && grad_bd, "rel_softmax_dropout_bwd: null pointer argument");
  int rc = 0;
  NMTG_DISPATCH_DTYPE(dtype, T, rc = softmax_rel_launch<T>(a, true, static_cast<hipStream_t>(stream)));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("rel_softmax_dropout_bwd");
  return 0;
}
