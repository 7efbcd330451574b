// Label-smoothed softmax cross-entropy over large vocabularies, forward and backward, gfx950.
//
// Stands in for xentropy_cuda.forward / backward of the reference
// (onmt/modules/extensions/xentropy/xentropy_kernel.cu:382-474 kernels, :571-718 host side,
// interface.cpp:24-47) plus the padding handling its Python wrapper does afterwards with
// masked_fill_ (onmt/modules/optimized/softmax_xentropy.py:10,24), which is fused here.
//
//   lse_i  = max_j x_ij + log sum_j exp(x_ij - max)
//   loss_i = eps (lse_i - mean_j x_ij) + (1 - eps)(lse_i - x_{i,y_i});   0 if y_i == padding_idx
//   dx_ij  = g_i (exp(x_ij - lse_i) - (1 - eps)[j == y_i] - eps / V);    0 if y_i == padding_idx
//
// One block per row. The forward makes ONE pass over the row (the reference makes two): every
// lane keeps an online (max, sum-exp) pair plus the plain sum, merged across the block at the end.
// Rows are not 16-byte aligned in general (V * sizeof(T) need not be a multiple of 16): each row is
// split into a scalar head up to the first 16-byte boundary, a body of 16-byte vectors and a
// scalar tail. All indexing is 64-bit (N * V exceeds 2^31 at the benchmark shape).
//
// Bandwidth bound: forward reads N*V elements once; backward reads them once and writes N*V
// (rows whose label is the padding index are written as zeros without reading the logits).
#include "common.hip.h"

namespace nmtg {
namespace {

constexpr int XE_THREADS = 1024;
constexpr int XE_WAVES = XE_THREADS / kWave;
// 16-byte loads a lane keeps in flight in the streaming loops: one load per trip leaves 16 bytes per lane in flight,
// which at two 1024-thread blocks per CU (32 KB) is less than the memory latency needs at full bandwidth
constexpr int XE_INFLIGHT = 4;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
// start value of the running maximum: below every finite logit, and small enough in magnitude that NEG_BIG * LOG2E is
// still finite (a lane that has only seen -inf logits must not turn them into NaN)
constexpr float NEG_BIG = -1.0e30f;

struct Online {
  float m, s;  // running max and sum of exp(x - m)
};
__device__ __forceinline__ Online merge(Online a, Online b) {
  const float m = fmaxf(a.m, b.m);
  Online r;
  r.m = m;
  r.s = a.s * exp2f((a.m - m) * LOG2E) + b.s * exp2f((b.m - m) * LOG2E);
  return r;
}

template <int N>
__device__ __forceinline__ void online_add(Online& st, float& sx, const float (&v)[N]) {
  float cm = v[0];
#pragma unroll
  for (int j = 1; j < N; ++j) cm = fmaxf(cm, v[j]);
  if (cm > st.m) {
    st.s *= exp2f((st.m - cm) * LOG2E);
    st.m = cm;
  }
  const float mb = st.m * LOG2E;
  float acc = 0.f, sum = 0.f;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    // bare v_exp_f32: terms below 2^-126 of the running maximum flush to zero, which a sum of at least one
    // term equal to 1 cannot notice; the library exp2f spends four more instructions per element on that
    // range, and the forward pass is as much VALU- as HBM-bound (one exponential per 2 bytes read)
    acc += __builtin_amdgcn_exp2f(fmaf(v[j], LOG2E, -mb));
    sum += v[j];
  }
  st.s += acc;
  sx += sum;
}

// Running argmax with torch.argmax's rule: the largest value, NaN counting as larger than everything, and the lowest
// index among equals (bf16 logits tie all the time, so the rule decides most rows).
struct Best {
  float v;
  int64_t i;
};
__device__ __forceinline__ bool better(float v, int64_t i, const Best& b) {
  const bool vn = v != v, bn = b.v != b.v;
  if (vn || bn) return vn && (!bn || i < b.i);
  return v > b.v || (v == b.v && i < b.i);
}
__device__ __forceinline__ void best_add(Best& b, float v, int64_t i) {
  if (better(v, i, b)) { b.v = v; b.i = i; }
}

// ARGMAX: also writes the index of each row's largest logit (the evaluation branch of the loss counts correct
// predictions from it, onmt/modules/loss.py:293-311); its own instantiation, the training forward pays nothing for it.
template <typename T, bool ARGMAX>
__global__ __launch_bounds__(XE_THREADS) void xentropy_fwd_kernel(
    const T* __restrict__ logits, const int64_t* __restrict__ labels, float* __restrict__ losses,
    float* __restrict__ lse_out, int64_t* __restrict__ argmax_out, int64_t vocab, int64_t ld, float smoothing,
    int64_t padding_idx) {
  constexpr int EPV = 16 / sizeof(T);
  __shared__ float sm_m[XE_WAVES], sm_s[XE_WAVES], sm_x[XE_WAVES];
  __shared__ float sm_bv[ARGMAX ? XE_WAVES : 1];
  __shared__ int64_t sm_bi[ARGMAX ? XE_WAVES : 1];
  Best best{-INFINITY, INT64_MAX};
  const int64_t row = blockIdx.x;
  const T* x = logits + row * ld;
  const int tid = threadIdx.x;

  const uintptr_t addr = reinterpret_cast<uintptr_t>(x);
  int64_t head = static_cast<int64_t>(((16 - (addr & 15)) & 15) / sizeof(T));
  if (head > vocab) head = vocab;
  const int64_t nvec = (vocab - head) / EPV;
  const int64_t tail0 = head + nvec * EPV;

  Online st{NEG_BIG, 0.f};
  float sx = 0.f;
  if (tid < head) {
    float v[1] = {elem<T>::to_float(x[tid])};
    online_add<1>(st, sx, v);
    if constexpr (ARGMAX) best_add(best, v[0], tid);
  }
  const T* body = x + head;
  int64_t i = tid;
  // XE_INFLIGHT vectors in flight per lane per trip: all loads are issued (and pinned) before the first is used; the
  // vectors are consumed in the same order as one at a time
  for (; i + (XE_INFLIGHT - 1) * XE_THREADS < nvec; i += XE_INFLIGHT * XE_THREADS) {
    pack<T, EPV> raw[XE_INFLIGHT];
#pragma unroll
    for (int u = 0; u < XE_INFLIGHT; ++u) raw[u] = load_raw<T, EPV>(body + (i + u * XE_THREADS) * EPV);
#pragma unroll
    for (int u = 0; u < XE_INFLIGHT; ++u) pin_raw(raw[u]);
#pragma unroll
    for (int u = 0; u < XE_INFLIGHT; ++u) {
      float a[EPV];
      unpack_raw<T, EPV>(raw[u], a);
      online_add<EPV>(st, sx, a);
      if constexpr (ARGMAX) {
#pragma unroll
        for (int j = 0; j < EPV; ++j) best_add(best, a[j], head + (i + u * XE_THREADS) * EPV + j);
      }
    }
  }
  for (; i < nvec; i += XE_THREADS) {
    float a[EPV];
    load_pack<T, EPV>(body + i * EPV, a);
    online_add<EPV>(st, sx, a);
    if constexpr (ARGMAX) {
#pragma unroll
      for (int j = 0; j < EPV; ++j) best_add(best, a[j], head + i * EPV + j);
    }
  }
  if (tail0 + tid < vocab) {
    float v[1] = {elem<T>::to_float(x[tail0 + tid])};
    online_add<1>(st, sx, v);
    if constexpr (ARGMAX) best_add(best, v[0], tail0 + tid);
  }

  // wavefront merge, then across the block's wavefronts
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    Online o{__shfl_xor(st.m, m, 64), __shfl_xor(st.s, m, 64)};
    st = merge(st, o);
    sx += __shfl_xor(sx, m, 64);
    if constexpr (ARGMAX) {
      const float ov = __shfl_xor(best.v, m, 64);
      const int64_t oi = __shfl_xor(best.i, m, 64);
      best_add(best, ov, oi);
    }
  }
  const int wave = tid / kWave, lane = tid & (kWave - 1);
  if (lane == 0) {
    sm_m[wave] = st.m; sm_s[wave] = st.s; sm_x[wave] = sx;
    if constexpr (ARGMAX) { sm_bv[wave] = best.v; sm_bi[wave] = best.i; }
  }
  __syncthreads();
  if (tid == 0) {
    if constexpr (ARGMAX) {
      Best b{sm_bv[0], sm_bi[0]};
      for (int w = 1; w < XE_WAVES; ++w) best_add(b, sm_bv[w], sm_bi[w]);
      argmax_out[row] = b.i;
    }
    Online tot{sm_m[0], sm_s[0]};
    float tx = sm_x[0];
#pragma unroll
    for (int w = 1; w < XE_WAVES; ++w) { tot = merge(tot, Online{sm_m[w], sm_s[w]}); tx += sm_x[w]; }
    const float lse = tot.m + log2f(tot.s) * LN2;
    const int64_t y = labels[row];
    float loss = 0.f;
    if (y != padding_idx) {
      const float xy = (y >= 0 && y < vocab) ? elem<T>::to_float(x[y]) : 0.f;
      loss = (1.f - smoothing) * (lse - xy);
      // without smoothing the mean logit does not enter (it is -inf when a class is masked out, and 0 * inf is NaN)
      if (smoothing != 0.f) loss += smoothing * (lse - tx / static_cast<float>(vocab));
    }
    losses[row] = loss;
    lse_out[row] = lse;
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(XE_THREADS) void xentropy_bwd_kernel(
    const float* __restrict__ grad_loss, const T* logits, const float* __restrict__ lse_in,
    const int64_t* __restrict__ labels, T* grad_logits, int64_t vocab, int64_t ld, int64_t ld_grad,
    int64_t class_offset, int64_t total_classes, float smoothing, int64_t padding_idx) {
  constexpr int EPV = 16 / sizeof(T);
  const int64_t row = blockIdx.x;
  const T* x = logits + row * ld;
  T* dx = grad_logits + row * ld_grad;
  const int tid = threadIdx.x;
  // the row holds classes [class_offset, class_offset + vocab) of total_classes: y is the label's position in the row
  // (outside [0, vocab) if the label belongs to another slice)
  const bool padded = labels[row] == padding_idx;
  const int64_t y = labels[row] - class_offset;
  const float g = padded ? 0.f : grad_loss[row];

  const uintptr_t addr = reinterpret_cast<uintptr_t>(dx);
  int64_t head = VEC ? static_cast<int64_t>(((16 - (addr & 15)) & 15) / sizeof(T)) : vocab;
  if (head > vocab) head = vocab;
  const int64_t nvec = (vocab - head) / EPV;
  const int64_t tail0 = head + nvec * EPV;

  if (padded) {  // exact zeros, logits untouched
    for (int64_t c = tid; c < head; c += XE_THREADS) dx[c] = elem<T>::from_float(0.f);
    const float z[EPV] = {};
    for (int64_t i = tid; i < nvec; i += XE_THREADS) store_pack<T, EPV>(dx + head + i * EPV, z);
    for (int64_t c = tail0 + tid; c < vocab; c += XE_THREADS) dx[c] = elem<T>::from_float(0.f);
    return;
  }

  const float nlse = -lse_in[row] * LOG2E;
  const float sm = smoothing / static_cast<float>(total_classes);
  const float onem = 1.f - smoothing;
  auto one = [&](int64_t c) {
    float v = __builtin_amdgcn_exp2f(fmaf(elem<T>::to_float(x[c]), LOG2E, nlse)) - sm;
    if (c == y) v -= onem;
    dx[c] = elem<T>::from_float(g * v);
  };
  for (int64_t c = tid; c < head; c += XE_THREADS) one(c);
  // one vector of the row: v holds the logits on entry
  auto finish = [&](int64_t c0, float (&v)[EPV]) {
    // the bare v_exp_f32: its argument is x - lse <= 0, and a probability below 2^-126 may as well be 0 (the library
    // exp2f spends four more instructions per element on keeping it a denormal; this kernel is close to VALU-bound)
#pragma unroll
    for (int j = 0; j < EPV; ++j) v[j] = __builtin_amdgcn_exp2f(fmaf(v[j], LOG2E, nlse)) - sm;
    if (y >= c0 && y < c0 + EPV) {
#pragma unroll
      for (int j = 0; j < EPV; ++j) if (c0 + j == y) v[j] -= onem;
    }
#pragma unroll
    for (int j = 0; j < EPV; ++j) v[j] *= g;
    store_pack<T, EPV>(dx + c0, v);
  };
  int64_t i = tid;
  // XE_INFLIGHT loads in flight per lane per trip (see the forward kernel)
  for (; i + (XE_INFLIGHT - 1) * XE_THREADS < nvec; i += XE_INFLIGHT * XE_THREADS) {
    pack<T, EPV> raw[XE_INFLIGHT];
#pragma unroll
    for (int u = 0; u < XE_INFLIGHT; ++u) raw[u] = load_raw<T, EPV>(x + head + (i + u * XE_THREADS) * EPV);
#pragma unroll
    for (int u = 0; u < XE_INFLIGHT; ++u) pin_raw(raw[u]);
#pragma unroll
    for (int u = 0; u < XE_INFLIGHT; ++u) {
      float v[EPV];
      unpack_raw<T, EPV>(raw[u], v);
      finish(head + (i + u * XE_THREADS) * EPV, v);
    }
  }
  for (; i < nvec; i += XE_THREADS) {
    const int64_t c0 = head + i * EPV;
    float v[EPV];
    load_pack<T, EPV>(x + c0, v);
    finish(c0, v);
  }
  for (int64_t c = tail0 + tid; c < vocab; c += XE_THREADS) one(c);
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

namespace {
int xentropy_fwd_run(const char* who, const void* logits, const int64_t* labels, float* losses, float* lse, int64_t* argmax,
                     bool want_argmax, int64_t rows, int64_t vocab, int64_t ld_logits, float smoothing, int64_t padding_idx,
                     int dtype, void* stream) {
  NMTG_REQUIRE(rows >= 0 && rows <= INT32_MAX, "%s: bad row count %lld", who, (long long)rows);
  NMTG_REQUIRE(vocab > 0, "%s: number of classes must be positive", who);
  NMTG_REQUIRE(ld_logits >= vocab, "%s: row pitch %lld is below the number of classes %lld", who,
               (long long)ld_logits, (long long)vocab);
  if (rows == 0) return 0;
  NMTG_REQUIRE(logits && labels && losses && lse && (!want_argmax || argmax), "%s: null pointer argument", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  TraceScope trace(want_argmax ? "xentropy_fwd_argmax" : "xentropy_fwd", st);
  NMTG_DISPATCH_DTYPE(
      dtype, T,
      if (want_argmax) hipLaunchKernelGGL((xentropy_fwd_kernel<T, true>), dim3(static_cast<unsigned>(rows)), dim3(XE_THREADS), 0, st,
                                          static_cast<const T*>(logits), labels, losses, lse, argmax, vocab, ld_logits, smoothing,
                                          padding_idx);
      else hipLaunchKernelGGL((xentropy_fwd_kernel<T, false>), dim3(static_cast<unsigned>(rows)), dim3(XE_THREADS), 0, st,
                              static_cast<const T*>(logits), labels, losses, lse, static_cast<int64_t*>(nullptr), vocab, ld_logits,
                              smoothing, padding_idx));
  NMTG_CHECK_LAUNCH(who);
  return 0;
}
}  // namespace

extern "C" int nmtg_xentropy_fwd(const void* logits, const int64_t* labels, float* losses, float* lse, int64_t rows,
                                 int64_t vocab, int64_t ld_logits, float smoothing, int64_t padding_idx, int dtype,
                                 void* stream) {
  return xentropy_fwd_run("xentropy_fwd", logits, labels, losses, lse, nullptr, false, rows, vocab, ld_logits, smoothing,
                          padding_idx, dtype, stream);
}

extern "C" int nmtg_xentropy_fwd_argmax(const void* logits, const int64_t* labels, float* losses, float* lse, int64_t* argmax,
                                        int64_t rows, int64_t vocab, int64_t ld_logits, float smoothing, int64_t padding_idx,
                                        int dtype, void* stream) {
  return xentropy_fwd_run("xentropy_fwd_argmax", logits, labels, losses, lse, argmax, true, rows, vocab, ld_logits, smoothing,
                          padding_idx, dtype, stream);
}

extern "C" int nmtg_xentropy_bwd(const float* grad_loss, const void* logits, const float* lse, const int64_t* labels,
                                 void* grad_logits, int64_t rows, int64_t vocab, int64_t ld_logits, int64_t ld_grad,
                                 int64_t class_offset, int64_t total_classes, float smoothing, int64_t padding_idx,
                                 int dtype, void* stream) {
  NMTG_REQUIRE(rows >= 0 && rows <= INT32_MAX, "xentropy_bwd: bad row count %lld", (long long)rows);
  NMTG_REQUIRE(vocab > 0, "xentropy_bwd: number of classes must be positive");
  NMTG_REQUIRE(ld_logits >= vocab && ld_grad >= vocab, "xentropy_bwd: a row pitch (%lld, %lld) is below the number of classes %lld",
               (long long)ld_logits, (long long)ld_grad, (long long)vocab);
  NMTG_REQUIRE(class_offset >= 0 && total_classes >= class_offset + vocab,
               "xentropy_bwd: classes [%lld, %lld) do not lie within %lld classes", (long long)class_offset,
               (long long)(class_offset + vocab), (long long)total_classes);
  if (rows == 0) return 0;
  NMTG_REQUIRE(grad_loss && logits && lse && labels && grad_logits, "xentropy_bwd: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Vector accesses need every logits row and its gradient row to share their 16-byte phase: the two bases do, and the
  // two pitches differ by a multiple of 16 bytes.
  const int64_t esize = dtype == NMTG_F32 ? 4 : 2;
  const bool vec = ((reinterpret_cast<uintptr_t>(logits) ^ reinterpret_cast<uintptr_t>(grad_logits)) & 15u) == 0 &&
                   ((ld_logits - ld_grad) * esize) % 16 == 0;
  TraceScope trace("xentropy_bwd", st);
  NMTG_DISPATCH_DTYPE(
      dtype, T,
      if (vec) hipLaunchKernelGGL((xentropy_bwd_kernel<T, true>), dim3(static_cast<unsigned>(rows)), dim3(XE_THREADS), 0, st,
                                  grad_loss, static_cast<const T*>(logits), lse, labels, static_cast<T*>(grad_logits), vocab,
                                  ld_logits, ld_grad, class_offset, total_classes, smoothing, padding_idx);
      else hipLaunchKernelGGL((xentropy_bwd_kernel<T, false>), dim3(static_cast<unsigned>(rows)), dim3(XE_THREADS), 0, st,
                              grad_loss, static_cast<const T*>(logits), lse, labels, static_cast<T*>(grad_logits), vocab,
                              ld_logits, ld_grad, class_offset, total_classes, smoothing, padding_idx));
  NMTG_CHECK_LAUNCH("xentropy_bwd");
  return 0;
}
