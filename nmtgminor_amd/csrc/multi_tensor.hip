// Optimizer-side elementwise passes over a LIST of tensors in one launch (per 48 tensors), for gfx950.
//
// Stand in for fused_optim.multi_tensor_adam / multi_tensor_scale / multi_tensor_axpby / multi_tensor_l2norm /
// multi_tensor_l2norm_scale of the reference
// (onmt/modules/extensions/fused_optim/frontend.cpp:45-53; kernels multi_tensor_adam.cu:22-129,
// multi_tensor_scale_kernel.cu:29-113, multi_tensor_axpby_kernel.cu:27-126, multi_tensor_l2norm_kernel.cu:27-232,
// multi_tensor_l2norm_scale_kernel.cu:28-125; launch machinery multi_tensor_apply.cuh).
// A model has hundreds of parameter tensors, most of them small: one launch per tensor would be launch-bound, so the
// tensors' addresses and sizes travel in the kernel arguments (a table of as many tensors as fit the 4 KB of kernel arguments: 84 for the four lists of an Adam step) and block b finds
// its tensor and its 32768-element chunk from the table's prefix of block counts. All three passes are bandwidth bound:
// Adam reads g, p, m, v and writes p, m, v (28 B per fp32 element), scale reads and writes once, the norm reads once.
// 16-byte accesses whenever a tensor's pointers are 16-byte aligned (chunks start on multiples of 32768 elements), with
// four loads in flight per lane in the Adam pass. fp32 arithmetic whatever the storage type. The norm is deterministic:
// one partial per block, then fixed-order sums.
#include "common.hip.h"

#include <algorithm>
#include <cmath>

namespace nmtg {
namespace {

// tensors per launch for a table of L pointer lists: 8 L + 12 bytes per tensor inside the 4 KB of kernel arguments,
// beside the kernel's scalars
template <int L> constexpr int mt_max() { return L >= 4 ? 84 : L == 3 ? 100 : L == 2 ? 128 : 160; }
constexpr int MT_CHUNK = 8192;      // elements per block
constexpr int MT_THREADS = 256;
constexpr int MT_WAVES = MT_THREADS / kWave;

template <int L>
struct MtTable {
  void* addr[L][mt_max<L>()];
  int64_t size[mt_max<L>()];
  int first_block[mt_max<L>() + 1];   // prefix sums of the tensors' chunk counts
  int count;
};

// The block's place: tensor index, first element of its chunk, elements in the chunk.
template <int L>
__device__ __forceinline__ int mt_locate(const MtTable<L>& t, int64_t& first, int& n) {
  const int block = blockIdx.x;
  int lo = 0;
  for (int i = 1; i < t.count; ++i)
    if (block >= t.first_block[i]) lo = i;
  first = static_cast<int64_t>(block - t.first_block[lo]) * MT_CHUNK;
  n = static_cast<int>(min(static_cast<int64_t>(MT_CHUNK), t.size[lo] - first));
  return lo;
}

__device__ __forceinline__ bool is_finite_f(float v) { return fabsf(v) <= 3.402823466e38f; }   // false for inf and NaN

struct AdamCoef {
  float beta1, beta2, corr1, corr2, eps, lr, decay;
  int mode;                         // 0: L2 regularisation (decay added to the gradient), 1: decoupled weight decay
};

__device__ __forceinline__ void adam_update(float g, float& p, float& m, float& v, const AdamCoef& c) {
  if (c.mode == 0) g += c.decay * p;
  m = c.beta1 * m + (1.f - c.beta1) * g;
  v = c.beta2 * v + (1.f - c.beta2) * g * g;
  const float m_hat = m / c.corr1, v_hat = v / c.corr2;
  float update = m_hat / (sqrtf(v_hat) + c.eps);
  if (c.mode != 0) update += c.decay * p;
  p -= c.lr * update;
}

template <typename T>
__global__ __launch_bounds__(MT_THREADS) void mt_adam_kernel(const MtTable<4> tab, const AdamCoef c) {
  constexpr int EPV = 16 / sizeof(T);
  int64_t first;
  int n;
  const int t = mt_locate(tab, first, n);
  const T* g = static_cast<const T*>(tab.addr[0][t]) + first;
  T* p = static_cast<T*>(tab.addr[1][t]) + first;
  T* m = static_cast<T*>(tab.addr[2][t]) + first;
  T* v = static_cast<T*>(tab.addr[3][t]) + first;
  const bool vec = ((reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(m) |
                     reinterpret_cast<uintptr_t>(v)) & 15u) == 0;
  const int nvec = vec ? n / EPV : 0;
  auto update = [&](int i, const pack<T, EPV>& rg, const pack<T, EPV>& rp, const pack<T, EPV>& rm, const pack<T, EPV>& rv) {
    float gv[EPV], pv[EPV], mv[EPV], vv[EPV];
    unpack_raw<T, EPV>(rg, gv); unpack_raw<T, EPV>(rp, pv); unpack_raw<T, EPV>(rm, mv); unpack_raw<T, EPV>(rv, vv);
#pragma unroll
    for (int j = 0; j < EPV; ++j) adam_update(gv[j], pv[j], mv[j], vv[j], c);
    store_pack<T, EPV>(p + i * EPV, pv);
    store_pack<T, EPV>(m + i * EPV, mv);
    store_pack<T, EPV>(v + i * EPV, vv);
  };
  int i = threadIdx.x;
  for (; i + MT_THREADS < nvec; i += 2 * MT_THREADS) {
    // two vectors of each of the four streams in flight before the first conversion
    const int k = i + MT_THREADS;
    pack<T, EPV> rg = load_raw<T, EPV>(g + i * EPV), rp = load_raw<T, EPV>(p + i * EPV), rm = load_raw<T, EPV>(m + i * EPV),
                 rv = load_raw<T, EPV>(v + i * EPV);
    pack<T, EPV> sg = load_raw<T, EPV>(g + k * EPV), sp = load_raw<T, EPV>(p + k * EPV), sm = load_raw<T, EPV>(m + k * EPV),
                 sv = load_raw<T, EPV>(v + k * EPV);
    pin_raw(rg); pin_raw(rp); pin_raw(rm); pin_raw(rv);
    pin_raw(sg); pin_raw(sp); pin_raw(sm); pin_raw(sv);
    update(i, rg, rp, rm, rv);
    update(k, sg, sp, sm, sv);
  }
  for (; i < nvec; i += MT_THREADS) {
    pack<T, EPV> rg = load_raw<T, EPV>(g + i * EPV), rp = load_raw<T, EPV>(p + i * EPV), rm = load_raw<T, EPV>(m + i * EPV),
                 rv = load_raw<T, EPV>(v + i * EPV);
    pin_raw(rg); pin_raw(rp); pin_raw(rm); pin_raw(rv);
    update(i, rg, rp, rm, rv);
  }
  for (int i = nvec * EPV + threadIdx.x; i < n; i += MT_THREADS) {
    float pv = elem<T>::to_float(p[i]), mv = elem<T>::to_float(m[i]), vv = elem<T>::to_float(v[i]);
    adam_update(elem<T>::to_float(g[i]), pv, mv, vv, c);
    p[i] = elem<T>::from_float(pv);
    m[i] = elem<T>::from_float(mv);
    v[i] = elem<T>::from_float(vv);
  }
}

// out = in * scale; a block that meets an inf or NaN in its input raises the flag (all writers store the same 1).
template <typename TI, typename TO>
__global__ __launch_bounds__(MT_THREADS) void mt_scale_kernel(const MtTable<2> tab, float scale, int* __restrict__ noop_flag) {
  constexpr int EPV = 16 / (sizeof(TI) > sizeof(TO) ? sizeof(TI) : sizeof(TO));     // the wider type moves 16 bytes
  int64_t first;
  int n;
  const int t = mt_locate(tab, first, n);
  const TI* in = static_cast<const TI*>(tab.addr[0][t]) + first;
  TO* out = static_cast<TO*>(tab.addr[1][t]) + first;
  const bool vec = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int nvec = vec ? n / EPV : 0;
  bool ok = true;
  for (int i = threadIdx.x; i < nvec; i += MT_THREADS) {
    float x[EPV];
    load_pack<TI, EPV>(in + i * EPV, x);
#pragma unroll
    for (int j = 0; j < EPV; ++j) {
      ok = ok && is_finite_f(x[j]);
      x[j] *= scale;
    }
    store_pack<TO, EPV>(out + i * EPV, x);
  }
  for (int i = nvec * EPV + threadIdx.x; i < n; i += MT_THREADS) {
    const float x = elem<TI>::to_float(in[i]);
    ok = ok && is_finite_f(x);
    out[i] = elem<TO>::from_float(x * scale);
  }
  if (!ok && noop_flag) *noop_flag = 1;
}

// Sum over the block of one value per thread, fixed order (wavefront butterflies, then the wavefronts in index order).
__device__ __forceinline__ float mt_block_sum(float v, float* red) {
  v = wave_sum(v);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < MT_WAVES; ++w) s += red[w];
  __syncthreads();
  return s;
}

// partial[block_base + b] = sum of squares of block b's chunk
template <typename T>
__global__ __launch_bounds__(MT_THREADS) void mt_sumsq_kernel(const MtTable<1> tab, float* __restrict__ partial) {
  constexpr int EPV = 16 / sizeof(T);
  __shared__ float red[MT_WAVES];
  int64_t first;
  int n;
  const int t = mt_locate(tab, first, n);
  const T* x = static_cast<const T*>(tab.addr[0][t]) + first;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
  const int nvec = vec ? n / EPV : 0;
  float acc = 0.f;
  for (int i = threadIdx.x; i < nvec; i += MT_THREADS) {
    float v[EPV];
    load_pack<T, EPV>(x + i * EPV, v);
#pragma unroll
    for (int j = 0; j < EPV; ++j) acc += v[j] * v[j];
  }
  for (int i = nvec * EPV + threadIdx.x; i < n; i += MT_THREADS) {
    const float v = elem<T>::to_float(x[i]);
    acc += v * v;
  }
  const float s = mt_block_sum(acc, red);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

// out = a x + b y; a block that meets an inf or NaN in the checked operand(s) raises the flag. check: -1 both, 0 x, 1 y.
template <typename TX, typename TO>
__global__ __launch_bounds__(MT_THREADS) void mt_axpby_kernel(const MtTable<3> tab, float a, float b, int check,
                                                              int* __restrict__ noop_flag) {
  constexpr int EPV = 16 / (sizeof(TX) > sizeof(TO) ? sizeof(TX) : sizeof(TO));
  int64_t first;
  int n;
  const int t = mt_locate(tab, first, n);
  const TX* x = static_cast<const TX*>(tab.addr[0][t]) + first;
  const TO* y = static_cast<const TO*>(tab.addr[1][t]) + first;
  TO* out = static_cast<TO*>(tab.addr[2][t]) + first;
  const bool vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int nvec = vec ? n / EPV : 0;
  const bool check_x = check != 1, check_y = check != 0;
  bool ok = true;
  for (int i = threadIdx.x; i < nvec; i += MT_THREADS) {
    float xv[EPV], yv[EPV];
    load_pack<TX, EPV>(x + i * EPV, xv);
    load_pack<TO, EPV>(y + i * EPV, yv);
#pragma unroll
    for (int j = 0; j < EPV; ++j) {
      ok = ok && (!check_x || is_finite_f(xv[j])) && (!check_y || is_finite_f(yv[j]));
      xv[j] = a * xv[j] + b * yv[j];
    }
    store_pack<TO, EPV>(out + i * EPV, xv);
  }
  for (int i = nvec * EPV + threadIdx.x; i < n; i += MT_THREADS) {
    const float xv = elem<TX>::to_float(x[i]), yv = elem<TO>::to_float(y[i]);
    ok = ok && (!check_x || is_finite_f(xv)) && (!check_y || is_finite_f(yv));
    out[i] = elem<TO>::from_float(a * xv + b * yv);
  }
  if (!ok && noop_flag) *noop_flag = 1;
}

// out = in * scale and partial[b] = sum of squares of block b's chunk of the UNSCALED input
template <typename TI, typename TO>
__global__ __launch_bounds__(MT_THREADS) void mt_sumsq_scale_kernel(const MtTable<2> tab, float scale, float* __restrict__ partial) {
  constexpr int EPV = 16 / (sizeof(TI) > sizeof(TO) ? sizeof(TI) : sizeof(TO));
  __shared__ float red[MT_WAVES];
  int64_t first;
  int n;
  const int t = mt_locate(tab, first, n);
  const TI* in = static_cast<const TI*>(tab.addr[0][t]) + first;
  TO* out = static_cast<TO*>(tab.addr[1][t]) + first;
  const bool vec = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int nvec = vec ? n / EPV : 0;
  float acc = 0.f;
  for (int i = threadIdx.x; i < nvec; i += MT_THREADS) {
    float v[EPV];
    load_pack<TI, EPV>(in + i * EPV, v);
#pragma unroll
    for (int j = 0; j < EPV; ++j) {
      acc += v[j] * v[j];
      v[j] *= scale;
    }
    store_pack<TO, EPV>(out + i * EPV, v);
  }
  for (int i = nvec * EPV + threadIdx.x; i < n; i += MT_THREADS) {
    const float v = elem<TI>::to_float(in[i]);
    acc += v * v;
    out[i] = elem<TO>::from_float(v * scale);
  }
  const float s = mt_block_sum(acc, red);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

// tensor_sq[t] = sum of the partials of tensor t (block t of the launch); partial points at this launch's first block
template <int L>
__global__ __launch_bounds__(MT_THREADS) void mt_tensor_sumsq_kernel(const MtTable<L> tab, const float* __restrict__ partial,
                                                                     float* __restrict__ tensor_sq) {
  __shared__ float red[MT_WAVES];
  const int t = blockIdx.x;
  float acc = 0.f;
  for (int b = tab.first_block[t] + threadIdx.x; b < tab.first_block[t + 1]; b += MT_THREADS) acc += partial[b];
  const float s = mt_block_sum(acc, red);
  if (threadIdx.x == 0) tensor_sq[t] = s;
}

// norm[0] = sqrt(sum_t tensor_sq[t]); per_tensor[t] = sqrt(tensor_sq[t]) when asked for. One block.
__global__ __launch_bounds__(MT_THREADS) void mt_norm_final_kernel(const float* __restrict__ tensor_sq, int n_tensors,
                                                                   float* __restrict__ norm, float* __restrict__ per_tensor) {
  __shared__ float red[MT_WAVES];
  float acc = 0.f;
  for (int t = threadIdx.x; t < n_tensors; t += MT_THREADS) {
    const float s = tensor_sq[t];
    acc += s;
    if (per_tensor) per_tensor[t] = sqrtf(s);
  }
  const float s = mt_block_sum(acc, red);
  if (threadIdx.x == 0) norm[0] = sqrtf(s);
}

int64_t chunks_of(int64_t n) { return (n + MT_CHUNK - 1) / MT_CHUNK; }

// Walks the tensor list in groups that fit one table (at most mt_max<L>() tensors, at most 2^30 blocks); empty tensors take
// no blocks. launch(table, blocks, first tensor of the group, first block of the group).
template <int L, typename F>
int mt_for_groups(int n_tensors, const void* const* const (&lists)[L], const int64_t* sizes, F launch) {
  int64_t block_base = 0;
  int t0 = 0;
  while (t0 < n_tensors) {
    MtTable<L> tab{};
    int64_t blocks = 0;
    int cnt = 0;
    while (t0 + cnt < n_tensors && cnt < mt_max<L>() && blocks + chunks_of(sizes[t0 + cnt]) <= (int64_t(1) << 30)) {
      for (int l = 0; l < L; ++l) tab.addr[l][cnt] = const_cast<void*>(lists[l][t0 + cnt]);
      tab.size[cnt] = sizes[t0 + cnt];
      tab.first_block[cnt] = static_cast<int>(blocks);
      blocks += chunks_of(sizes[t0 + cnt]);
      ++cnt;
    }
    if (cnt == 0) return fail(NMTG_ERR_INVALID, "multi_tensor: tensor %d has too many elements for one launch", t0);
    tab.first_block[cnt] = static_cast<int>(blocks);
    for (int i = cnt + 1; i <= mt_max<L>(); ++i) tab.first_block[i] = static_cast<int>(blocks);
    tab.count = cnt;
    if (int rc = launch(tab, static_cast<int>(blocks), t0, block_base)) return rc;
    block_base += blocks;
    t0 += cnt;
  }
  return 0;
}

int check_list(const char* what, int n_tensors, const int64_t* sizes, std::initializer_list<const void* const*> lists) {
  if (n_tensors < 0) return fail(NMTG_ERR_INVALID, "%s: negative tensor count", what);
  if (n_tensors == 0) return 0;
  if (!sizes) return fail(NMTG_ERR_INVALID, "%s: null size list", what);
  for (const void* const* l : lists)
    if (!l) return fail(NMTG_ERR_INVALID, "%s: null pointer list", what);
  for (int t = 0; t < n_tensors; ++t) {
    if (sizes[t] < 0) return fail(NMTG_ERR_INVALID, "%s: tensor %d has a negative size", what, t);
    if (sizes[t] > 0)
      for (const void* const* l : lists)
        if (!l[t]) return fail(NMTG_ERR_INVALID, "%s: tensor %d is a null pointer", what, t);
  }
  return 0;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_multi_tensor_adam(int n_tensors, const void* const* grads, void* const* params, void* const* exp_avg,
                                      void* const* exp_avg_sq, const int64_t* sizes, float lr, float beta1, float beta2, float eps,
                                      int step, int mode, int bias_correction, float weight_decay, int dtype, void* stream) {
  const void* const* const lists[4] = {grads, const_cast<const void* const*>(params), const_cast<const void* const*>(exp_avg),
                                       const_cast<const void* const*>(exp_avg_sq)};
  if (int rc = check_list("multi_tensor_adam", n_tensors, sizes, {lists[0], lists[1], lists[2], lists[3]})) return rc;
  NMTG_REQUIRE(step >= 1 && (mode == 0 || mode == 1), "multi_tensor_adam: step must be >= 1 and mode 0 (L2) or 1 (decoupled decay)");
  AdamCoef c{};
  c.beta1 = beta1; c.beta2 = beta2; c.eps = eps; c.lr = lr; c.decay = weight_decay; c.mode = mode;
  // double-precision powers rounded to float (the reference: 1 - std::pow(beta, step) on floats promoted by std::pow)
  c.corr1 = bias_correction ? static_cast<float>(1.0 - std::pow(static_cast<double>(beta1), step)) : 1.f;
  c.corr2 = bias_correction ? static_cast<float>(1.0 - std::pow(static_cast<double>(beta2), step)) : 1.f;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return mt_for_groups<4>(n_tensors, lists, sizes, [&](const MtTable<4>& tab, int blocks, int, int64_t) -> int {
    if (blocks == 0) return 0;
    TraceScope trace("multi_tensor_adam", st);
    NMTG_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL((mt_adam_kernel<T>), dim3(blocks), dim3(MT_THREADS), 0, st, tab, c));
    NMTG_CHECK_LAUNCH("multi_tensor_adam");
    return 0;
  });
}

extern "C" int nmtg_multi_tensor_scale(int n_tensors, const void* const* in, void* const* out, const int64_t* sizes, float scale,
                                       int* noop_flag, int in_dtype, int out_dtype, void* stream) {
  const void* const* const lists[2] = {in, const_cast<const void* const*>(out)};
  if (int rc = check_list("multi_tensor_scale", n_tensors, sizes, {lists[0], lists[1]})) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return mt_for_groups<2>(n_tensors, lists, sizes, [&](const MtTable<2>& tab, int blocks, int, int64_t) -> int {
    if (blocks == 0) return 0;
    TraceScope trace("multi_tensor_scale", st);
    NMTG_DISPATCH_DTYPE(in_dtype, TI,
                        NMTG_DISPATCH_DTYPE(out_dtype, TO,
                                            hipLaunchKernelGGL((mt_scale_kernel<TI, TO>), dim3(blocks), dim3(MT_THREADS), 0, st,
                                                               tab, scale, noop_flag)));
    NMTG_CHECK_LAUNCH("multi_tensor_scale");
    return 0;
  });
}

extern "C" int64_t nmtg_multi_tensor_l2norm_workspace_bytes(int n_tensors, const int64_t* sizes) {
  if (n_tensors <= 0 || !sizes) return 0;
  int64_t blocks = 0;
  for (int t = 0; t < n_tensors; ++t) blocks += sizes[t] > 0 ? chunks_of(sizes[t]) : 0;
  return (blocks + n_tensors) * static_cast<int64_t>(sizeof(float));
}

extern "C" int nmtg_multi_tensor_l2norm(int n_tensors, const void* const* x, const int64_t* sizes, float* norm, float* per_tensor,
                                        void* workspace, int64_t workspace_bytes, int dtype, void* stream) {
  const void* const* const lists[1] = {x};
  if (int rc = check_list("multi_tensor_l2norm", n_tensors, sizes, {lists[0]})) return rc;
  NMTG_REQUIRE(norm, "multi_tensor_l2norm: null result pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t need = nmtg_multi_tensor_l2norm_workspace_bytes(n_tensors, sizes);
  NMTG_REQUIRE(n_tensors == 0 || (workspace && workspace_bytes >= need), "multi_tensor_l2norm: workspace of %lld bytes, need %lld",
               (long long)workspace_bytes, (long long)need);
  float* tensor_sq = static_cast<float*>(workspace);                 // [n_tensors], then one partial per block
  float* partial = tensor_sq + n_tensors;
  int rc = mt_for_groups<1>(n_tensors, lists, sizes, [&](const MtTable<1>& tab, int blocks, int t0, int64_t block_base) -> int {
    if (blocks > 0) {
      TraceScope trace("multi_tensor_sumsq", st);
      NMTG_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL((mt_sumsq_kernel<T>), dim3(blocks), dim3(MT_THREADS), 0, st, tab,
                                                       partial + block_base));
      NMTG_CHECK_LAUNCH("multi_tensor_l2norm");
    }
    TraceScope trace("multi_tensor_tensor_sumsq", st);
    hipLaunchKernelGGL((mt_tensor_sumsq_kernel<1>), dim3(tab.count), dim3(MT_THREADS), 0, st, tab, partial + block_base, tensor_sq + t0);
    NMTG_CHECK_LAUNCH("multi_tensor_l2norm");
    return 0;
  });
  if (rc) return rc;
  TraceScope trace("multi_tensor_norm_final", st);
  hipLaunchKernelGGL(mt_norm_final_kernel, dim3(1), dim3(MT_THREADS), 0, st, tensor_sq, n_tensors, norm, per_tensor);
  NMTG_CHECK_LAUNCH("multi_tensor_l2norm");
  return 0;
}

extern "C" int nmtg_multi_tensor_axpby(int n_tensors, const void* const* x, const void* const* y, void* const* out,
                                       const int64_t* sizes, float a, float b, int arg_to_check, int* noop_flag, int x_dtype,
                                       int out_dtype, void* stream) {
  const void* const* const lists[3] = {x, y, const_cast<const void* const*>(out)};
  if (int rc = check_list("multi_tensor_axpby", n_tensors, sizes, {lists[0], lists[1], lists[2]})) return rc;
  NMTG_REQUIRE(arg_to_check >= -1 && arg_to_check <= 1, "multi_tensor_axpby: arg_to_check must be -1 (both), 0 (x) or 1 (y)");
  hipStream_t st = static_cast<hipStream_t>(stream);
  return mt_for_groups<3>(n_tensors, lists, sizes, [&](const MtTable<3>& tab, int blocks, int, int64_t) -> int {
    if (blocks == 0) return 0;
    TraceScope trace("multi_tensor_axpby", st);
    NMTG_DISPATCH_DTYPE(x_dtype, TX,
                        NMTG_DISPATCH_DTYPE(out_dtype, TO,
                                            hipLaunchKernelGGL((mt_axpby_kernel<TX, TO>), dim3(blocks), dim3(MT_THREADS), 0, st,
                                                               tab, a, b, arg_to_check, noop_flag)));
    NMTG_CHECK_LAUNCH("multi_tensor_axpby");
    return 0;
  });
}

extern "C" int nmtg_multi_tensor_l2norm_scale(int n_tensors, const void* const* in, void* const* out, const int64_t* sizes,
                                              float scale, float* norm, float* per_tensor, void* workspace, int64_t workspace_bytes,
                                              int in_dtype, int out_dtype, void* stream) {
  const void* const* const lists[2] = {in, const_cast<const void* const*>(out)};
  if (int rc = check_list("multi_tensor_l2norm_scale", n_tensors, sizes, {lists[0], lists[1]})) return rc;
  NMTG_REQUIRE(norm, "multi_tensor_l2norm_scale: null result pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t need = nmtg_multi_tensor_l2norm_workspace_bytes(n_tensors, sizes);
  NMTG_REQUIRE(n_tensors == 0 || (workspace && workspace_bytes >= need),
               "multi_tensor_l2norm_scale: workspace of %lld bytes, need %lld", (long long)workspace_bytes, (long long)need);
  float* tensor_sq = static_cast<float*>(workspace);
  float* partial = tensor_sq + n_tensors;
  int rc = mt_for_groups<2>(n_tensors, lists, sizes, [&](const MtTable<2>& tab, int blocks, int t0, int64_t block_base) -> int {
    if (blocks > 0) {
      TraceScope trace("multi_tensor_sumsq_scale", st);
      NMTG_DISPATCH_DTYPE(in_dtype, TI,
                          NMTG_DISPATCH_DTYPE(out_dtype, TO,
                                              hipLaunchKernelGGL((mt_sumsq_scale_kernel<TI, TO>), dim3(blocks), dim3(MT_THREADS), 0,
                                                                 st, tab, scale, partial + block_base)));
      NMTG_CHECK_LAUNCH("multi_tensor_l2norm_scale");
    }
    TraceScope trace("multi_tensor_tensor_sumsq", st);
    hipLaunchKernelGGL((mt_tensor_sumsq_kernel<2>), dim3(tab.count), dim3(MT_THREADS), 0, st, tab, partial + block_base,
                       tensor_sq + t0);
    NMTG_CHECK_LAUNCH("multi_tensor_l2norm_scale");
    return 0;
  });
  if (rc) return rc;
  TraceScope trace("multi_tensor_norm_final", st);
  hipLaunchKernelGGL(mt_norm_final_kernel, dim3(1), dim3(MT_THREADS), 0, st, tensor_sq, n_tensors, norm, per_tensor);
  NMTG_CHECK_LAUNCH("multi_tensor_l2norm_scale");
  return 0;
}
