// Attention of one new query position over cached keys and values: the inner step of incremental decoding.
//
// The reference reaches this case through the same functions as training (self_attention_func.py:162-174 with
// incremental=True: keys / values concatenated onto the cache, one query row; encdec_attention_func_bias.py:181-213:
// cached encoder keys / values) and runs it as two batched GEMMs of one row each plus a softmax. With one query row
// there is nothing for a matrix core to reuse: every key and value element is read once and used once, so the step is
// bound by reading the cache. One block per (sentence, head) reads the keys straight from the time-first cache
// ([keys, batch, embed]: 2 * head_dim bytes per key, the sentence's other heads next to them), keeps the scores of the
// whole row in LDS, normalises them, writes the probabilities (the reference returns them as coverage) and accumulates
// the context from the values in a second pass. Rounding points as on the GEMM path: scores and probabilities are
// rounded to the 16-bit type where that path stores them.
#include "common.hip.h"

namespace nmtg {
namespace {

constexpr int DEC_THREADS = 256;
constexpr int DEC_MAX_KEYS = 16384;   // scores of one row in LDS: 64 KB

struct DecArgs {
  const void *q, *keys, *values;
  const uint8_t* kmask;   // [batch, tk], 1 = masked key; may be null
  void *probs, *ctx;      // probs [batch * heads, tk] dense; ctx like q
  int64_t q_sb, k_st, k_sb, v_st, v_sb, c_sb;   // element strides: per sentence (sb) and per key position (st)
  int heads, tk;
  float scale;
};

template <typename T>
__device__ __forceinline__ float round_to(float v) { return elem<T>::to_float(elem<T>::from_float(v)); }

__device__ __forceinline__ float block_reduce(float v, bool is_max, float* red) {
  v = is_max ? wave_max(v) : wave_sum(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();                       // red may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < DEC_THREADS / 64; ++w) r = is_max ? fmaxf(r, red[w]) : r + red[w];
  return r;
}

// LPR lanes share one key row: head_dim = 8 * LPR
template <typename T, int LPR>
__global__ __launch_bounds__(DEC_THREADS) void attn_decode_kernel(DecArgs a) {
  extern __shared__ __align__(16) float lds[];
  float* sc = lds;                       // [tk]
  float* red = lds + a.tk;               // [4] + [4][8 * LPR]
  constexpr int D = 8 * LPR, RPS = DEC_THREADS / LPR, U = 8;   // U loads of 16 bytes in flight per lane
  const int bh = blockIdx.x, b = bh / a.heads, h = bh % a.heads;
  const int tid = threadIdx.x, slot = tid / LPR, c = tid % LPR;
  const int64_t head_off = static_cast<int64_t>(h) * D + 8 * c;
  uint32_t qw[4];
  {
    const pack<T, 8> qraw = load_raw<T, 8>(static_cast<const T*>(a.q) + b * a.q_sb + head_off);
    __builtin_memcpy(qw, &qraw, 16);
  }
  const T* kb = static_cast<const T*>(a.keys) + b * a.k_sb + head_off;
  const T* vb = static_cast<const T*>(a.values) + b * a.v_sb + head_off;
  const uint8_t* km = a.kmask ? a.kmask + static_cast<int64_t>(b) * a.tk : nullptr;

  // Keys behind the sentence's last live one (the padding of a shorter sentence) have probability zero whatever the
  // cache holds there: their keys and values are not read.
  int live = a.tk;
  if (km != nullptr) {
    int last = 0;
    for (int j = tid; j < a.tk; j += DEC_THREADS)
      if (!km[j]) last = j + 1;
    live = static_cast<int>(block_reduce(static_cast<float>(last), true, red));   // <= 16384: exact in fp32
    for (int j = live + tid; j < a.tk; j += DEC_THREADS) sc[j] = -INFINITY;
  }

  // ---- scores ----
  for (int j0 = 0; j0 < live; j0 += RPS * U) {
    pack<T, 8> raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = j0 + u * RPS + slot;
      raw[u] = load_raw<T, 8>(kb + static_cast<int64_t>(j < live ? j : 0) * a.k_st);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = j0 + u * RPS + slot;
      uint32_t kw[4];
      __builtin_memcpy(kw, &raw[u], 16);
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) dot = dot2<T>(qw[e], kw[e], dot);
#pragma unroll
      for (int d = 1; d < LPR; d <<= 1) dot += __shfl_xor(dot, d);
      if (c == 0 && j < live) sc[j] = (km != nullptr && km[j]) ? -INFINITY : round_to<T>(dot * a.scale);
    }
  }
  __syncthreads();

  // ---- softmax over the row; a row without any live key gives zeros ----
  constexpr float LOG2E = 1.4426950408889634f;
  float mx = -INFINITY;
  for (int j = tid; j < a.tk; j += DEC_THREADS) mx = fmaxf(mx, sc[j]);
  mx = block_reduce(mx, true, red);
  const float base = mx == -INFINITY ? 0.f : mx;
  float sum = 0.f;
  for (int j = tid; j < a.tk; j += DEC_THREADS) {
    const float e = __builtin_amdgcn_exp2f((sc[j] - base) * LOG2E);
    sc[j] = e;
    sum += e;
  }
  sum = block_reduce(sum, false, red);
  const float inv = sum > 0.f ? 1.f / sum : 0.f;
  T* pr = static_cast<T*>(a.probs) + static_cast<int64_t>(bh) * a.tk;
  for (int j = tid; j < a.tk; j += DEC_THREADS) {
    const T p = elem<T>::from_float(sc[j] * inv);
    pr[j] = p;
    sc[j] = elem<T>::to_float(p);
  }
  __syncthreads();

  // ---- context = probabilities x values ----
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int j0 = 0; j0 < live; j0 += RPS * U) {
    pack<T, 8> raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = j0 + u * RPS + slot;
      raw[u] = load_raw<T, 8>(vb + static_cast<int64_t>(j < live ? j : 0) * a.v_st);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = j0 + u * RPS + slot;
      const float p = j < live ? sc[j] : 0.f;
      float vv[8];
      unpack_raw<T, 8>(raw[u], vv);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf(p, vv[e], acc[e]);
    }
  }
  // the row slots of one wavefront (lanes with equal c), then the four wavefronts through LDS
#pragma unroll
  for (int d = LPR; d < 64; d <<= 1)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += __shfl_xor(acc[e], d);
  float* part = red + 4;
  if ((tid & 63) < LPR) {
#pragma unroll
    for (int e = 0; e < 8; ++e) part[(tid >> 6) * D + 8 * c + e] = acc[e];
  }
  __syncthreads();
  if (tid < LPR) {
    float out[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = part[8 * c + e] + part[D + 8 * c + e] + part[2 * D + 8 * c + e] + part[3 * D + 8 * c + e];
    store_pack<T, 8>(static_cast<T*>(a.ctx) + b * a.c_sb + head_off, out);
  }
}

template <typename T>
int decode_launch(const DecArgs& a, int head_dim, int64_t blocks, hipStream_t st) {
  const int lds = (a.tk + 4 + 4 * head_dim) * static_cast<int>(sizeof(float));
  TraceScope trace("attn_decode", st);
#define DEC_LAUNCH(LPR)                                                                                                   \
  {                                                                                                                       \
    if (lds > 64 * 1024) {                                                                                                \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_decode_kernel<T, LPR>),                      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);                                \
      if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "attn_decode: cannot reserve %d bytes of LDS", lds);              \
    }                                                                                                                     \
    hipLaunchKernelGGL((attn_decode_kernel<T, LPR>), dim3(static_cast<unsigned>(blocks)), dim3(DEC_THREADS), lds, st, a); \
  }
  if (head_dim == 32) DEC_LAUNCH(4)
  else if (head_dim == 64) DEC_LAUNCH(8)
  else DEC_LAUNCH(16)
#undef DEC_LAUNCH
  return 0;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_attn_decode(const void* q, int64_t q_stride_b, const void* keys, int64_t k_stride_t, int64_t k_stride_b,
                                const void* values, int64_t v_stride_t, int64_t v_stride_b, const uint8_t* key_mask, void* probs,
                                void* context, int64_t ctx_stride_b, int64_t batch, int64_t heads, int64_t head_dim, int64_t tk,
                                float scale, int dtype, void* stream) {
  NMTG_REQUIRE(batch >= 0 && heads >= 1 && tk >= 0 && batch * heads <= 0x7fffffff, "attn_decode: bad shape batch=%lld heads=%lld keys=%lld",
               (long long)batch, (long long)heads, (long long)tk);
  NMTG_REQUIRE(head_dim == 32 || head_dim == 64 || head_dim == 128, "attn_decode: head dimension %lld (32, 64 and 128 are built)",
               (long long)head_dim);
  NMTG_REQUIRE(dtype == NMTG_F16 || dtype == NMTG_BF16, "attn_decode: fp16 or bf16 tensors required");
  NMTG_REQUIRE(tk <= DEC_MAX_KEYS, "attn_decode: %lld keys, at most %d (the scores of a row are kept in LDS)", (long long)tk, DEC_MAX_KEYS);
  if (batch == 0) return 0;
  NMTG_REQUIRE(q && probs && context && (tk == 0 || (keys && values)), "attn_decode: null pointer argument");
  const int64_t strides[] = {q_stride_b, k_stride_t, k_stride_b, v_stride_t, v_stride_b, ctx_stride_b};
  for (int64_t s : strides) NMTG_REQUIRE(s % 8 == 0 && s >= 0, "attn_decode: strides must be non-negative multiples of 8 elements");
  NMTG_REQUIRE(aligned16(q) && aligned16(keys) && aligned16(values) && aligned16(context), "attn_decode: 16-byte aligned tensors required");
  DecArgs a = {};
  a.q = q; a.keys = keys; a.values = values; a.kmask = key_mask; a.probs = probs; a.ctx = context;
  a.q_sb = q_stride_b; a.k_st = k_stride_t; a.k_sb = k_stride_b; a.v_st = v_stride_t; a.v_sb = v_stride_b; a.c_sb = ctx_stride_b;
  a.heads = static_cast<int>(heads); a.tk = static_cast<int>(tk); a.scale = scale;
  int rc;
  if (dtype == NMTG_F16) rc = decode_launch<f16_t>(a, static_cast<int>(head_dim), batch * heads, static_cast<hipStream_t>(stream));
  else rc = decode_launch<bf16_t>(a, static_cast<int>(head_dim), batch * heads, static_cast<hipStream_t>(stream));
  if (rc) return rc;
  NMTG_CHECK_LAUNCH("attn_decode");
  return 0;
}
