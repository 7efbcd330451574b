// MFMA GEMM core for gfx950 (MI355X): C[m][n] = alpha * sum_k A(m,k) * B(n,k) with fused epilogues.
//
// Stands in for the cuBLAS / cuBLASLt calls of the reference's fused MLP and attention
// (onmt/modules/extensions/mlp/mlp_gelu_cuda.cu:86-201 mlp_gemm; mlp_blaslt/cublaslt_wrapper.cuh
// epilogues BIAS / GELU_AUX_BIAS / BGRADB; multihead_attn_blaslt/strided_batched_gemm_blaslt.cuh:9-126)
// and for the element-wise kernels that follow them there (biasAddGeLU_fprop,
// biasAddDropoutGeLU_fprop, *_bprop: mlp_gelu_cuda.cu:206-1216), which here run inside the GEMM
// epilogue so the [tokens, inner] activations cross HBM once per direction instead of three times.
//
// Shape of the kernel
//   * 16-bit inputs (fp16 or bf16), fp32 accumulation in v_mfma_f32_32x32x16 (64-lane wavefronts).
//   * A block owns a BM x BN tile of C; WAVES_M x WAVES_N wavefronts each own (BM/WAVES_M) x
//     (BN/WAVES_N) of it as 32x32 MFMA tiles. K is walked in steps of 64 through a double-buffered
//     LDS stage; the next step's global loads are in flight in registers while the current step
//     multiplies.
//   * Operand layouts: "KC" = the reduction index is contiguous in memory (row-major [rows][k]);
//     "MC" = the row index is contiguous ([k][rows]). MC operands are transposed in registers
//     (4x8 blocks, v_perm_b32) on their way into LDS, so LDS always holds [rows][64 k] and the
//     MFMA fragment reads are single 128-bit LDS loads.
//   * LDS rows are 128 bytes; the 16-byte chunk c of row r lives at chunk c ^ ((r ^ (r >> 3)) & 7),
//     which makes the fragment reads, the KC writes and the transposing MC writes conflict free.
//   * The MFMA is issued with the B tile as its first operand, so a lane ends up holding 4
//     consecutive n for one m: the epilogue packs them, stages the tile through LDS and leaves
//     with 16-byte row-contiguous global stores (and coalesced loads of bias / masks / saved
//     activations).
//   * blockIdx.x is remapped so that each of the 8 XCDs (which receive consecutive block ids
//     round-robin) works on a contiguous run of tiles and re-uses A / B through its own L2.
#pragma once
#include "common.hip.h"
#include "reduce.hip.h"
#include <type_traits>

namespace nmtg {

enum GemmEpi {
  EPI_PLAIN = 0,    // C = alpha*acc (+ bias[n])
  EPI_ACT_FWD = 1,  // h = acc + bias -> aux_out;  C = act(h) * keep * dscale
  EPI_ACT_BWD = 2,  // C = T(acc) * act'(aux_in) * dscale * keep (keep = 1 without a mask);  colsum_part[m_tile][n] = sum_m C
  EPI_SCORES = 3,   // C = alpha*acc, -inf where the key-padding / time mask is set
  EPI_SPLITK = 4,   // fp32 partial tile -> workspace (reduced by splitk_reduce_kernel)
  // C = alpha*acc with the mask as -inf (as EPI_SCORES), then the row softmax of the stored (rounded) scores and
  // dropout in the same pass: aux_out = softmax (optional), out2 = dropped probabilities. The block tile spans
  // the whole row (N <= BN), one wavefront normalises one row.
  EPI_SCORES_SOFTMAX = 5,
  // Backward counterpart on the same whole-row tile: acc = dP (gradient of the dropped probabilities, rounded to
  // T as the two-kernel path stores it); P is recomputed from the saved scores (aux_in, laid out like C) and
  // C = P * (g - sum_k P g), g = keep * dP / (1 - p).
  EPI_DSOFTMAX = 6,
  // EPI_SCORES_SOFTMAX with the dropout keep mask drawn from Philox in the kernel (and stored). Its own instantiation:
  // as a run-time branch the generator's integer work is scheduled ahead of the branch and runs in every mode.
  EPI_SCORES_SOFTMAX_RNG = 7
};

struct GemmArgs {
  const void* A;
  const void* B;
  void* C;
  int64_t lda, ldb, ldc;
  int64_t sA, sB, sC;  // batch strides in elements
  int M, N, K;
  int batch;
  int splits, k_per_split;
  float alpha;
  int vec;                  // widest access (elements: 8, 4 or 1) every operand and extent allows
  int ring;                 // the call meets the requirements of the slot-ring kernel (gemm_ring.hip.h)
  const void* bias;
  void* aux_out;
  void* out2;               // EPI_SCORES_SOFTMAX: dropped probabilities, laid out like C
  const void* aux_in;
  int64_t ld_aux;
  const uint8_t* dmask;     // dropout keep mask [M, N] dense; read, or written when rng != 0
  float dscale, keep_p;
  int rng;                  // ACT_FWD: draw the keep mask from Philox and store it to dmask
  uint64_t seed, offset;
  int act;
  int act_lut;              // gelu / gelu' through the LDS table (ring kernels only; set by the host on request)
  int defer_reduce;         // host only: a split-K call leaves its reduction to the caller (who queues it in a ReduceTail)
  int tile_used;            // host only, filled by gemm_run: the tile the call ran with
  // host only: a list of small reduction jobs (TailArgs, reduce.hip.h) that `rider_blocks` extra blocks of this launch
  // run beside the GEMM's own blocks (they have no part in the product; what they read must be complete before the
  // launch). Kernels that cannot carry them leave riders_taken at 0 and the caller launches the list itself.
  const void* riders;
  int rider_blocks;
  int riders_taken;
  float* colsum_part;
  const uint8_t* kmask;
  int kmask_kind, heads;
  float* ws;
  int m_tiles, n_tiles;
#ifdef NMTG_GEMM_PROF
  long long* prof;          // per-block phase timestamps (tuning builds only)
#endif
};

#ifdef NMTG_GEMM_PROF
// slots 0..4: shader-clock stamps of the phases; slots 5 and 6: constant-rate (100 MHz) stamps of the block's start and end
#define NMTG_PROF_MARK(i) do { if (g.prof != nullptr && threadIdx.x == 0) { long long* pr_ = g.prof + (static_cast<long long>(blockIdx.y) * gridDim.x + blockIdx.x) * 8; pr_[(i)] = clock64(); if ((i) == 0) pr_[5] = wall_clock64(); if ((i) == 4) pr_[6] = wall_clock64(); } } while (0)
#else
#define NMTG_PROF_MARK(i) do { } while (0)
#endif

template <typename T> struct mfma;
typedef float acc16_t __attribute__((ext_vector_type(16)));
template <> struct mfma<f16_t> {
  typedef _Float16 vec __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, acc16_t& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(vec, a), __builtin_bit_cast(vec, b), c, 0, 0, 0);
  }
};
template <> struct mfma<bf16_t> {
  typedef __bf16 vec __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, acc16_t& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(vec, a), __builtin_bit_cast(vec, b), c, 0, 0, 0);
  }
};

constexpr int GEMM_BK = 64;

__device__ __forceinline__ int lds_swz(int row) { return (row ^ (row >> 3)) & 7; }

// Activation and derivative (fp32 math). Codes are nmtg_act.
//
// The exact-erf gelu is the hot one (it runs on every hidden activation inside the GEMM
// epilogue), so the normal CDF uses the rational approximation 7.1.26 of Abramowitz & Stegun,
//   erfc(z) = (a1 t + a2 t^2 + a3 t^3 + a4 t^4 + a5 t^5) exp(-z^2),  t = 1 / (1 + p z),  z >= 0,
// absolute error < 1.5e-7 (fp32 rounding level, far inside the 16-bit output precision), at
// about a third of the instructions of erff(); Phi and the density share the one exponential.
// Single-instruction reciprocal and 2^x (v_rcp_f32 / v_exp_f32, 1 ulp): the library forms expand to a
// ten-instruction IEEE division and a range-checked exponential, which dominated the epilogue.
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct NormalCdfPdf { float cdf, pdf; };
__device__ __forceinline__ NormalCdfPdf normal_cdf_pdf(float h) {
  const float z = fabsf(h) * 0.70710678118654752f;
  const float t = fast_rcp(fmaf(0.3275911f, z, 1.f));
  // coefficients pre-multiplied by 1/2: half_erfc = 0.5 * erfc(z)
  float poly = fmaf(0.5f * 1.061405429f, t, 0.5f * -1.453152027f);
  poly = fmaf(poly, t, 0.5f * 1.421413741f);
  poly = fmaf(poly, t, 0.5f * -0.284496736f);
  poly = fmaf(poly, t, 0.5f * 0.254829592f);
  const float e = fast_exp2(h * h * -0.72134752044448170f);  // exp(-h^2 / 2)
  const float half_erfc = poly * t * e;
  NormalCdfPdf r;
  r.cdf = h >= 0.f ? 1.f - half_erfc : half_erfc;
  r.pdf = 0.3989422804014327f * e;
  return r;
}

// gelu through a table. The activation epilogues are VALU-bound (about 30 instruction slots per element, two of
// them quarter-rate transcendentals), so Phi(h) and gelu'(h) can instead be read from a 2049-entry table over
// [-6, 6] (16 KB) that the block builds in LDS with the exact formula: one fused multiply-add for the table
// coordinate, a clamp, a fraction, one 8-byte LDS read of (value, difference to the next entry) and one fused
// multiply-add. Linear interpolation error: step^2 / 8 * max|f''| = 1.0e-6 for Phi, 2.6e-6 for gelu': a rounded
// 16-bit result differs from the formula's in about one element in a thousand, by one unit in the last place.
// (A 513-entry table, error 1.7e-5, flipped enough bf16 roundings to push the second layer's output past the
// absolute tolerance on a few elements in 10^5 at the benchmark shape.) Outside [-6, 6] the end values are used.
constexpr int NMTG_ACT_GELU_LUT = 100;      // internal activation code: gelu evaluated through the table
constexpr int ACT_LUT_N = 2048;
constexpr float ACT_LUT_R = 6.f;
constexpr int ACT_LUT_BYTES = (ACT_LUT_N + 1) * 8;

template <bool GRAD>
__device__ __forceinline__ void act_lut_fill(float2* tab, int tid, int nthreads) {
  constexpr float STEP = 2.f * ACT_LUT_R / ACT_LUT_N;
  for (int t = tid; t <= ACT_LUT_N; t += nthreads) {
    const float x0 = -ACT_LUT_R + STEP * static_cast<float>(t);
    const NormalCdfPdf a = normal_cdf_pdf(x0), b = normal_cdf_pdf(x0 + STEP);
    const float f0 = GRAD ? fmaf(x0, a.pdf, a.cdf) : a.cdf;
    const float f1 = GRAD ? fmaf(x0 + STEP, b.pdf, b.cdf) : b.cdf;
    tab[t] = make_float2(f0, f1 - f0);
  }
}
__device__ __forceinline__ float act_lut_eval(const float2* tab, float h) {
  float u = fmaf(h, ACT_LUT_N / (2.f * ACT_LUT_R), 0.5f * ACT_LUT_N);
  u = __builtin_amdgcn_fmed3f(u, 0.f, static_cast<float>(ACT_LUT_N));
  const float2 e = tab[static_cast<int>(u)];
  return fmaf(__builtin_amdgcn_fractf(u), e.y, e.x);
}

template <int ACT>
__device__ __forceinline__ float act_apply(float h, const float2* tab) {
  if constexpr (ACT == NMTG_ACT_RELU) return fmaxf(h, 0.f);
  else if constexpr (ACT == NMTG_ACT_GELU) return h * normal_cdf_pdf(h).cdf;
  else if constexpr (ACT == NMTG_ACT_GELU_LUT) return h * act_lut_eval(tab, h);
  else if constexpr (ACT == NMTG_ACT_SILU) return h * fast_rcp(1.f + fast_exp2(h * -1.4426950408889634f));
  else if constexpr (ACT == NMTG_ACT_AGELU) {
    // 0.5 h (1 + tanh u) = h * sigmoid(2u)
    const float u2 = 1.5957691216057308f * (h + 0.044715f * h * h * h);
    return h * fast_rcp(1.f + fast_exp2(u2 * -1.4426950408889634f));
  } else return h;
}
template <int ACT>
__device__ __forceinline__ float act_grad(float h, const float2* tab) {
  if constexpr (ACT == NMTG_ACT_RELU) return h > 0.f ? 1.f : 0.f;
  else if constexpr (ACT == NMTG_ACT_GELU) {
    const NormalCdfPdf n = normal_cdf_pdf(h);
    return fmaf(h, n.pdf, n.cdf);
  } else if constexpr (ACT == NMTG_ACT_GELU_LUT) {
    return act_lut_eval(tab, h);
  } else if constexpr (ACT == NMTG_ACT_SILU) {
    const float s = fast_rcp(1.f + fast_exp2(h * -1.4426950408889634f));
    return s * (1.f + h * (1.f - s));
  } else if constexpr (ACT == NMTG_ACT_AGELU) {
    // d/dh [h s(2u)] = s + h s (1 - s) 2u',  u' = k (1 + 3 c h^2)
    const float u2 = 1.5957691216057308f * (h + 0.044715f * h * h * h);
    const float sg = fast_rcp(1.f + fast_exp2(u2 * -1.4426950408889634f));
    return sg + h * sg * (1.f - sg) * 1.5957691216057308f * (1.f + 0.134145f * h * h);
  } else return 1.f;
}

// Calls f(std::integral_constant<int, ACT>) for the runtime activation code: one uniform branch
// outside the element loops instead of a switch per element.
template <bool LUT_OK, typename F>
__device__ __forceinline__ void dispatch_act(int act, int lut, F&& f) {
  if constexpr (LUT_OK) {
    if (lut && act == NMTG_ACT_GELU) {
      f(std::integral_constant<int, NMTG_ACT_GELU_LUT>{});
      return;
    }
  }
  switch (act) {
    case NMTG_ACT_RELU: f(std::integral_constant<int, NMTG_ACT_RELU>{}); break;
    case NMTG_ACT_GELU: f(std::integral_constant<int, NMTG_ACT_GELU>{}); break;
    case NMTG_ACT_SILU: f(std::integral_constant<int, NMTG_ACT_SILU>{}); break;
    case NMTG_ACT_AGELU: f(std::integral_constant<int, NMTG_ACT_AGELU>{}); break;
    default: f(std::integral_constant<int, NMTG_ACT_NONE>{}); break;
  }
}

// ---------------------------------------------------------------------------------------------
// Vector-width-templated, branch-free global accesses. VEC (8, 4 or 1 elements) is the widest
// access every operand of the call allows; a group of 8 elements moves as 8/VEC accesses, each
// with its own validity bit. Out-of-range loads read a clamped (always mapped) address and are
// zeroed by a select, so the loads of a tile are straight-line code the compiler can issue back
// to back.
// ---------------------------------------------------------------------------------------------
template <int VEC> struct raw_vec;
template <> struct raw_vec<8> { typedef uint4 type; };
template <> struct raw_vec<4> { typedef uint2 type; };
template <> struct raw_vec<1> { typedef uint16_t type; };

// Zeroes the 16-bit elements e >= nvalid of an 8-element group (0 <= nvalid < 8).
__device__ __forceinline__ uint4 keep_first(const uint4& v, int nvalid) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int left = nvalid - 2 * i;   // valid elements of word i
    w[i] = left >= 2 ? w[i] : left == 1 ? (w[i] & 0xffffu) : 0u;
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Loads elements [0, 8) at p; element e is valid iff e < nvalid. A vector that holds at least one valid element is
// read whole: p is VEC-aligned and the operand's pitch a multiple of VEC, so the access stays inside the row's own
// pitch (and inside the aligned 2 VEC bytes that hold a valid element: same page, hence mapped, even at the end of
// an allocation). With ZERO the invalid elements come back as zeros, without it they are unspecified.
// `safe` is any mapped address of the same alignment class.
template <int VEC, bool ZERO = true>
__device__ __forceinline__ uint4 load8(const uint16_t* __restrict__ p, const uint16_t* __restrict__ safe, int nvalid) {
  typedef typename raw_vec<VEC>::type R;
  union { uint4 v; R r[8 / VEC]; } u;
#pragma unroll
  for (int h = 0; h < 8 / VEC; ++h) {
    const bool ok = h * VEC < nvalid;
    R val = *reinterpret_cast<const R*>(ok ? p + h * VEC : safe);
    if (ZERO && !ok) val = R{};
    u.r[h] = val;
  }
  if constexpr (ZERO && VEC > 1) {
    if (nvalid > 0 && nvalid < 8 && nvalid % VEC != 0) u.v = keep_first(u.v, nvalid);
  }
  return u.v;
}

// Stores the elements e < nvalid; a partly valid vector goes out element by element.
template <int VEC>
__device__ __forceinline__ void store8(uint16_t* __restrict__ p, const uint4& v, int nvalid) {
  typedef typename raw_vec<VEC>::type R;
  union { uint4 v; R r[8 / VEC]; uint16_t e[8]; } u;
  u.v = v;
#pragma unroll
  for (int h = 0; h < 8 / VEC; ++h) {
    const int left = nvalid - h * VEC;
    if (left >= VEC) {
      // Non-temporal: the output is read next by another kernel (through another XCD's L2 at the earliest), so it
      // should stream out to memory while the kernel runs instead of waiting in L2 for the write-back at its end.
      if constexpr (VEC == 8) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(u32x4, u.r[h]), reinterpret_cast<u32x4*>(p + h * VEC));
      } else {
        *reinterpret_cast<R*>(p + h * VEC) = u.r[h];
      }
    } else if (VEC > 1 && left > 0) {
#pragma unroll
      for (int e = 0; e < VEC - 1; ++e)
        if (e < left) p[h * VEC + e] = u.e[h * VEC + e];
    }
  }
}

template <int VEC, bool ZERO = true>
__device__ __forceinline__ uint2 load8_bytes(const uint8_t* __restrict__ p, const uint8_t* __restrict__ safe, int nvalid) {
  if constexpr (VEC == 8) {
    const bool ok = nvalid > 0;
    uint2 v = *reinterpret_cast<const uint2*>(ok ? p : safe);
    if (ZERO && !ok) v = make_uint2(0, 0);
    return v;
  } else if constexpr (VEC == 4) {
    uint2 v;
    const bool ok0 = nvalid > 0, ok1 = nvalid > 4;
    v.x = *reinterpret_cast<const uint32_t*>(ok0 ? p : safe);
    v.y = *reinterpret_cast<const uint32_t*>(ok1 ? p + 4 : safe);
    if (ZERO && !ok0) v.x = 0;
    if (ZERO && !ok1) v.y = 0;
    return v;
  } else {
    uint32_t w[2] = {0, 0};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const bool ok = e < nvalid;
      uint32_t b = *(ok ? p + e : safe);
      if (!ok) b = 0;
      w[e >> 2] |= b << (8 * (e & 3));
    }
    return make_uint2(w[0], w[1]);
  }
}

template <int VEC>
__device__ __forceinline__ void store8_bytes(uint8_t* __restrict__ p, uint2 v, int nvalid) {
  if constexpr (VEC == 8) {
    if (nvalid > 0) *reinterpret_cast<uint2*>(p) = v;
  } else if constexpr (VEC == 4) {
    if (nvalid > 0) *reinterpret_cast<uint32_t*>(p) = v.x;
    if (nvalid > 4) *reinterpret_cast<uint32_t*>(p + 4) = v.y;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (e < nvalid) p[e] = static_cast<uint8_t>(((e < 4 ? v.x : v.y) >> (8 * (e & 3))) & 0xffu);
  }
}

__device__ __forceinline__ uint8_t byte_of(uint2 v, int e) { return ((e < 4 ? v.x : v.y) >> (8 * (e & 3))) & 0xffu; }

template <typename T>
__device__ __forceinline__ void unpack8(const uint4& raw, float (&v)[8]) {
  const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
  for (int k = 0; k < 8; ++k) v[k] = elem<T>::to_float(e[k]);
}
template <typename T>
__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
  uint4 raw;
  T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
  for (int k = 0; k < 8; ++k) e[k] = elem<T>::from_float(v[k]);
  return raw;
}

// ---------------------------------------------------------------------------------------------
// Global -> register -> LDS staging of one operand tile [ROWS][64 k].
// ---------------------------------------------------------------------------------------------
template <typename T, int ROWS, int NT, bool KC, int VEC>
struct TileStage {
  static constexpr int UNITS = KC ? ROWS * 8 : ROWS * 2;  // 16-byte chunks (KC) or 4k x 8row blocks (MC)
  static constexpr int PER = (UNITS + NT - 1) / NT;
  static constexpr int NREG = KC ? PER : PER * 4;
  static constexpr int RG8 = ROWS / 64 > 0 ? ROWS / 64 : 1;
  // With 16-byte accesses a register is wholly valid or wholly out of range: the loads leave
  // out-of-range registers unzeroed and remember them in `valid`; store() zeroes them. That keeps
  // every use of a loaded value (and so the wait for it) behind the MFMA work of the step.
  static constexpr bool DEFER = VEC == 8;
  uint4 regs[NREG];
  uint32_t valid;
  int kleft;   // valid k of the step being staged (>= 64: all of them)

  // base: operand pointer for this batch; rows_total / row0: extent and tile origin in the row
  // index; k0: first k of this step; kend: one past the last valid k.
  __device__ __forceinline__ void load(const T* __restrict__ base, int64_t ld, int rows_total, int row0, int k0,
                                       int kend, int tid) {
    const uint16_t* b16 = reinterpret_cast<const uint16_t*>(base);
    valid = 0;
    kleft = kend - k0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = tid + i * NT;
      if constexpr (KC) {
        const int row = q >> 3, c = q & 7;
        const int grow = row0 + row, gk = k0 + c * 8;
        const bool ok = (UNITS % NT == 0 || q < UNITS) && grow < rows_total;
        const int nvalid = ok ? kend - gk : 0;
        regs[i] = load8<VEC, !DEFER>(b16 + static_cast<int64_t>(ok ? grow : 0) * ld + (nvalid > 0 ? gk : 0), b16, nvalid);
        if (nvalid > 0) valid |= 1u << i;
      } else {
        const int rg_lo = q & 7, kq_lo = (q >> 3) & 1, rest = q >> 4;
        const int rg = rg_lo + 8 * (rest % RG8), kq = kq_lo + 2 * (rest / RG8);
        const int grow = row0 + rg * 8;
        const bool qok = (UNITS % NT == 0 || q < UNITS);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const int gk = k0 + kq * 4 + kk;
          const bool ok = qok && gk < kend;
          const int nvalid = ok ? rows_total - grow : 0;
          regs[i * 4 + kk] = load8<VEC, !DEFER>(b16 + static_cast<int64_t>(ok ? gk : 0) * ld + (nvalid > 0 ? grow : 0), b16, nvalid);
          if (nvalid > 0) valid |= 1u << (i * 4 + kk);
        }
      }
    }
  }

  __device__ __forceinline__ void store(T* __restrict__ buf, int tid) {
    if constexpr (DEFER) {
#pragma unroll
      for (int r = 0; r < NREG; ++r)
        if (!((valid >> r) & 1u)) regs[r] = make_uint4(0, 0, 0, 0);
      if constexpr (KC) {
        // last step of a reduction that is not a multiple of 8: the chunk that straddles the end keeps its valid k only
        if (kleft < GEMM_BK && (kleft & 7) != 0) {
#pragma unroll
          for (int i = 0; i < PER; ++i) {
            const int nv = kleft - ((tid + i * NT) & 7) * 8;
            if (nv > 0 && nv < 8) regs[i] = keep_first(regs[i], nv);
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = tid + i * NT;
      if (UNITS % NT != 0 && q >= UNITS) continue;
      if constexpr (KC) {
        const int row = q >> 3, c = q & 7;
        *reinterpret_cast<uint4*>(buf + row * GEMM_BK + ((c ^ lds_swz(row)) * 8)) = regs[i];
      } else {
        const int rg_lo = q & 7, kq_lo = (q >> 3) & 1, rest = q >> 4;
        const int rg = rg_lo + 8 * (rest % RG8), kq = kq_lo + 2 * (rest / RG8);
        const uint32_t* w0 = reinterpret_cast<const uint32_t*>(&regs[i * 4 + 0]);
        const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&regs[i * 4 + 1]);
        const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&regs[i * 4 + 2]);
        const uint32_t* w3 = reinterpret_cast<const uint32_t*>(&regs[i * 4 + 3]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int row = rg * 8 + j;
          const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
          uint2 o;
          o.x = __builtin_amdgcn_perm(w1[j >> 1], w0[j >> 1], sel);  // k+0, k+1 of this row
          o.y = __builtin_amdgcn_perm(w3[j >> 1], w2[j >> 1], sel);  // k+2, k+3
          const int c = kq >> 1, half = kq & 1;
          *reinterpret_cast<uint2*>(buf + row * GEMM_BK + ((c ^ lds_swz(row)) * 8) + half * 4) = o;
        }
      }
    }
  }
};

// ---------------------------------------------------------------------------------------------
// Epilogue shared by the GEMM kernels: accumulators -> (bias, activation, masks, ...) -> global.
// ---------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int EPI, int VEC, bool LUT_OK = false>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, acc16_t (&acc)[BM / WAVES_M / 32][BN / WAVES_N / 32],
                                              uint8_t* lds_raw, int tile_m, int tile_n, int bz, int split) {
  constexpr int NT = 64 * WAVES_M * WAVES_N;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int ntile = g.m_tiles * g.n_tiles;
  // Lane (l) register r of tile (i, j) holds C[m][n] with
  //   m = m0 + wm0 + 32 i + (l & 31),   n = n0 + wn0 + 32 j + 8 (r / 4) + 4 (l >> 5) + (r % 4).
  if constexpr (EPI == EPI_SPLITK) {
    // fp32 partials in the accumulator's own layout: every store is 64 lanes x 16 contiguous bytes
    const int64_t blk = (static_cast<int64_t>(split) * gridDim.y + bz) * ntile + (tile_m * g.n_tiles + tile_n);
    float4* ws = reinterpret_cast<float4*>(g.ws) + (blk * (NT / 64) + wave) * (TM * TN * 4) * 64;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          ws[((i * TN + j) * 4 + q) * 64 + lane] =
              make_float4(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
    return;
  } else {
    // ---- phase 1: accumulators -> T -> LDS tile [BM][BN] (row pitch BN*2 + 8 bytes) ----
    constexpr int PITCH = BN * 2 + 8;  // bytes
    uint8_t* sC = lds_raw;
    const T* bias = static_cast<const T*>(g.bias);
    // bias values of this lane's columns, loaded together ahead of the conversion loop (one
    // uniform branch around all of them: loads inside per-iteration branches wait one by one)
    float bv[TN][4][4];
    // the bias is not pitched: a tile that holds the ragged end of N (N not a multiple of 4) reads it element by element
    const bool bias_vec = VEC >= 4 && !((g.N & 3) != 0 && n0 + BN > g.N);
    if (EPI != EPI_ACT_BWD && bias != nullptr) {
      if (bias_vec) {
        uint2 braw[TN][4];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int nn = n0 + wn0 + j * 32 + q * 8 + (lane >> 5) * 4;
            braw[j][q] = *reinterpret_cast<const uint2*>(bias + (nn < g.N ? nn : 0));  // columns past N are never stored
          }
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const T* e4 = reinterpret_cast<const T*>(&braw[j][q]);
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[j][q][e] = elem<T>::to_float(e4[e]);
          }
      } else {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int nn = n0 + wn0 + j * 32 + q * 8 + (lane >> 5) * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[j][q][e] = elem<T>::to_float(bias[min(nn + e, g.N - 1)]);
          }
      }
    } else {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) bv[j][q][e] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nl = wn0 + j * 32 + q * 8 + (lane >> 5) * 4;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int ml = wm0 + i * 32 + (lane & 31);
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][q * 4 + e] * g.alpha + bv[j][q][e];
          store_pack<T, 4>(reinterpret_cast<T*>(sC + ml * PITCH + nl * 2), v);
        }
      }
    }
    // activation table behind the staged tile (LUT_OK: the kernel's LDS allocation has the room)
    const float2* act_tab = reinterpret_cast<const float2*>(sC + ((BM * PITCH + 15) & ~15));
    if constexpr (LUT_OK && (EPI == EPI_ACT_FWD || EPI == EPI_ACT_BWD)) {
      if (g.act_lut && g.act == NMTG_ACT_GELU) act_lut_fill<EPI == EPI_ACT_BWD>(const_cast<float2*>(act_tab), tid, NT);
    }
    __syncthreads();
    NMTG_PROF_MARK(3);

    // ---- phase 2: row-contiguous 8-element chunks, coalesced global traffic ----
    constexpr int CPR = BN / 8;        // chunks per tile row
    constexpr int RPP = NT / CPR;      // rows per pass
    constexpr int PASSES = BM / RPP;
    constexpr int GRP = PASSES < 8 ? PASSES : 8;   // passes whose side loads are issued together
    static_assert(NT % CPR == 0 && BM % RPP == 0 && PASSES % GRP == 0, "epilogue mapping");
    const int cc = tid % CPR, r_in = tid / CPR;
    const int n = n0 + cc * 8;
    const int ncols = g.N - n;         // valid columns of this lane's chunk (<= 0: none)
    uint16_t* C = reinterpret_cast<uint16_t*>(g.C) + static_cast<int64_t>(bz) * g.sC;
    uint16_t* AUX = reinterpret_cast<uint16_t*>(g.aux_out);
    if (AUX != nullptr) AUX += static_cast<int64_t>(bz) * g.sC;
    const uint16_t* HIN = reinterpret_cast<const uint16_t*>(g.aux_in);
    float csum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const bool use_dmask = (EPI == EPI_ACT_FWD || EPI == EPI_ACT_BWD) && g.dmask != nullptr;
    const bool dmask_in = use_dmask && !(EPI == EPI_ACT_FWD && g.rng);
    const bool tmask = EPI == EPI_SCORES && g.kmask_kind == 2;
    const uint8_t* side_mask = dmask_in ? g.dmask : tmask ? g.kmask : nullptr;   // [M, N] byte mask read per chunk
    uint2 padm = make_uint2(0, 0);
    if (EPI == EPI_SCORES && g.kmask_kind == 1)
      padm = load8_bytes<VEC>(g.kmask + static_cast<int64_t>(bz / g.heads) * g.N + n, g.kmask, ncols);

    if constexpr (EPI == EPI_SCORES_SOFTMAX || EPI == EPI_SCORES_SOFTMAX_RNG) {
      constexpr bool RNG = EPI == EPI_SCORES_SOFTMAX_RNG;
      // One wavefront per row: lane cc holds the row's elements 8 cc .. 8 cc + 7.
      static_assert(CPR == 64 && VEC == 8, "the row tile is 512 columns wide and moves 16-byte chunks");
      uint16_t* OUT2 = reinterpret_cast<uint16_t*>(g.out2) + static_cast<int64_t>(bz) * g.sC;
      const bool time_mask = g.kmask_kind == 2;
      const bool drop = g.dmask != nullptr;
      const bool replay = drop && !RNG;
      uint2 padm2 = make_uint2(0, 0);
      if (g.kmask_kind == 1) padm2 = load8_bytes<VEC>(g.kmask + static_cast<int64_t>(bz / g.heads) * g.N + n, g.kmask, ncols);
      constexpr float LOG2E = 1.4426950408889634f;
      [[maybe_unused]] const Philox gen(g.seed);
      for (int p0 = 0; p0 < PASSES; p0 += GRP) {
        uint2 traw[GRP], draw[GRP];
        if (time_mask) {
#pragma unroll
          for (int u = 0; u < GRP; ++u) {
            const int m = m0 + (p0 + u) * RPP + r_in;
            const int nv = m < g.M ? ncols : 0;
            traw[u] = load8_bytes<VEC, false>(g.kmask + static_cast<int64_t>(m < g.M ? m : 0) * g.N + (nv > 0 ? n : 0), g.kmask, nv);
          }
        } else {
#pragma unroll
          for (int u = 0; u < GRP; ++u) traw[u] = padm2;
        }
        if (replay) {
#pragma unroll
          for (int u = 0; u < GRP; ++u) {
            const int m = m0 + (p0 + u) * RPP + r_in;
            const int nv = m < g.M ? ncols : 0;
            const int64_t row = static_cast<int64_t>(bz) * g.M + (m < g.M ? m : 0);
            draw[u] = load8_bytes<VEC, false>(g.dmask + row * g.N + (nv > 0 ? n : 0), g.dmask, nv);
          }
        } else {
#pragma unroll
          for (int u = 0; u < GRP; ++u) draw[u] = make_uint2(0x01010101u, 0x01010101u);
        }
#pragma unroll
        for (int u = 0; u < GRP; ++u) {
          const int ml = (p0 + u) * RPP + r_in;
          const int m = m0 + ml;
          const int nv = m < g.M ? ncols : 0;
          float v[8];
          {
            const uint2* sp = reinterpret_cast<const uint2*>(sC + ml * PITCH + cc * 16);
            const uint2 lo = sp[0], hi = sp[1];
            unpack8<T>(make_uint4(lo.x, lo.y, hi.x, hi.y), v);
          }
          // masked keys and the columns past N count as -inf
#pragma unroll
          for (int k = 0; k < 8; ++k)
            if (byte_of(traw[u], k) || ncols <= 0) v[k] = -INFINITY;
          const int64_t off = static_cast<int64_t>(m) * g.ldc + n;
          store8<VEC>(C + off, pack8<T>(v), nv);
          float mx = v[0];
#pragma unroll
          for (int k = 1; k < 8; ++k) mx = fmaxf(mx, v[k]);
          mx = wave_max(mx);
          const float base = (mx == -INFINITY) ? 0.f : mx;   // a row without any key gives zeros
          float sum = 0.f;
#pragma unroll
          for (int k = 0; k < 8; ++k) { v[k] = fast_exp2((v[k] - base) * LOG2E); sum += v[k]; }
          sum = wave_sum(sum);
          const float inv = sum > 0.f ? 1.f / sum : 0.f;
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] *= inv;
          if (AUX != nullptr) store8<VEC>(AUX + off, pack8<T>(v), nv);
          if (drop) {
            uint2 keep = draw[u];
            if constexpr (RNG) {
              uint8_t kb[8];
              const uint64_t first = (static_cast<uint64_t>(bz) * g.M + m) * g.N + n;
              philox_keep<8>(gen, first, g.offset, g.keep_p, kb);
              keep.x = kb[0] | (kb[1] << 8) | (kb[2] << 16) | (static_cast<uint32_t>(kb[3]) << 24);
              keep.y = kb[4] | (kb[5] << 8) | (kb[6] << 16) | (static_cast<uint32_t>(kb[7]) << 24);
              store8_bytes<VEC>(const_cast<uint8_t*>(g.dmask) + first, keep, nv);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = byte_of(keep, k) ? v[k] * g.dscale : 0.f;
          }
          store8<VEC>(OUT2 + off, pack8<T>(v), nv);
        }
      }
      return;
    }

    if constexpr (EPI == EPI_DSOFTMAX) {
      static_assert(CPR == 64 && VEC == 8, "the row tile is 512 columns wide and moves 16-byte chunks");
      const uint16_t* SC = reinterpret_cast<const uint16_t*>(g.aux_in) + static_cast<int64_t>(bz) * g.sC;
      const bool drop = g.dmask != nullptr;
      constexpr float LOG2E = 1.4426950408889634f;
      for (int p0 = 0; p0 < PASSES; p0 += GRP) {
        uint4 sraw[GRP];
        uint2 draw[GRP];
#pragma unroll
        for (int u = 0; u < GRP; ++u) {
          const int m = m0 + (p0 + u) * RPP + r_in;
          const int nv = m < g.M ? ncols : 0;
          sraw[u] = load8<VEC, false>(SC + static_cast<int64_t>(m < g.M ? m : 0) * g.ldc + (nv > 0 ? n : 0), SC, nv);
        }
        if (drop) {
#pragma unroll
          for (int u = 0; u < GRP; ++u) {
            const int m = m0 + (p0 + u) * RPP + r_in;
            const int nv = m < g.M ? ncols : 0;
            const int64_t row = static_cast<int64_t>(bz) * g.M + (m < g.M ? m : 0);
            draw[u] = load8_bytes<VEC, false>(g.dmask + row * g.N + (nv > 0 ? n : 0), g.dmask, nv);
          }
        } else {
#pragma unroll
          for (int u = 0; u < GRP; ++u) draw[u] = make_uint2(0x01010101u, 0x01010101u);
        }
#pragma unroll
        for (int u = 0; u < GRP; ++u) {
          const int ml = (p0 + u) * RPP + r_in;
          const int m = m0 + ml;
          const int nv = m < g.M ? ncols : 0;
          float gr[8], pr[8];
          {
            const uint2* sp = reinterpret_cast<const uint2*>(sC + ml * PITCH + cc * 16);
            const uint2 lo = sp[0], hi = sp[1];
            unpack8<T>(make_uint4(lo.x, lo.y, hi.x, hi.y), gr);
          }
          unpack8<T>(sraw[u], pr);
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            if (ncols <= 0) { pr[k] = -INFINITY; gr[k] = 0.f; }            // columns past N
            else gr[k] = byte_of(draw[u], k) ? gr[k] * g.dscale : 0.f;      // g = keep * dP / (1 - p)
          }
          float mx = pr[0];
#pragma unroll
          for (int k = 1; k < 8; ++k) mx = fmaxf(mx, pr[k]);
          mx = wave_max(mx);
          const float base = (mx == -INFINITY) ? 0.f : mx;
          float sum = 0.f;
#pragma unroll
          for (int k = 0; k < 8; ++k) { pr[k] = fast_exp2((pr[k] - base) * LOG2E); sum += pr[k]; }
          sum = wave_sum(sum);
          const float inv = sum > 0.f ? 1.f / sum : 0.f;
          float dot = 0.f;
#pragma unroll
          for (int k = 0; k < 8; ++k) { pr[k] *= inv; dot += pr[k] * gr[k]; }
          dot = wave_sum(dot);
#pragma unroll
          for (int k = 0; k < 8; ++k) gr[k] = pr[k] * (gr[k] - dot);
          store8<VEC>(C + static_cast<int64_t>(m) * g.ldc + n, pack8<T>(gr), nv);
        }
      }
      return;
    }

    auto phase2 = [&](auto act_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    for (int p0 = 0; p0 < PASSES; p0 += GRP) {
      // side inputs of GRP passes first (independent loads in flight together), then the math and stores
      uint4 hraw[GRP];
      uint2 mraw[GRP];
      // Values of out-of-range chunks are never stored, so with 16-byte accesses the loads skip the
      // zeroing select (it would make each load wait for its own data); the mask branch encloses
      // the whole group so that its loads stay in one basic block.
      constexpr bool ZSIDE = VEC != 8;
      if constexpr (EPI == EPI_ACT_BWD) {
#pragma unroll
        for (int u = 0; u < GRP; ++u) {
          const int m = m0 + (p0 + u) * RPP + r_in;
          const int nv = m < g.M ? ncols : 0;
          hraw[u] = load8<VEC, ZSIDE>(HIN + static_cast<int64_t>(m < g.M ? m : 0) * g.ld_aux + (nv > 0 ? n : 0), HIN, nv);
        }
      }
      if (side_mask != nullptr) {
#pragma unroll
        for (int u = 0; u < GRP; ++u) {
          const int m = m0 + (p0 + u) * RPP + r_in;
          const int nv = m < g.M ? ncols : 0;
          mraw[u] = load8_bytes<VEC, ZSIDE>(side_mask + static_cast<int64_t>(m < g.M ? m : 0) * g.N + (nv > 0 ? n : 0), side_mask, nv);
        }
      } else {
#pragma unroll
        for (int u = 0; u < GRP; ++u) mraw[u] = make_uint2(0x01010101u, 0x01010101u);
      }
#pragma unroll
      for (int u = 0; u < GRP; ++u) {
        const int ml = (p0 + u) * RPP + r_in;
        const int m = m0 + ml;
        const int nv = m < g.M ? ncols : 0;
        float v[8];
        uint4 raw;
        {
          const uint2* s = reinterpret_cast<const uint2*>(sC + ml * PITCH + cc * 16);
          const uint2 lo = s[0], hi = s[1];
          raw = make_uint4(lo.x, lo.y, hi.x, hi.y);
          unpack8<T>(raw, v);
        }
        const int64_t off = static_cast<int64_t>(m) * g.ldc + n;
        if constexpr (EPI == EPI_PLAIN) {
          store8<VEC>(C + off, raw, nv);
        } else if constexpr (EPI == EPI_ACT_FWD) {
          if (AUX != nullptr) store8<VEC>(AUX + off, raw, nv);
          float a[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) a[k] = act_apply<ACT>(v[k], act_tab);
          if (use_dmask) {
            uint2 keep = mraw[u];
            if (g.rng) {
              uint8_t kb[8];
              const uint64_t first = static_cast<uint64_t>(m) * g.N + n;
              if ((g.N & 3) == 0) {
                philox_keep<8>(Philox(g.seed), first, g.offset, g.keep_p, kb);
              } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                  uint8_t one[1];
                  philox_keep<1>(Philox(g.seed), first + k, g.offset, g.keep_p, one);
                  kb[k] = one[0];
                }
              }
              keep.x = kb[0] | (kb[1] << 8) | (kb[2] << 16) | (static_cast<uint32_t>(kb[3]) << 24);
              keep.y = kb[4] | (kb[5] << 8) | (kb[6] << 16) | (static_cast<uint32_t>(kb[7]) << 24);
              store8_bytes<VEC>(const_cast<uint8_t*>(g.dmask) + static_cast<int64_t>(m) * g.N + n, keep, nv);
            }
            // keep bytes are 0 / 1: scale = float(byte) * 1/(1-p)
#pragma unroll
            for (int k = 0; k < 8; ++k) a[k] *= static_cast<float>(byte_of(keep, k)) * g.dscale;
          }
          store8<VEC>(C + off, pack8<T>(a), nv);
        } else if constexpr (EPI == EPI_ACT_BWD) {
          float h[8];
          unpack8<T>(hraw[u], h);
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] *= act_grad<ACT>(h[k], act_tab) * (static_cast<float>(byte_of(mraw[u], k)) * g.dscale);
          // the bias gradient sums the values as stored (rounded to T), as the reference does
          const uint4 packed = pack8<T>(v);
          float r[8];
          unpack8<T>(packed, r);
          if (nv > 0) {
#pragma unroll
            for (int k = 0; k < 8; ++k) csum[k] += (k < nv) ? r[k] : 0.f;
          }
          store8<VEC>(C + off, packed, nv);
        } else if constexpr (EPI == EPI_SCORES) {
          if (g.kmask_kind != 0) {
            const uint2 mk = g.kmask_kind == 1 ? padm : mraw[u];
#pragma unroll
            for (int k = 0; k < 8; ++k) if (byte_of(mk, k)) v[k] = -INFINITY;
          }
          store8<VEC>(C + off, pack8<T>(v), nv);
        }
      }
    }
    };
    if constexpr (EPI == EPI_ACT_FWD || EPI == EPI_ACT_BWD) dispatch_act<LUT_OK>(g.act, g.act_lut, phase2);
    else phase2(std::integral_constant<int, NMTG_ACT_NONE>{});

    NMTG_PROF_MARK(4);
    if constexpr (EPI == EPI_ACT_BWD) {
      if (g.colsum_part != nullptr) {
        __syncthreads();
        float* red = reinterpret_cast<float*>(lds_raw);  // [RPP][BN]
#pragma unroll
        for (int k = 0; k < 8; ++k) red[r_in * BN + cc * 8 + k] = csum[k];
        __syncthreads();
        for (int col = tid; col < BN; col += NT) {
          float s = 0.f;
          for (int r = 0; r < RPP; ++r) s += red[r * BN + col];
          if (n0 + col < g.N) g.colsum_part[static_cast<int64_t>(tile_m) * g.N + n0 + col] = s;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The kernel.
// ---------------------------------------------------------------------------------------------
template <int BM, int BN>
constexpr int gemm_lds_bytes() {
  constexpr int main_loop = 2 * (BM + BN) * GEMM_BK * 2;
  constexpr int c_tile = BM * (BN * 2 + 8);
  return main_loop > c_tile ? main_loop : c_tile;
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, int EPI, int VEC>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_kernel(const GemmArgs g) {
  constexpr int NT = 64 * WAVES_M * WAVES_N;
  constexpr int BK = GEMM_BK;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA tile");
  extern __shared__ __align__(16) uint8_t lds_raw[];
  T* sA = reinterpret_cast<T*>(lds_raw);
  T* sB = sA + 2 * BM * BK;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;

  // Tile coordinates. Consecutive block ids go round-robin to the 8 XCDs (each with its own L2), so
  // block ids are first regrouped to give every XCD a contiguous run of the tile order, and the
  // tile order itself walks groups of GM tile rows column by column: the ~32 tiles an XCD runs at
  // once then form a GM x 32/GM patch and share their A / B panels through that XCD's L2.
  int bid = blockIdx.x;
  const int ntile = g.m_tiles * g.n_tiles;
  if ((ntile & 7) == 0) bid = (bid & 7) * (ntile >> 3) + (bid >> 3);
  constexpr int GM = 4;
  const int in_group = GM * g.n_tiles;
  const int first_m = (bid / in_group) * GM;
  const int gsize = min(g.m_tiles - first_m, GM);
  const int tile_m = first_m + (bid % in_group) % gsize, tile_n = (bid % in_group) / gsize;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int bz = blockIdx.y, split = blockIdx.z;

  const T* A = static_cast<const T*>(g.A) + static_cast<int64_t>(bz) * g.sA;
  const T* B = static_cast<const T*>(g.B) + static_cast<int64_t>(bz) * g.sB;
  const int kbeg = split * g.k_per_split;
  const int kend = min(g.K, kbeg + g.k_per_split);
  const int nk = (kend - kbeg + BK - 1) / BK;

  acc16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  TileStage<T, BM, NT, A_KC, VEC> stA;
  TileStage<T, BN, NT, B_KC, VEC> stB;

  NMTG_PROF_MARK(0);
  if (nk > 0) {
    stA.load(A, g.lda, g.M, m0, kbeg, kend, tid);
    stB.load(B, g.ldb, g.N, n0, kbeg, kend, tid);
    stA.store(sA, tid);
    stB.store(sB, tid);
  }
  __syncthreads();

  NMTG_PROF_MARK(1);
  // per-lane LDS offsets of the MFMA fragments (elements), constant over the K loop
  int offA[TM][2], offB[TN][2];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = wm0 + i * 32 + (lane & 31);
    offA[i][0] = row * BK;
    offA[i][1] = lds_swz(row);
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int row = wn0 + j * 32 + (lane & 31);
    offB[j][0] = row * BK;
    offB[j][1] = lds_swz(row);
  }

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      stA.load(A, g.lda, g.M, m0, kbeg + (kt + 1) * BK, kend, tid);
      stB.load(B, g.ldb, g.N, n0, kbeg + (kt + 1) * BK, kend, tid);
    }
    const T* cA = sA + cur * BM * BK;
    const T* cB = sB + cur * BN * BK;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      uint4 fm[TM], fn[TN];
      const int c = kk * 2 + (lane >> 5);
#pragma unroll
      for (int i = 0; i < TM; ++i) fm[i] = *reinterpret_cast<const uint4*>(cA + offA[i][0] + ((c ^ offA[i][1]) * 8));
#pragma unroll
      for (int j = 0; j < TN; ++j) fn[j] = *reinterpret_cast<const uint4*>(cB + offB[j][0] + ((c ^ offB[j][1]) * 8));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma<T>::run(fn[j], fm[i], acc[i][j]);
    }
    if (kt + 1 < nk) {
      stA.store(sA + (cur ^ 1) * BM * BK, tid);
      stB.store(sB + (cur ^ 1) * BN * BK, tid);
    }
    __syncthreads();
  }

  NMTG_PROF_MARK(2);
  gemm_epilogue<T, BM, BN, WAVES_M, WAVES_N, EPI, VEC>(g, acc, lds_raw, tile_m, tile_n, bz, split);
}

// ---------------------------------------------------------------------------------------------
// Host-side description of one GEMM call; implemented in gemm.hip.
// ---------------------------------------------------------------------------------------------
enum GemmLayout { LAYOUT_NT = 0 /* A KC, B KC */, LAYOUT_NN = 1 /* A KC, B MC */, LAYOUT_TN = 2 /* A MC, B MC */ };

// Workspace bytes a split-K call of this shape needs (0 if it would not split).
size_t gemm_splitk_workspace_bytes(int M, int N, int K, int batch);

// Runs one GEMM. `epi` is a GemmEpi; for LAYOUT_TN with epi == EPI_PLAIN and a workspace the call
// may split K. Returns 0 or a negative nmtg_status; *m_tiles_out receives the number of row tiles
// used (= rows of colsum_part written by EPI_ACT_BWD).
int gemm_run(int dtype, int layout, int epi, GemmArgs a, void* workspace, size_t workspace_bytes, hipStream_t st,
             int* m_tiles_out = nullptr, GemmArgs* planned_out = nullptr);
// planned_out (optional) receives the arguments as launched (splits, tiles, vec, ws, tile_used): with a.defer_reduce
// set and planned_out->splits > 1 the caller owes the reduction of the partials (tail_add_splitk).
// dtype NMTG_F32 goes to the fp32 matrix-core kernel (gemm_f32.hip): plain and the two activation epilogues, no split-K.
int gemm_f32_run(int layout, int epi, GemmArgs a, hipStream_t st, int* m_tiles_out, GemmArgs* planned_out);
// Products with at most 32 rows against a row-major weight (the projections of a decoding step): one output column per
// wavefront (gemm_skinny.hip).
bool gemm_skinny_ok(int dtype, int layout, int epi, const GemmArgs& a);
int gemm_skinny_run(int dtype, const GemmArgs& a, hipStream_t st);

// Attention probabilities and context of an inference call in one kernel (flash_attn.hip): probs [batch * heads, tq, tk]
// = softmax over the keys of round(scale q k^T) with masked keys at -inf (rows without a live key: zeros), ctx = probs v;
// probs may be null (context only).
// The score tensor is never written. q, k, v, ctx: element (token t, sentence b, head h, :) at t * st + b * sb + h * sh.
struct AttnProbsCall {
  const void *q, *k, *v;
  void *ctx, *probs;
  int64_t q_st, q_sb, q_sh, k_st, k_sb, k_sh, v_st, v_sb, v_sh, c_st, c_sb, c_sh;
  const uint8_t* mask;      // mask_kind 1: [batch, tk] key padding; 2: [tq, tk] time mask; 1 = masked
  int mask_kind;
  int batch, heads, d, tq, tk;
  float scale;
  int dtype;
};
bool attn_probs_ok(const AttnProbsCall& c);    // NMTG_ATTN_PROBS=0 switches the kernel off
int attn_probs_run(const AttnProbsCall& c, hipStream_t st);

// Fused Q K^T -> mask -> softmax -> dropout (EPI_SCORES_SOFTMAX) for rows of at most 512 keys. `a` is filled as
// for EPI_SCORES plus out2 (dropped probabilities), aux_out (softmax, optional), dmask / rng / keep_p / dscale /
// seed / offset. Returns 1 if the kernel was launched, 0 if the call does not qualify (the caller then runs the
// scores GEMM and the softmax kernel), or a negative nmtg_status.
int gemm_scores_softmax_try(int dtype, GemmArgs a, hipStream_t st);
// Backward counterpart (EPI_DSOFTMAX): A = dctx, B = v, aux_in = saved scores, dmask / dscale for a replayed
// dropout mask, C = gradient of the scores. Same return convention.
int gemm_dsoftmax_try(int dtype, GemmArgs a, hipStream_t st);

}  // namespace nmtg
