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
#include "common.cuh"

namespace nmtg {

enum GemmEpi {
  EPI_PLAIN = 0,    // C = alpha*acc (+ bias[n])
  EPI_ACT_FWD = 1,  // h = acc + bias -> aux_out;  C = act(h) * keep * dscale
  EPI_ACT_BWD = 2,  // C = T(acc) * act'(aux_in) * dscale * keep (keep = 1 without a mask);  colsum_part[m_tile][n] = sum_m C
  EPI_SCORES = 3,   // C = alpha*acc, -inf where the key-padding / time mask is set
  EPI_SPLITK = 4    // fp32 partial tile -> workspace (reduced by splitk_reduce_kernel)
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
  int a_vec, b_vec, c_vec;  // widest legal vector (in elements: 8, 4 or 1) on each side
  const void* bias;
  void* aux_out;
  const void* aux_in;
  int64_t ld_aux;
  const uint8_t* dmask;     // dropout keep mask [M, N] dense; read, or written when rng != 0
  float dscale, keep_p;
  int rng;                  // ACT_FWD: draw the keep mask from Philox and store it to dmask
  uint64_t seed, offset;
  int act;
  float* colsum_part;
  const uint8_t* kmask;
  int kmask_kind, heads;
  float* ws;
  int m_tiles, n_tiles;
};

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
__device__ __forceinline__ float act_apply(float h, int act) {
  switch (act) {
    case NMTG_ACT_RELU: return fmaxf(h, 0.f);
    case NMTG_ACT_GELU: return 0.5f * h * (1.f + erff(h * 0.70710678118654752f));
    case NMTG_ACT_SILU: return h / (1.f + __expf(-h));
    case NMTG_ACT_AGELU: {
      const float u = 0.7978845608028654f * (h + 0.044715f * h * h * h);
      return 0.5f * h * (1.f + tanhf(u));
    }
    default: return h;
  }
}
__device__ __forceinline__ float act_grad(float h, int act) {
  switch (act) {
    case NMTG_ACT_RELU: return h > 0.f ? 1.f : 0.f;
    case NMTG_ACT_GELU: {
      const float cdf = 0.5f * (1.f + erff(h * 0.70710678118654752f));
      const float pdf = 0.3989422804014327f * __expf(-0.5f * h * h);
      return cdf + h * pdf;
    }
    case NMTG_ACT_SILU: {
      const float s = 1.f / (1.f + __expf(-h));
      return s * (1.f + h * (1.f - s));
    }
    case NMTG_ACT_AGELU: {
      const float k = 0.7978845608028654f;
      const float t = tanhf(k * (h + 0.044715f * h * h * h));
      return 0.5f * (1.f + t) + 0.5f * h * (1.f - t * t) * k * (1.f + 0.134145f * h * h);
    }
    default: return 1.f;
  }
}

// ---------------------------------------------------------------------------------------------
// Global -> register -> LDS staging of one operand tile [ROWS][64 k].
// ---------------------------------------------------------------------------------------------
template <typename T, int ROWS, int NT, bool KC>
struct TileStage {
  static constexpr int UNITS = KC ? ROWS * 8 : ROWS * 2;  // 16-byte chunks (KC) or 4k x 8row blocks (MC)
  static constexpr int PER = (UNITS + NT - 1) / NT;
  static constexpr int NREG = KC ? PER : PER * 4;
  uint4 regs[NREG];

  // base: operand pointer for this batch; rows_total / row0: extent and tile origin in the row
  // index; k0: first k of this step; kend: one past the last valid k.
  __device__ __forceinline__ void load(const T* __restrict__ base, int64_t ld, int rows_total, int row0, int k0,
                                       int kend, int vec, int tid) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = tid + i * NT;
      if constexpr (KC) {
        uint4 v = make_uint4(0, 0, 0, 0);
        const int row = q >> 3, c = q & 7;
        const int grow = row0 + row, gk = k0 + c * 8;
        if (q < UNITS && grow < rows_total && gk < kend) {
          const T* p = base + static_cast<int64_t>(grow) * ld + gk;
          if (vec == 8 && gk + 8 <= kend) {
            v = *reinterpret_cast<const uint4*>(p);
          } else if (vec >= 4 && gk + 8 <= kend) {
            const uint2 lo = *reinterpret_cast<const uint2*>(p), hi = *reinterpret_cast<const uint2*>(p + 4);
            v = make_uint4(lo.x, lo.y, hi.x, hi.y);
          } else {
            uint16_t e[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) e[j] = (gk + j < kend) ? reinterpret_cast<const uint16_t*>(p)[j] : 0;
            v = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
          }
        }
        regs[i] = v;
      } else {
        constexpr int RG8 = ROWS / 64 > 0 ? ROWS / 64 : 1;
        const int rg_lo = q & 7, kq_lo = (q >> 3) & 1, rest = q >> 4;
        const int rg = rg_lo + 8 * (rest % RG8), kq = kq_lo + 2 * (rest / RG8);
        const int grow = row0 + rg * 8;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          uint4 v = make_uint4(0, 0, 0, 0);
          const int gk = k0 + kq * 4 + kk;
          if (q < UNITS && gk < kend && grow < rows_total) {
            const T* p = base + static_cast<int64_t>(gk) * ld + grow;
            if (vec == 8 && grow + 8 <= rows_total) {
              v = *reinterpret_cast<const uint4*>(p);
            } else if (vec >= 4 && grow + 8 <= rows_total) {
              const uint2 lo = *reinterpret_cast<const uint2*>(p), hi = *reinterpret_cast<const uint2*>(p + 4);
              v = make_uint4(lo.x, lo.y, hi.x, hi.y);
            } else {
              uint16_t e[8];
#pragma unroll
              for (int j = 0; j < 8; ++j) e[j] = (grow + j < rows_total) ? reinterpret_cast<const uint16_t*>(p)[j] : 0;
              v = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
            }
          }
          regs[i * 4 + kk] = v;
        }
      }
    }
  }

  __device__ __forceinline__ void store(T* __restrict__ buf, int tid) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = tid + i * NT;
      if (q >= UNITS) continue;
      if constexpr (KC) {
        const int row = q >> 3, c = q & 7;
        *reinterpret_cast<uint4*>(buf + row * GEMM_BK + ((c ^ lds_swz(row)) * 8)) = regs[i];
      } else {
        constexpr int RG8 = ROWS / 64 > 0 ? ROWS / 64 : 1;
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
// The kernel.
// ---------------------------------------------------------------------------------------------
template <int BM, int BN>
constexpr int gemm_lds_bytes() {
  constexpr int main_loop = 2 * (BM + BN) * GEMM_BK * 2;
  constexpr int c_tile = BM * (BN * 2 + 8);
  return main_loop > c_tile ? main_loop : c_tile;
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, int EPI>
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

  // tile coordinates, XCD-aware
  int bid = blockIdx.x;
  const int ntile = g.m_tiles * g.n_tiles;
  if ((ntile & 7) == 0) bid = (bid & 7) * (ntile >> 3) + (bid >> 3);
  const int tile_m = bid / g.n_tiles, tile_n = bid % g.n_tiles;
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

  TileStage<T, BM, NT, A_KC> stA;
  TileStage<T, BN, NT, B_KC> stB;

  if (nk > 0) {
    stA.load(A, g.lda, g.M, m0, kbeg, kend, g.a_vec, tid);
    stB.load(B, g.ldb, g.N, n0, kbeg, kend, g.b_vec, tid);
    stA.store(sA, tid);
    stB.store(sB, tid);
  }
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      stA.load(A, g.lda, g.M, m0, kbeg + (kt + 1) * BK, kend, g.a_vec, tid);
      stB.load(B, g.ldb, g.N, n0, kbeg + (kt + 1) * BK, kend, g.b_vec, tid);
    }
    const T* cA = sA + cur * BM * BK;
    const T* cB = sB + cur * BN * BK;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      uint4 fm[TM], fn[TN];
      const int c = kk * 2 + (lane >> 5);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm0 + i * 32 + (lane & 31);
        fm[i] = *reinterpret_cast<const uint4*>(cA + row * BK + ((c ^ lds_swz(row)) * 8));
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wn0 + j * 32 + (lane & 31);
        fn[j] = *reinterpret_cast<const uint4*>(cB + row * BK + ((c ^ lds_swz(row)) * 8));
      }
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
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nl = wn0 + j * 32 + q * 8 + (lane >> 5) * 4;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (EPI != EPI_ACT_BWD && bias != nullptr) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n0 + nl + e < g.N) bv[e] = elem<T>::to_float(bias[n0 + nl + e]);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int ml = wm0 + i * 32 + (lane & 31);
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][q * 4 + e] * g.alpha + bv[e];
          store_pack<T, 4>(reinterpret_cast<T*>(sC + ml * PITCH + nl * 2), v);
        }
      }
    }
    __syncthreads();

    // ---- phase 2: row-contiguous 8-element chunks, coalesced global traffic ----
    constexpr int CPR = BN / 8;        // chunks per tile row
    constexpr int RPP = NT / CPR;      // rows per pass
    static_assert(NT % CPR == 0 && BM % RPP == 0, "epilogue mapping");
    const int cc = tid % CPR, r_in = tid / CPR;
    const int n = n0 + cc * 8;
    T* C = static_cast<T*>(g.C) + static_cast<int64_t>(bz) * g.sC;
    float csum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int nvalid = min(8, g.N - n);

    auto store8 = [&](T* dst, const float (&v)[8]) {
      if (nvalid == 8 && g.c_vec == 8) {
        store_pack<T, 8>(dst, v);
      } else if (nvalid == 8 && g.c_vec >= 4) {
        const float lo[4] = {v[0], v[1], v[2], v[3]}, hi[4] = {v[4], v[5], v[6], v[7]};
        store_pack<T, 4>(dst, lo);
        store_pack<T, 4>(dst + 4, hi);
      } else {
        for (int e = 0; e < nvalid; ++e) dst[e] = elem<T>::from_float(v[e]);
      }
    };
    auto load8 = [&](const T* src, float (&v)[8]) {
      if (nvalid == 8 && g.c_vec == 8) {
        load_pack<T, 8>(src, v);
      } else {
        for (int e = 0; e < 8; ++e) v[e] = e < nvalid ? elem<T>::to_float(src[e]) : 0.f;
      }
    };

    if (nvalid > 0) {
#pragma unroll 4
      for (int p = 0; p < BM / RPP; ++p) {
        const int ml = p * RPP + r_in;
        const int m = m0 + ml;
        if (m >= g.M) break;
        float v[8];
        {
          const uint2* s = reinterpret_cast<const uint2*>(sC + ml * PITCH + cc * 16);
          const uint2 lo = s[0], hi = s[1];
          const uint4 raw = make_uint4(lo.x, lo.y, hi.x, hi.y);
          const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] = elem<T>::to_float(e[k]);
        }
        const int64_t off = static_cast<int64_t>(m) * g.ldc + n;
        if constexpr (EPI == EPI_PLAIN) {
          store8(C + off, v);
        } else if constexpr (EPI == EPI_ACT_FWD) {
          if (g.aux_out != nullptr) store8(static_cast<T*>(g.aux_out) + static_cast<int64_t>(bz) * g.sC + off, v);
          float a[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) a[k] = act_apply(v[k], g.act);
          if (g.dmask != nullptr) {
            uint8_t* mk = const_cast<uint8_t*>(g.dmask) + static_cast<int64_t>(m) * g.N + n;
            uint8_t keep[8];
            if (g.rng) {
              const uint64_t first = static_cast<uint64_t>(m) * g.N + n;
              if ((g.N & 3) == 0) {
                philox_keep<8>(Philox(g.seed), first, g.offset, g.keep_p, keep);
              } else {
                for (int k = 0; k < 8; ++k) {
                  uint8_t one[1];
                  philox_keep<1>(Philox(g.seed), first + k, g.offset, g.keep_p, one);
                  keep[k] = one[0];
                }
              }
              if (nvalid == 8 && (g.N & 7) == 0) store_bytes<8>(mk, keep);
              else for (int k = 0; k < nvalid; ++k) mk[k] = keep[k];
            } else {
              if (nvalid == 8 && (g.N & 7) == 0) load_bytes<8>(mk, keep);
              else for (int k = 0; k < 8; ++k) keep[k] = k < nvalid ? mk[k] : 0;
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) a[k] = keep[k] ? a[k] * g.dscale : 0.f;
          }
          store8(C + off, a);
        } else if constexpr (EPI == EPI_ACT_BWD) {
          float h[8];
          load8(static_cast<const T*>(g.aux_in) + static_cast<int64_t>(m) * g.ld_aux + n, h);
#pragma unroll
          for (int k = 0; k < 8; ++k) v[k] *= act_grad(h[k], g.act) * g.dscale;
          if (g.dmask != nullptr) {
            const uint8_t* mk = g.dmask + static_cast<int64_t>(m) * g.N + n;
            uint8_t keep[8];
            if (nvalid == 8 && (g.N & 7) == 0) load_bytes<8>(mk, keep);
            else for (int k = 0; k < 8; ++k) keep[k] = k < nvalid ? mk[k] : 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = keep[k] ? v[k] : 0.f;
          }
          // the bias gradient sums the values as stored (rounded to T), as the reference does
#pragma unroll
          for (int k = 0; k < 8; ++k) { v[k] = elem<T>::to_float(elem<T>::from_float(v[k])); csum[k] += v[k]; }
          store8(C + off, v);
        } else if constexpr (EPI == EPI_SCORES) {
          if (g.kmask_kind != 0) {
            const uint8_t* mk = g.kmask_kind == 1 ? g.kmask + static_cast<int64_t>(bz / g.heads) * g.N + n
                                                  : g.kmask + static_cast<int64_t>(m) * g.N + n;
            for (int k = 0; k < nvalid; ++k) if (mk[k]) v[k] = -INFINITY;
          }
          store8(C + off, v);
        }
      }
    }

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

// Sums the split-K partials (in the accumulator layout written above), scales, converts to T and
// writes row-major C; fixed summation order.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, T* __restrict__ C, int64_t ldc,
                                                            int M, int N, int m_tiles, int n_tiles, int batch,
                                                            int64_t sC, int splits, float alpha, int c_vec) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int PER_BLK = NW * TM * TN * 4 * 64;  // float4 slots per tile
  const int64_t total = static_cast<int64_t>(batch) * m_tiles * n_tiles * PER_BLK;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
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
  for (int sp = 0; sp < splits; ++sp) {
    const float4 v = w[sp * per_split];
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  const float v[4] = {s.x * alpha, s.y * alpha, s.z * alpha, s.w * alpha};
  T* dst = C + static_cast<int64_t>(bz) * sC + static_cast<int64_t>(m) * ldc + n;
  if (n + 4 <= N && c_vec >= 4) store_pack<T, 4>(dst, v);
  else for (int e = 0; e < 4 && n + e < N; ++e) dst[e] = elem<T>::from_float(v[e]);
}

// Column sums of a row-major [M, N] matrix: partial[mb][n] over row blocks (fp32), fixed order.
template <typename T>
__global__ __launch_bounds__(256) void colsum_partial_kernel(const T* __restrict__ X, int64_t ld, int M, int N,
                                                             int rows_per_block, float* __restrict__ part) {
  // thread -> 2 adjacent columns x (256/32 = 8) row lanes
  __shared__ float red[8][64];
  const int cl = threadIdx.x & 31, rl = threadIdx.x >> 5;
  const int n = blockIdx.x * 64 + cl * 2;
  const int r0 = blockIdx.y * rows_per_block;
  const int r1 = min(M, r0 + rows_per_block);
  float s0 = 0.f, s1 = 0.f;
  if (n < N) {
    for (int r = r0 + rl; r < r1; r += 8) {
      const T* p = X + static_cast<int64_t>(r) * ld + n;
      s0 += elem<T>::to_float(p[0]);
      if (n + 1 < N) s1 += elem<T>::to_float(p[1]);
    }
  }
  red[rl][cl * 2] = s0;
  red[rl][cl * 2 + 1] = s1;
  __syncthreads();
  if (threadIdx.x < 64) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) s += red[k][threadIdx.x];
    const int col = blockIdx.x * 64 + threadIdx.x;
    if (col < N) part[static_cast<int64_t>(blockIdx.y) * N + col] = s;
  }
}

// out[n] = T(sum_p part[p][n]) in order p = 0..parts-1.
template <typename T>
__global__ __launch_bounds__(256) void colsum_final_kernel(const float* __restrict__ part, int parts, int N,
                                                           T* __restrict__ out) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float s = 0.f;
  for (int p = 0; p < parts; ++p) s += part[static_cast<int64_t>(p) * N + n];
  out[n] = elem<T>::from_float(s);
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
             int* m_tiles_out = nullptr);

// bias-gradient style column sums: out[n] = sum_m X[m][n]; part is fp32 scratch of
// colsum_parts(M) * N floats.
int colsum_parts(int M);
int colsum_run(int dtype, const void* X, int64_t ld, int M, int N, float* part, void* out, hipStream_t st);
int colsum_finish(int dtype, const float* part, int parts, int N, void* out, hipStream_t st);

}  // namespace nmtg
