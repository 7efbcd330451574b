// GEMM main loop fed by a ring of LDS slots that the gfx950 direct global -> LDS loads fill several
// 64-k steps ahead of the MFMA work.
//
// Why a second main loop: with one 64-k step of prefetch (the two-buffer loop in gemm.hip.h) a step
// cannot be shorter than the latency of its own loads (~2000 clocks on a loaded chip), while the
// MFMA work of a 128x128 step is 256 clocks and that of a 256x256 step 2048. Keeping several steps
// in flight turns the loads from a latency into a throughput problem (measured: ~44 B/clk/CU from L2
// with >= 64 KB in flight against ~28 B/clk/CU with one step in flight).
//
// Layout. A slot holds 128 operand rows x 64 k (16 KB). A stage (one 64-k step of the block tile)
// is SA = BM/128 slots of A followed by SB = BN/128 slots of B; slots are issued in that order for
// stage 0, 1, 2, ... and slot number q lives at ring position q % RING. RING >= 2 (SA + SB), so
// while stage s is multiplied the slots of stage s+1 (and part of s+2) are landing.
//   reduction-contiguous operand ("KC", element (row, k) at base[row * ld + k]):
//     slot = [128 rows][8 chunks of 16 B], chunk position c' of row r holds k-chunk c' ^ swz(r);
//     MFMA fragments are read with ds_read_b128.
//   row-contiguous operand ("MC", element (row, k) at base[k * ld + row]):
//     slot = [64 k][16 chunks of 16 B], chunk position c' of k-row k holds row-chunk c' ^ 4 (k & 3);
//     MFMA fragments are read with the LDS transpose read (ds_read_b64_tr_b16): the 16 lanes of a
//     group read 4 k-rows x 16 rows and each lane receives the 4 consecutive k of its own row.
// Both are filled by one-kilobyte transfers (64 lanes x 16 B, LDS destination contiguous, the
// swizzle applied on the global side), 16 per slot, dealt round-robin to the wavefronts.
//
// The transfers are issued from inline assembly: the compiler orders every LDS read behind all
// outstanding LDS-DMA it knows of (vmcnt(0)), which would serialise the ring. The waits are
// therefore explicit: vmcnt counts this wavefront's transfers in issue order, and before the
// barrier that ends stage s each wavefront waits until only the transfers issued after stage s+1's
// are outstanding.
//
// Requirements (checked on the host, the two-buffer kernel takes everything else): 16-bit
// elements, K a multiple of 64 per split, 16-byte aligned operands and leading dimensions, operand
// extents below 4 GB (32-bit lane offsets).
#pragma once
#include "gemm.hip.h"

#include <type_traits>

namespace nmtg {

constexpr int RING_SLOT_BYTES = 128 * GEMM_BK * 2;

typedef short short4_t __attribute__((ext_vector_type(4)));

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// One transfer: lane l copies the 16 bytes at sbase + voff(l) to LDS address lds_addr + 16 l.
// M0 carries the LDS address. The compiler warns that M0 is a reserved register it will not save
// around the statement; that is what is wanted: on gfx9 it only ever writes M0 immediately before
// an instruction of its own that reads it, never keeps a value in it across other code.
__device__ __forceinline__ void dma16(uint32_t voff, const void* sbase, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(sbase), "s"(lds_addr)
               : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
}
// Waits until at most min(n, MAX) transfers of this wavefront are outstanding; n is a multiple of STEP.
template <int MAX, int STEP>
__device__ __forceinline__ void wait_vmcnt_upto(int n) {
  if constexpr (MAX <= 0) {
    wait_vmcnt<0>();
  } else {
    if (n >= MAX) wait_vmcnt<MAX>();
    else wait_vmcnt_upto<MAX - STEP, STEP>(n);
  }
}

// All LDS reads of this wavefront done, then the workgroup barrier (also a compiler barrier).
__device__ __forceinline__ void ring_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int BM, int BN, int RING>
constexpr int gemm_ring_lds_bytes() {
  constexpr int main_loop = RING * RING_SLOT_BYTES;
  constexpr int c_tile = ((BM * (BN * 2 + 8) + 15) & ~15) + ACT_LUT_BYTES;   // staged output tile + activation table
  return main_loop > c_tile ? main_loop : c_tile;
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, int EPI, int RING>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_ring_kernel(const GemmArgs g) {
  constexpr int NT = 64 * WAVES_M * WAVES_N, NW = NT / 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int SA = BM / 128, SB = (BN + 127) / 128, SPS = SA + SB;
  constexpr int IPS = 16 / NW;  // transfers per wavefront per slot
  // BN = 64 (the per-head products) fills a whole B slot too: its upper 64 rows hold clamped duplicates no
  // fragment reads, which keeps the transfer count per slot uniform for the vmcnt bookkeeping.
  static_assert(BM % 128 == 0 && (BN % 128 == 0 || BN == 64), "block tile is a whole number of slots (or a 64-row B tile)");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && 128 % WTM == 0 && 128 % WTN == 0, "a wave tile lies inside one slot");
  static_assert(16 % NW == 0, "slots are dealt evenly to the wavefronts");
  static_assert(RING >= 2 * SPS, "the ring must hold the stage being read and the next one");
  static_assert((RING - SPS) * IPS < 64, "vmcnt range");
  extern __shared__ __align__(16) uint8_t lds_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WAVES_N) * WTM, wn0 = (wave % WAVES_N) * WTN;

  // tile order: see gemm_kernel
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

  const int kbeg = split * g.k_per_split;
  const int kend = min(g.K, kbeg + g.k_per_split);
  const int nk = (kend - kbeg) / GEMM_BK;  // whole steps only (host guarantee)
  const int total = nk * SPS;

  const int64_t lda_b = g.lda * 2, ldb_b = g.ldb * 2;  // bytes
  const char* a_base = static_cast<const char*>(g.A) + static_cast<int64_t>(bz) * g.sA * 2 + static_cast<int64_t>(kbeg) * (A_KC ? 2 : lda_b);
  const char* b_base = static_cast<const char*>(g.B) + static_cast<int64_t>(bz) * g.sB * 2 + static_cast<int64_t>(kbeg) * (B_KC ? 2 : ldb_b);
  const int64_t step_a = A_KC ? GEMM_BK * 2 : GEMM_BK * lda_b;
  const int64_t step_b = B_KC ? GEMM_BK * 2 : GEMM_BK * ldb_b;

  // per-lane source offsets of this wavefront's transfers (bytes from a_base / b_base at k = 0 of a stage)
  uint32_t dA[SA][IPS], dB[SB][IPS];
  auto lane_offsets = [&](auto kc_tag, int rows_total, int row0, int64_t ld_b, int j, int i) -> uint32_t {
    const int ii = i * NW + wave;
    if constexpr (decltype(kc_tag)::value) {
      const int r = 8 * ii + (lane >> 3);
      const int c = (lane & 7) ^ lds_swz(r);
      const int row = min(row0 + 128 * j + r, rows_total - 1);
      return static_cast<uint32_t>(static_cast<int64_t>(row) * ld_b + c * 16);
    } else {
      const int k = 4 * ii + (lane >> 4);
      const int c = (lane & 15) ^ (4 * ((lane >> 4) & 3));
      const int row = min(row0 + 128 * j + 8 * c, (rows_total - 1) & ~7);   // last (possibly partial) aligned group of 8 rows
      return static_cast<uint32_t>(static_cast<int64_t>(k) * ld_b + row * 2);
    }
  };
#pragma unroll
  for (int j = 0; j < SA; ++j)
#pragma unroll
    for (int i = 0; i < IPS; ++i) dA[j][i] = lane_offsets(std::integral_constant<bool, A_KC>{}, g.M, m0, lda_b, j, i);
#pragma unroll
  for (int j = 0; j < SB; ++j)
#pragma unroll
    for (int i = 0; i < IPS; ++i) dB[j][i] = lane_offsets(std::integral_constant<bool, B_KC>{}, g.N, n0, ldb_b, j, i);

  // Issues slot j of a stage whose k = 0 is at (a_stage, b_stage) into ring position pos.
  auto issue = [&](auto jtag, const char* a_stage, const char* b_stage, int pos) {
    constexpr int j = decltype(jtag)::value;
    const uint32_t dst = static_cast<uint32_t>(pos * RING_SLOT_BYTES + wave * 1024);
#pragma unroll
    for (int i = 0; i < IPS; ++i) {
      if constexpr (j < SA) dma16(dA[j][i], a_stage, dst + i * NW * 1024);
      else dma16(dB[j - SA][i], b_stage, dst + i * NW * 1024);
    }
  };

  // per-lane LDS offsets of the MFMA fragments inside a slot
  const int ja = wm0 / 128, jb = wn0 / 128;
  uint32_t fa[TM][A_KC ? 4 : 1], fb[TN][B_KC ? 4 : 1];
  auto frag_offsets = [&](auto kc_tag, int r0, int i, int kk) -> uint32_t {
    if constexpr (decltype(kc_tag)::value) {
      const int row = r0 + 32 * i + (lane & 31);
      return static_cast<uint32_t>(row * 128 + (((2 * kk + (lane >> 5)) ^ lds_swz(row)) * 16));
    } else {
      const int kq = 8 * (lane >> 5) + ((lane >> 2) & 3);
      const int c = r0 / 8 + 4 * i + 2 * ((lane >> 4) & 1) + ((lane >> 1) & 1);
      const int cp = c ^ (4 * ((lane >> 2) & 3));
      return static_cast<uint32_t>(kq * 256 + cp * 16 + (lane & 1) * 8);
    }
  };
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int kk = 0; kk < (A_KC ? 4 : 1); ++kk) fa[i][kk] = frag_offsets(std::integral_constant<bool, A_KC>{}, wm0 % 128, i, kk);
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int kk = 0; kk < (B_KC ? 4 : 1); ++kk) fb[j][kk] = frag_offsets(std::integral_constant<bool, B_KC>{}, wn0 % 128, j, kk);

  acc16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  NMTG_PROF_MARK(0);
  // ---- prologue: fill the ring ----
  static_for<0, RING>([&](auto tt) {
    constexpr int t = decltype(tt)::value;
    constexpr int j = t % SPS, st = t / SPS;
    if (st < nk) issue(std::integral_constant<int, j>{}, a_base + st * step_a, b_base + st * step_b, t);
  });
  if (nk > 0) wait_vmcnt_upto<(RING - SPS) * IPS, IPS>((min(RING, total) - SPS) * IPS);
  ring_barrier();

  NMTG_PROF_MARK(1);
  int pos_r = 0, pos_w = 0;
  const char* a_cur = a_base - step_a;  // stage s - 1 at the top of iteration s
  const char* b_cur = b_base - step_b;
  for (int s = 0; s < nk; ++s) {
    if (s >= 1) {
      // the slots of stage s - 1 are free: issue the next SPS slots of the sequence
      static_for<0, SPS>([&](auto tt) {
        constexpr int t = decltype(tt)::value;
        constexpr int j = (RING + t) % SPS, d = (RING + t) / SPS;
        if (s - 1 + d < nk) issue(std::integral_constant<int, j>{}, a_cur + d * step_a, b_cur + d * step_b, pos_w);
        pos_w = (pos_w + 1 == RING) ? 0 : pos_w + 1;
      });
    }
    a_cur += step_a;
    b_cur += step_b;

    int pa = pos_r + ja, pb = pos_r + SA + jb;
    if (pa >= RING) pa -= RING;
    if (pb >= RING) pb -= RING;
    const uint8_t* sa = lds_raw + pa * RING_SLOT_BYTES;
    const uint8_t* sb = lds_raw + pb * RING_SLOT_BYTES;
    // Fragments are double-buffered in registers: the LDS reads of k-group kk + 1 are issued ahead of the MFMAs of
    // k-group kk, so the matrix pipe does not wait for the LDS latency (with the 128x128 tile there is one wavefront
    // per SIMD and nothing else to hide it).
    uint4 fm[2][TM], fn[2][TN];
    auto load_frags = [&](auto kk_tag, uint4 (&fm_)[TM], uint4 (&fn_)[TN]) {
      constexpr int kk = decltype(kk_tag)::value;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        if constexpr (A_KC) {
          fm_[i] = *reinterpret_cast<const uint4*>(sa + fa[i][kk]);
        } else {
          const uint8_t* p = sa + fa[i][0] + kk * 16 * 256;
          const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(p));
          const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(p + 4 * 256));
          union { short4_t s[2]; uint4 u; } cv;
          cv.s[0] = lo;
          cv.s[1] = hi;
          fm_[i] = cv.u;
        }
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (B_KC) {
          fn_[j] = *reinterpret_cast<const uint4*>(sb + fb[j][kk]);
        } else {
          const uint8_t* p = sb + fb[j][0] + kk * 16 * 256;
          const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(p));
          const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(p + 4 * 256));
          union { short4_t s[2]; uint4 u; } cv;
          cv.s[0] = lo;
          cv.s[1] = hi;
          fn_[j] = cv.u;
        }
      }
    };
    load_frags(std::integral_constant<int, 0>{}, fm[0], fn[0]);
    static_for<0, GEMM_BK / 16>([&](auto kk_tag) {
      constexpr int kk = decltype(kk_tag)::value;
      if constexpr (kk + 1 < GEMM_BK / 16) load_frags(std::integral_constant<int, kk + 1>{}, fm[(kk + 1) & 1], fn[(kk + 1) & 1]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma<T>::run(fn[kk & 1][j], fm[kk & 1][i], acc[i][j]);
    });
    // Pin that order (the scheduler otherwise sinks the reads back down to save registers): the first k-group's reads,
    // then for every k-group its MFMAs with the next group's reads dealt out one per MFMA from the start.
    constexpr int READS = (A_KC ? TM : 2 * TM) + (B_KC ? TN : 2 * TN);   // LDS read instructions per k-group
    constexpr int MFMAS = TM * TN;
    __builtin_amdgcn_sched_group_barrier(0x100, READS, 0);
    static_for<0, GEMM_BK / 16>([&](auto kk_tag) {
      constexpr int kk = decltype(kk_tag)::value;
      if constexpr (kk + 1 < GEMM_BK / 16) {
        constexpr int PAIRS = READS < MFMAS ? READS : MFMAS;
        static_for<0, PAIRS>([&](auto) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        });
        if constexpr (READS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x100, READS - PAIRS, 0);
        if constexpr (MFMAS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - PAIRS, 0);
      } else {
        __builtin_amdgcn_sched_group_barrier(0x008, MFMAS, 0);
      }
    });
    pos_r += SPS;
    if (pos_r >= RING) pos_r -= RING;

    // stage s + 1 must have landed for every wavefront before anyone reads it
    if (s + 1 < nk) {
      const int issued = min(RING + s * SPS, total);
      wait_vmcnt_upto<(RING - 2 * SPS) * IPS, IPS>((issued - (s + 2) * SPS) * IPS);
    }
    ring_barrier();
  }

  NMTG_PROF_MARK(2);
  gemm_epilogue<T, BM, BN, WAVES_M, WAVES_N, EPI, 8, true>(g, acc, lds_raw, tile_m, tile_n, bz, split);
}

}  // namespace nmtg
