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

// STEPBUF = false: a step reads its operand fragments from LDS k-group by k-group, one k-group ahead of the MFMAs
// that use them, and ends with the wait for the next stage and the barrier: the matrix pipe drains there, which two
// wavefronts per SIMD (the 256x256 tile) cover in part and a single one (the 128x128 tile) does not.
// STEPBUF = true (one wavefront per SIMD): "phase p" reads the fragments of the whole stage p into one of two register
// sets while it multiplies stage p - 1 out of the other. The phase starts with the MFMAs of the first k-group, then
// waits for stage p's transfers, passes the barrier (the reads of phase p - 1 have had those MFMAs to land; behind the
// barrier every wavefront is done with stage p - 1's slots, which are refilled right there) and deals stage p's reads
// out between the MFMAs of the remaining k-groups. The matrix pipe has work on both sides of the barrier. Phase 0
// only reads, one more phase without reads follows the last stage; the ring positions and the vmcnt bookkeeping are
// those of the plain loop.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, int EPI, int RING, bool STEPBUF = false>
__device__ __forceinline__ void gemm_ring_body(const GemmArgs& g, int block_x) {
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
  int bid = block_x;
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
  // A reduction-contiguous operand is addressed from the first row of this block's tile (64-bit, scalar), so that the
  // per-lane offsets span one tile's rows and fit 32 bits whatever the size of the operand.
  const char* a_base = static_cast<const char*>(g.A) + static_cast<int64_t>(bz) * g.sA * 2 + static_cast<int64_t>(kbeg) * (A_KC ? 2 : lda_b) +
                       (A_KC ? static_cast<int64_t>(m0) * lda_b : 0);
  const char* b_base = static_cast<const char*>(g.B) + static_cast<int64_t>(bz) * g.sB * 2 + static_cast<int64_t>(kbeg) * (B_KC ? 2 : ldb_b) +
                       (B_KC ? static_cast<int64_t>(n0) * ldb_b : 0);
  const int64_t step_a = A_KC ? GEMM_BK * 2 : GEMM_BK * lda_b;
  const int64_t step_b = B_KC ? GEMM_BK * 2 : GEMM_BK * ldb_b;

  // per-lane source offsets of this wavefront's transfers (bytes from a_base / b_base at k = 0 of a stage)
  uint32_t dA[SA][IPS], dB[SB][IPS];
  auto lane_offsets = [&](auto kc_tag, int rows_total, int row0, int64_t ld_b, int j, int i) -> uint32_t {
    const int ii = i * NW + wave;
    if constexpr (decltype(kc_tag)::value) {
      const int r = 8 * ii + (lane >> 3);
      const int c = (lane & 7) ^ lds_swz(r);
      const int row = min(row0 + 128 * j + r, rows_total - 1) - row0;      // from the tile's first row (see a_base)
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

  // LDS address of the ring (the transfers name their destination by address, not through a pointer)
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_raw)));
  // Issues slot j of a stage whose k = 0 is at (a_stage, b_stage) into ring position pos.
  auto issue = [&](auto jtag, const char* a_stage, const char* b_stage, int pos) {
    constexpr int j = decltype(jtag)::value;
    const uint32_t dst = lds_base + static_cast<uint32_t>(pos * RING_SLOT_BYTES + wave * 1024);
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
  constexpr int KG = GEMM_BK / 16;                                        // k-groups (MFMA depths) per stage
  constexpr int READS = (A_KC ? TM : 2 * TM) + (B_KC ? TN : 2 * TN);     // LDS read instructions per k-group
  constexpr int MFMAS = TM * TN;
  auto load_frags = [&](auto kk_tag, const uint8_t* sa, const uint8_t* sb, uint4 (&fm_)[TM], uint4 (&fn_)[TN]) {
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
  int pos_r = 0, pos_w = 0;
  const char* a_cur = a_base - step_a;  // stage p - 1 at the top of phase p
  const char* b_cur = b_base - step_b;
  // Top of phase p >= 1: the slots of stage p - 1 are free (every wavefront has passed the barrier behind its reads):
  // issue the next SPS slots of the sequence.
  auto refill = [&](int p) {
    if (p >= 1) {
      static_for<0, SPS>([&](auto tt) {
        constexpr int t = decltype(tt)::value;
        constexpr int j = (RING + t) % SPS, d = (RING + t) / SPS;
        if (p - 1 + d < nk) issue(std::integral_constant<int, j>{}, a_cur + d * step_a, b_cur + d * step_b, pos_w);
        pos_w = (pos_w + 1 == RING) ? 0 : pos_w + 1;
      });
    }
    a_cur += step_a;
    b_cur += step_b;
  };
  if constexpr (!STEPBUF) {
    // Fragments are double-buffered in registers by k-group: the LDS reads of a k-group are issued under the MFMAs of
    // the one before. The wait for the next stage and the barrier sit in front of the LAST k-group's MFMAs, not behind
    // them: by then every read of the stage has been issued (and has had a k-group's MFMAs to land), so the slots can be
    // handed back, and the last k-group multiplies out of registers while the first reads of the next stage go out. The
    // matrix pipe has work on both sides of the barrier.
    uint4 fm[2][TM], fn[2][TN];
    auto mfmas = [&](auto buf_tag) {
      constexpr int Bf = decltype(buf_tag)::value;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma<T>::run(fn[Bf][j], fm[Bf][i], acc[i][j]);
    };
    auto pin_pairs = [&]() {   // the MFMAs of one k-group with the reads of another dealt out one per MFMA from the start
      constexpr int PAIRS = READS < MFMAS ? READS : MFMAS;
      static_for<0, PAIRS>([&](auto) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      });
      if constexpr (READS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x100, READS - PAIRS, 0);
      if constexpr (MFMAS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - PAIRS, 0);
    };
    static_assert(KG % 2 == 0, "the fragment buffers alternate by k-group and the loop carries buffer 0 across steps");
    auto slots_of = [&](int pos, const uint8_t*& sa, const uint8_t*& sb) {
      int pa = pos + ja, pb = pos + SA + jb;
      if (pa >= RING) pa -= RING;
      if (pb >= RING) pb -= RING;
      sa = lds_raw + pa * RING_SLOT_BYTES;
      sb = lds_raw + pb * RING_SLOT_BYTES;
    };
    const uint8_t *sa, *sb;
    if (nk > 0) {
      refill(0);   // nothing to issue yet: moves the operand cursors onto stage 0
      slots_of(0, sa, sb);
      load_frags(std::integral_constant<int, 0>{}, sa, sb, fm[0], fn[0]);
    }
    // k-groups 0 .. KG - 2 of a stage, each under the reads of the next one
    auto leading_groups = [&]() {
      static_for<0, KG - 1>([&](auto kk_tag) {
        constexpr int kk = decltype(kk_tag)::value;
        load_frags(std::integral_constant<int, kk + 1>{}, sa, sb, fm[(kk + 1) & 1], fn[(kk + 1) & 1]);
        mfmas(std::integral_constant<int, kk & 1>{});
      });
      static_for<0, KG - 1>([&](auto) { pin_pairs(); });
    };
    // every stage but the last (the last one is peeled off: with the MFMAs of a step in two branches the accumulators
    // are copied where the branches join)
    for (int s = 0; s + 1 < nk; ++s) {
      leading_groups();
      pos_r += SPS;
      if (pos_r >= RING) pos_r -= RING;
      // stage s + 1 must have landed for every wavefront, and every wavefront must be done reading stage s
      const int issued = min(RING + s * SPS, total);
      wait_vmcnt_upto<(RING - 2 * SPS) * IPS, IPS>((issued - (s + 2) * SPS) * IPS);
      ring_barrier();
      slots_of(pos_r, sa, sb);
      load_frags(std::integral_constant<int, 0>{}, sa, sb, fm[0], fn[0]);
      mfmas(std::integral_constant<int, (KG - 1) & 1>{});
      pin_pairs();
      refill(s + 1);   // into the slots of stage s, behind the MFMAs that keep the pipe busy right after the barrier
    }
    if (nk > 0) {
      leading_groups();
      mfmas(std::integral_constant<int, (KG - 1) & 1>{});
      ring_barrier();   // every wavefront is done reading the ring: the epilogue stages the output tile there
    }
  } else {
    // Two register sets of a whole stage's fragments; phases alternate between them. Phase 0 only reads, the phase
    // behind the last stage only multiplies; they are peeled off so that the loop body is two straight middle phases
    // (with the MFMAs in branches the accumulators end up in different registers on different paths and are copied
    // at every join).
    uint4 fmS[2][KG][TM], fnS[2][KG][TN];
    auto stage_slots = [&](const uint8_t*& sa, const uint8_t*& sb) {
      int pa = pos_r + ja, pb = pos_r + SA + jb;
      if (pa >= RING) pa -= RING;
      if (pb >= RING) pb -= RING;
      sa = lds_raw + pa * RING_SLOT_BYTES;
      sb = lds_raw + pb * RING_SLOT_BYTES;
      pos_r += SPS;
      if (pos_r >= RING) pos_r -= RING;
    };
    auto multiply = [&](auto set_tag) {
      constexpr int Q = decltype(set_tag)::value;
      static_for<0, KG>([&](auto kk_tag) {
        constexpr int kk = decltype(kk_tag)::value;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) mfma<T>::run(fnS[Q][kk][j], fmS[Q][kk][i], acc[i][j]);
      });
    };
    // End of the first k-group of phase p >= 1: stage p must have landed for every wavefront, and every wavefront must be
    // done with its reads of stage p - 1 (issued in phase p - 1; their last ones land under this phase's first MFMAs).
    auto certify_cur = [&](int p) {
      const int issued = min(RING + (p - 1) * SPS, total);
      wait_vmcnt_upto<(RING - 2 * SPS) * IPS, IPS>((issued - (p + 1) * SPS) * IPS);
      ring_barrier();
    };
    auto middle = [&](auto par_tag, int p) {
      constexpr int P = decltype(par_tag)::value;   // set written in this phase; the MFMAs read set P ^ 1
      const uint8_t *sa, *sb;
      stage_slots(sa, sb);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma<T>::run(fnS[P ^ 1][0][j], fmS[P ^ 1][0][i], acc[i][j]);
      certify_cur(p);
      // the other k-groups of stage p - 1, with all of stage p's reads dealt out between them; the refill of the freed
      // slots goes out behind the first of them, so that MFMAs follow the barrier at once
      constexpr int NM = (KG - 1) * MFMAS, NR = KG * READS;
      load_frags(std::integral_constant<int, 0>{}, sa, sb, fmS[P][0], fnS[P][0]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma<T>::run(fnS[P ^ 1][1][j], fmS[P ^ 1][1][i], acc[i][j]);
      {
        constexpr int PAIRS = READS < MFMAS ? READS : MFMAS;
        static_for<0, PAIRS>([&](auto) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        });
        if constexpr (READS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x100, READS - PAIRS, 0);
        if constexpr (MFMAS > PAIRS) __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - PAIRS, 0);
      }
      refill(p);
      static_for<1, KG>([&](auto kk_tag) {
        constexpr int kk = decltype(kk_tag)::value;
        load_frags(kk_tag, sa, sb, fmS[P][kk], fnS[P][kk]);
        if constexpr (kk >= 2) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) mfma<T>::run(fnS[P ^ 1][kk][j], fmS[P ^ 1][kk][i], acc[i][j]);
        }
      });
      {
        constexpr int NM2 = (KG - 2) * MFMAS, NR2 = (KG - 1) * READS;
        static_for<0, NM2>([&](auto it) {
          constexpr int i = decltype(it)::value;
          constexpr int r = (i + 1) * NR2 / NM2 - i * NR2 / NM2;
          if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        });
      }
      (void)NM; (void)NR;
    };
    if (nk > 0) {
      {
        refill(0);
        const uint8_t *sa, *sb;
        stage_slots(sa, sb);
        static_for<0, KG>([&](auto kk_tag) {
          constexpr int kk = decltype(kk_tag)::value;
          load_frags(kk_tag, sa, sb, fmS[0][kk], fnS[0][kk]);
        });
      }
      int p = 1;
      for (; p + 1 < nk; p += 2) {
        middle(std::integral_constant<int, 1>{}, p);
        middle(std::integral_constant<int, 0>{}, p + 1);
      }
      if (p < nk) {
        middle(std::integral_constant<int, 1>{}, p);
        multiply(std::integral_constant<int, 1>{});
      } else {
        multiply(std::integral_constant<int, 0>{});
      }
      ring_barrier();   // every wavefront is done reading the ring: the epilogue stages the output tile there
    }
  }

  NMTG_PROF_MARK(2);
  gemm_epilogue<T, BM, BN, WAVES_M, WAVES_N, EPI, 8, true>(g, acc, lds_raw, tile_m, tile_n, bz, split);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, int EPI, int RING, bool STEPBUF = false>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_ring_kernel(const GemmArgs g) {
  gemm_ring_body<T, BM, BN, WAVES_M, WAVES_N, A_KC, B_KC, EPI, RING, STEPBUF>(g, static_cast<int>(blockIdx.x));
}

// The same kernel with riders: the first g.rider_blocks blocks of the grid's x extent (first batch and split only) run
// a list of small reduction jobs instead of a tile (reduce.hip.h). A product that leaves one block on a CU has room
// for a second one there; the riders' loads and adds fill the memory pipes that the main loop leaves idle, and the
// launches those jobs would otherwise need fall away. The jobs are independent of this product. The riders come
// first, one per CU, so that the tiles that follow spread over the CUs as they would without them.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KC, bool B_KC, int EPI, int RING, bool STEPBUF = false>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_ring_rider_kernel(const GemmArgs g, const TailArgs riders) {
  static_assert(64 * WAVES_M * WAVES_N == 256, "the reduction jobs are written for blocks of 256 threads");
  if (static_cast<int>(blockIdx.x) < g.rider_blocks) {
    extern __shared__ __align__(16) uint8_t lds_raw[];   // the launch's ring memory: far more than a rider needs
    if (blockIdx.y == 0 && blockIdx.z == 0)
      tail_ride<T>(riders, static_cast<int>(blockIdx.x), g.rider_blocks, reinterpret_cast<float*>(lds_raw));
    return;
  }
  gemm_ring_body<T, BM, BN, WAVES_M, WAVES_N, A_KC, B_KC, EPI, RING, STEPBUF>(g, static_cast<int>(blockIdx.x) - g.rider_blocks);
}

}  // namespace nmtg
