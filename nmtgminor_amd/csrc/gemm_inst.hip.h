// Per-layout instantiation units of the GEMM kernel (one translation unit per operand layout so
// they compile in parallel). Tile configurations:
//   L: 256x256 tile, 2x4 wavefronts (each 128x64), 512 threads  — large outputs
//   M: 128x128 tile, 2x2 wavefronts (each 64x64),  256 threads  — outputs too small to fill the chip with L
//   S: 256x64  tile, 4x1 wavefronts (each 64x64),  256 threads  — N <= 64 (per-head attention products)
//   R: 128x512 tile, 4x2 wavefronts (each 32x256), 512 threads  — whole score rows (fused softmax epilogue only)
#pragma once
#include "gemm.hip.h"
#include "gemm_ring.hip.h"
#include <string>

namespace nmtg {

// GemmTile and tile_cfg<TILE> (block tile and wavefront grid of each tile) live in reduce.hip.h: the reduction kernels need them too.

inline void tile_dims(int tile, int& bm, int& bn) {
  if (tile == TILE_L) { bm = 256; bn = 256; }
  else if (tile == TILE_M) { bm = 128; bn = 128; }
  else if (tile == TILE_R) { bm = 128; bn = 512; }
  else { bm = 256; bn = 64; }
}

template <typename T, int TILE, bool A_KC, bool B_KC, int EPI, int VEC>
int gemm_launch_vec(const GemmArgs& a, hipStream_t st) {
  using C = tile_cfg<TILE>;
  auto kern = gemm_kernel<T, C::BM, C::BN, C::WM, C::WN, A_KC, B_KC, EPI, VEC>;
  constexpr int lds = gemm_lds_bytes<C::BM, C::BN>();
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "gemm: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));
    attr_done = true;
  }
  dim3 grid(a.m_tiles * a.n_tiles, a.batch, a.splits);
  static const std::string name = std::string("gemm_") + (A_KC ? (B_KC ? "nt" : "nn") : "tn") + "_" +
                                  (TILE == TILE_L ? "256x256" : TILE == TILE_M ? "128x128" : TILE == TILE_R ? "128x512" : "256x64") + "_" +
                                  (EPI == EPI_PLAIN ? "plain" : EPI == EPI_ACT_FWD ? "actfwd" : EPI == EPI_ACT_BWD ? "actbwd"
                                   : EPI == EPI_SCORES ? "scores" : (EPI == EPI_SCORES_SOFTMAX || EPI == EPI_SCORES_SOFTMAX_RNG) ? "scores_softmax" : EPI == EPI_DSOFTMAX ? "dsoftmax"
                                   : "splitk") +
                                  (VEC == 8 ? "" : VEC == 4 ? "_v4" : "_v1");
  TraceScope trace(name.c_str(), st);
  hipLaunchKernelGGL(kern, grid, dim3(64 * C::WM * C::WN), lds, st, a);
  return 0;
}


// Slot-ring kernel (gemm_ring.hip.h): the 256x256 tile owns the whole LDS (10 slots), the 128x128
// tile takes 5 slots so that two blocks share a CU and one block's epilogue overlaps the other's
// main loop.
template <int TILE> struct ring_slots { static constexpr int value = TILE == TILE_M ? 5 : 10; };
// The 128x128 tile runs one wavefront per SIMD: its main loop keeps a whole stage's fragments in registers (STEPBUF).
template <int TILE> struct ring_stepbuf { static constexpr bool value = TILE == TILE_M; };

// Which kernels carry riders (GemmArgs::riders): the plain 128x128 data-gradient product, the last kernel of a backward
// pass, which leaves one block on a CU at the shapes of a feed-forward block.
template <int TILE, bool A_KC, bool B_KC, int EPI> struct ring_rider {
  static constexpr bool value = TILE == TILE_M && A_KC && !B_KC && EPI == EPI_PLAIN;
};

template <typename T, int TILE, bool A_KC, bool B_KC, int EPI>
int gemm_launch_ring(const GemmArgs& a, hipStream_t st) {
  using C = tile_cfg<TILE>;
  constexpr int RING = ring_slots<TILE>::value;
  constexpr bool RIDER = ring_rider<TILE, A_KC, B_KC, EPI>::value;
  auto kern = [] {
    if constexpr (RIDER) return gemm_ring_rider_kernel<T, C::BM, C::BN, C::WM, C::WN, A_KC, B_KC, EPI, RING, ring_stepbuf<TILE>::value>;
    else return gemm_ring_kernel<T, C::BM, C::BN, C::WM, C::WN, A_KC, B_KC, EPI, RING, ring_stepbuf<TILE>::value>;
  }();
  constexpr int lds = gemm_ring_lds_bytes<C::BM, C::BN, RING>();
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "gemm: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));
    attr_done = true;
  }
  dim3 grid(a.m_tiles * a.n_tiles, a.batch, a.splits);
  static const std::string name = std::string("gemm_") + (A_KC ? (B_KC ? "nt" : "nn") : "tn") + "_" +
                                  (TILE == TILE_L ? "256x256" : TILE == TILE_M ? "128x128" : "256x64") + "_" +
                                  (EPI == EPI_PLAIN ? "plain" : EPI == EPI_ACT_FWD ? "actfwd" : EPI == EPI_ACT_BWD ? "actbwd"
                                   : EPI == EPI_SCORES ? "scores" : "splitk") + "_ring";
  TraceScope trace(name.c_str(), st);
  if constexpr (RIDER) {
    const bool ride = a.riders != nullptr && a.rider_blocks > 0;
    TailArgs riders{};
    if (ride) {
      riders = *static_cast<const TailArgs*>(a.riders);
      grid.x += static_cast<unsigned>(a.rider_blocks);
    }
    hipLaunchKernelGGL(kern, grid, dim3(64 * C::WM * C::WN), lds, st, a, riders);
  } else {
    hipLaunchKernelGGL(kern, grid, dim3(64 * C::WM * C::WN), lds, st, a);
  }
  return 0;
}

// The 256x256 tile exists for 16-byte accesses only; narrower calls are routed to the smaller tiles.
template <typename T, int TILE, bool A_KC, bool B_KC, int EPI>
int gemm_launch_one(const GemmArgs& a, hipStream_t st) {
  if (a.vec == 8 && a.ring) return gemm_launch_ring<T, TILE, A_KC, B_KC, EPI>(a, st);
  if (a.vec == 8) return gemm_launch_vec<T, TILE, A_KC, B_KC, EPI, 8>(a, st);
  if constexpr (TILE != TILE_L) {
    if (a.vec == 4) return gemm_launch_vec<T, TILE, A_KC, B_KC, EPI, 4>(a, st);
    return gemm_launch_vec<T, TILE, A_KC, B_KC, EPI, 1>(a, st);
  } else {
    return fail(NMTG_ERR_UNSUPPORTED, "gemm: the 256x256 tile needs 16-byte aligned operands");
  }
}

template <typename T, int TILE>
int splitk_reduce_launch(const GemmArgs& a, hipStream_t st) {
  using C = tile_cfg<TILE>;
  constexpr int per_blk = C::WM * C::WN * (C::BM / C::WM / 32) * (C::BN / C::WN / 32) * 4 * 64;
  const int64_t total = static_cast<int64_t>(a.batch) * a.m_tiles * a.n_tiles * per_blk;
  TraceScope trace("splitk_reduce", st);
  hipLaunchKernelGGL((splitk_reduce_kernel<T, C::BM, C::BN, C::WM, C::WN>), dim3(static_cast<unsigned>((total + 255) / 256)),
                     dim3(256), 0, st, a.ws, static_cast<T*>(a.C), a.ldc, a.M, a.N, a.m_tiles, a.n_tiles, a.batch, a.sC,
                     a.splits, a.alpha, a.vec);
  return 0;
}

// Defined in gemm_nt.hip / gemm_nn.hip / gemm_tn.hip. Return NMTG_ERR_UNSUPPORTED for a
// (tile, epilogue) pair that is not instantiated.
int gemm_launch_nt(int dtype, int tile, int epi, const GemmArgs& a, hipStream_t st);
int gemm_launch_nn(int dtype, int tile, int epi, const GemmArgs& a, hipStream_t st);
int gemm_launch_tn(int dtype, int tile, int epi, const GemmArgs& a, hipStream_t st);
bool gemm_has(int layout, int tile, int epi);

}  // namespace nmtg
