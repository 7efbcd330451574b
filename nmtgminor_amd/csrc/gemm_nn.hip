// GEMM instantiations for A [M][K] reduction-contiguous, B [K][N] (row index contiguous):
// data gradients dX = dY W, P V, dQ = dS K.
#include "gemm_inst.hip.h"
namespace nmtg {
#define CASE(TILE, EPI) if (tile == TILE && epi == EPI) return gemm_launch_one<T, TILE, true, false, EPI>(a, st);
template <typename T> static int run(int tile, int epi, const GemmArgs& a, hipStream_t st) {
  CASE(TILE_L, EPI_PLAIN) CASE(TILE_M, EPI_PLAIN) CASE(TILE_S, EPI_PLAIN)
  CASE(TILE_L, EPI_ACT_BWD) CASE(TILE_M, EPI_ACT_BWD)
  return fail(NMTG_ERR_UNSUPPORTED, "gemm NN: no kernel for tile %d epilogue %d", tile, epi);
}
#undef CASE
int gemm_launch_nn(int dtype, int tile, int epi, const GemmArgs& a, hipStream_t st) {
  if (dtype == NMTG_F16) return run<f16_t>(tile, epi, a, st);
  if (dtype == NMTG_BF16) return run<bf16_t>(tile, epi, a, st);
  return fail(NMTG_ERR_UNSUPPORTED, "gemm: MFMA path takes fp16 or bf16, got dtype %d", dtype);
}
}  // namespace nmtg
