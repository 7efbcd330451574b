// GEMM instantiations for A [M][K], B [N][K] (both reduction-contiguous): forward linears,
// Q K^T scores, dP = dC V^T.
#include "gemm_inst.hip.h"
namespace nmtg {
#define CASE(TILE, EPI) if (tile == TILE && epi == EPI) return gemm_launch_one<T, TILE, true, true, EPI>(a, st);
template <typename T> static int run(int tile, int epi, const GemmArgs& a, hipStream_t st) {
  CASE(TILE_L, EPI_PLAIN) CASE(TILE_M, EPI_PLAIN)
  CASE(TILE_L, EPI_ACT_FWD) CASE(TILE_M, EPI_ACT_FWD)
  CASE(TILE_L, EPI_SCORES) CASE(TILE_M, EPI_SCORES)
  // whole-row tile with the fused softmax epilogue: 16-byte accesses only, two-buffer loop (K is one or two steps)
  if (tile == TILE_R && epi == EPI_SCORES_SOFTMAX) return gemm_launch_vec<T, TILE_R, true, true, EPI_SCORES_SOFTMAX, 8>(a, st);
  if (tile == TILE_R && epi == EPI_SCORES_SOFTMAX_RNG) return gemm_launch_vec<T, TILE_R, true, true, EPI_SCORES_SOFTMAX_RNG, 8>(a, st);
  if (tile == TILE_R && epi == EPI_DSOFTMAX) return gemm_launch_vec<T, TILE_R, true, true, EPI_DSOFTMAX, 8>(a, st);
  return fail(NMTG_ERR_UNSUPPORTED, "gemm NT: no kernel for tile %d epilogue %d", tile, epi);
}
#undef CASE
int gemm_launch_nt(int dtype, int tile, int epi, const GemmArgs& a, hipStream_t st) {
  if (dtype == NMTG_F16) return run<f16_t>(tile, epi, a, st);
  if (dtype == NMTG_BF16) return run<bf16_t>(tile, epi, a, st);
  return fail(NMTG_ERR_UNSUPPORTED, "gemm: MFMA path takes fp16 or bf16, got dtype %d", dtype);
}
}  // namespace nmtg
