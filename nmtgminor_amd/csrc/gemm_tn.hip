// GEMM instantiations for A [K][M], B [K][N] (both row-index contiguous): weight gradients
// dW = dY^T X (split over the token dimension), dV = P^T dC, dK = dS^T Q.
#include "gemm_inst.hip.h"
namespace nmtg {
#define CASE(TILE, EPI) if (tile == TILE && epi == EPI) return gemm_launch_one<T, TILE, false, false, EPI>(a, st);
template <typename T> static int run(int tile, int epi, const GemmArgs& a, hipStream_t st) {
  CASE(TILE_L, EPI_PLAIN) CASE(TILE_M, EPI_PLAIN) CASE(TILE_S, EPI_PLAIN)
  if (epi == EPI_SPLITK) {
    int rc = NMTG_ERR_UNSUPPORTED;
    if (tile == TILE_L) { rc = gemm_launch_one<T, TILE_L, false, false, EPI_SPLITK>(a, st); if (!rc && !a.defer_reduce) rc = splitk_reduce_launch<T, TILE_L>(a, st); return rc; }
    if (tile == TILE_M) { rc = gemm_launch_one<T, TILE_M, false, false, EPI_SPLITK>(a, st); if (!rc && !a.defer_reduce) rc = splitk_reduce_launch<T, TILE_M>(a, st); return rc; }
  }
  return fail(NMTG_ERR_UNSUPPORTED, "gemm TN: no kernel for tile %d epilogue %d", tile, epi);
}
#undef CASE
int gemm_launch_tn(int dtype, int tile, int epi, const GemmArgs& a, hipStream_t st) {
  if (dtype == NMTG_F16) return run<f16_t>(tile, epi, a, st);
  if (dtype == NMTG_BF16) return run<bf16_t>(tile, epi, a, st);
  return fail(NMTG_ERR_UNSUPPORTED, "gemm: MFMA path takes fp16 or bf16, got dtype %d", dtype);
}
}  // namespace nmtg
