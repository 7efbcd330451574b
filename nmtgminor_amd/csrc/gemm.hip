// Host side of the MFMA GEMM core: tile / split selection, alignment analysis, the column-sum
// (bias gradient) helpers and the stand-alone C entry point nmtg_gemm.
#include "gemm_inst.hip.h"
#include <algorithm>
#include <cstdlib>
#include <mutex>

namespace nmtg {

bool gemm_has(int layout, int tile, int epi) {
  if (layout == LAYOUT_NT)
    return (tile == TILE_L || tile == TILE_M) && (epi == EPI_PLAIN || epi == EPI_ACT_FWD || epi == EPI_SCORES);
  if (layout == LAYOUT_NN) {
    if (epi == EPI_PLAIN) return true;
    return epi == EPI_ACT_BWD && (tile == TILE_L || tile == TILE_M);
  }
  if (layout == LAYOUT_TN) {
    if (epi == EPI_PLAIN) return true;
    return epi == EPI_SPLITK && (tile == TILE_L || tile == TILE_M);
  }
  return false;
}

namespace {

int vec_of(const void* p, int64_t ld, int64_t batch_stride, int batch) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  auto ok = [&](int v) {
    return a % (2 * v) == 0 && ld % v == 0 && (batch <= 1 || batch_stride % v == 0);
  };
  if (ok(8)) return 8;
  if (ok(4)) return 4;
  return 1;
}

int ceil_div(int a, int b) { return (a + b - 1) / b; }

struct SplitPlan {
  int tile, splits, k_per_split;
};

// Weight-gradient style products (small output, long reduction): spread the reduction over
// enough blocks to occupy the chip; partial tiles go through an fp32 workspace.
SplitPlan plan_splitk(int M, int N, int K, int batch) {
  const int cus = num_cus();
  SplitPlan p{TILE_M, 1, ceil_div(K, GEMM_BK) * GEMM_BK};
  const int tiles_l = ceil_div(M, 256) * ceil_div(N, 256) * batch;
  const int tiles_m = ceil_div(M, 128) * ceil_div(N, 128) * batch;
  // prefer the large tile when it alone offers >= 1/8 of the chip (then <= 8-way split)
  int tiles;
  if (tiles_l * 8 >= cus) { p.tile = TILE_L; tiles = tiles_l; }
  else { p.tile = TILE_M; tiles = tiles_m; }
  int splits = std::max(1, (cus + tiles / 2) / tiles);
  const int max_splits = std::max(1, K / (4 * GEMM_BK));  // at least 4 reduction steps per block
  splits = std::min(splits, max_splits);
  p.k_per_split = ceil_div(ceil_div(K, splits), GEMM_BK) * GEMM_BK;
  p.splits = ceil_div(K, p.k_per_split);
  return p;
}

size_t splitk_ws_bytes(const SplitPlan& p, int M, int N, int batch) {
  int bm, bn;
  tile_dims(p.tile, bm, bn);
  const size_t area = static_cast<size_t>(ceil_div(M, bm)) * bm * ceil_div(N, bn) * bn;
  return area * batch * p.splits * sizeof(float);
}

}  // namespace

size_t gemm_splitk_workspace_bytes(int M, int N, int K, int batch) {
  const SplitPlan p = plan_splitk(M, N, K, batch);
  return splitk_ws_bytes(p, M, N, batch);
}

int gemm_run(int dtype, int layout, int epi, GemmArgs a, void* workspace, size_t workspace_bytes, hipStream_t st,
             int* m_tiles_out, GemmArgs* planned_out) {
  if (m_tiles_out) *m_tiles_out = 0;
  if (a.M <= 0 || a.N <= 0 || a.batch <= 0) return 0;
  if (a.K < 0) return fail(NMTG_ERR_INVALID, "gemm: negative K");
  if (!a.A || !a.B || !a.C) return fail(NMTG_ERR_INVALID, "gemm: null operand pointer");
  if (dtype == NMTG_F32) return gemm_f32_run(layout, epi, a, st, m_tiles_out, planned_out);
  if (gemm_skinny_ok(dtype, layout, epi, a)) {
    a.splits = 1;
    a.defer_reduce = 0;
    a.tile_used = -1;
    a.riders_taken = 0;
    if (planned_out) *planned_out = a;
    return gemm_skinny_run(dtype, a, st);
  }
  const bool a_kc = layout != LAYOUT_TN;
  const bool b_kc = layout == LAYOUT_NT;
  // Widest access (8, 4 or 1 elements) that every pointer, pitch and batch stride of this call allows. Extents do not
  // enter: a ragged M / N / K ends in a predicated last vector (loads stay inside the row's pitch, which is a multiple
  // of the vector; the K tail is zeroed; the stores of a partial vector and the bias of a ragged last tile go element
  // by element). Byte masks are addressed as row * N + n, so there N is the pitch and does count.
  int vec = 8;
  auto narrow = [&](const void* p, int64_t ld, int64_t stride, int batch) {
    vec = std::min(vec, vec_of(p, ld, stride, batch));
  };
  narrow(a.A, a.lda, a.sA, a.batch);
  narrow(a.B, a.ldb, a.sB, a.batch);
  narrow(a.C, a.ldc, a.sC, a.batch);
  if (a.aux_out) narrow(a.aux_out, a.ldc, a.sC, a.batch);
  if (a.bias) narrow(a.bias, 8, 0, 1);
  if (a.aux_in) narrow(a.aux_in, a.ld_aux, 0, 1);
  auto narrow_bytes = [&](const uint8_t* p) {
    int v = 8;
    while (v > 1 && (reinterpret_cast<uintptr_t>(p) % v != 0 || a.N % v != 0)) v = v == 8 ? 4 : 1;
    vec = std::min(vec, v);
  };
  if (a.dmask) narrow_bytes(a.dmask);
  if (a.kmask && a.kmask_kind != 0) narrow_bytes(a.kmask);
  a.vec = vec;

  int tile = -1;
  a.splits = 1;
  a.k_per_split = ceil_div(std::max(a.K, 1), GEMM_BK) * GEMM_BK;

  if (layout == LAYOUT_TN && epi == EPI_PLAIN && workspace != nullptr) {
    const SplitPlan p = plan_splitk(a.M, a.N, a.K, a.batch);
    if (p.splits > 1 && (p.tile != TILE_L || vec == 8) && splitk_ws_bytes(p, a.M, a.N, a.batch) <= workspace_bytes &&
        (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0) {
      epi = EPI_SPLITK;
      tile = p.tile;
      a.splits = p.splits;
      a.k_per_split = p.k_per_split;
      a.ws = static_cast<float*>(workspace);
    }
  }
  // NMTG_GEMM_TILE=0|1|2 (256x256 | 128x128 | 256x64) overrides the tile choice: a tuning aid.
  const int forced_tile = [] { const char* e = getenv("NMTG_GEMM_TILE"); return e ? atoi(e) : -1; }();
  if (tile < 0 && forced_tile >= 0 && gemm_has(layout, forced_tile, epi) && (forced_tile != TILE_L || vec == 8)) tile = forced_tile;
  if (tile < 0) {
    const int cus = num_cus();
    const int64_t cnt_l = static_cast<int64_t>(ceil_div(a.M, 256)) * ceil_div(a.N, 256) * a.batch;
    const bool l_ok = vec == 8 && gemm_has(layout, TILE_L, epi);
    // share of a tile grid's area that is output: a 256-row tile on 128 rows (the scores of 128 decoder positions)
    // multiplies and stages twice what it stores. The 256x256 loop sustains about 1.6 times the MFMA rate of the
    // 128x128 one, so it keeps the call unless it wastes more than that.
    auto fill = [&](int bm, int bn) {
      return static_cast<double>(a.M) * a.N / (static_cast<double>(ceil_div(a.M, bm)) * bm * ceil_div(a.N, bn) * bn);
    };
    const bool l_fills = fill(256, 256) * 1.6 >= fill(128, 128) || !gemm_has(layout, TILE_M, epi);
    if (a.N <= 64 && gemm_has(layout, TILE_S, epi)) tile = TILE_S;
    else if (cnt_l * 4 >= cus * 3 && l_ok && l_fills) tile = TILE_L;
    else if (gemm_has(layout, TILE_M, epi)) tile = TILE_M;
    else if (l_ok) tile = TILE_L;
    else tile = TILE_S;
  }
  if (!gemm_has(layout, tile, epi))
    return fail(NMTG_ERR_UNSUPPORTED, "gemm: layout %d has no kernel for epilogue %d", layout, epi);
  // The slot-ring kernel (direct global -> LDS loads) needs whole 64-k steps (k_per_split is a multiple of 64 already),
  // 16-byte accesses, and 32-bit lane offsets inside one tile of an operand: 256 rows of a reduction-contiguous one, 64
  // k-rows plus a row of the other kind. Every other call takes the two-buffer loop.
  const int64_t a_span = a_kc ? 256 * a.lda * 2 : 64 * a.lda * 2 + static_cast<int64_t>(a.M) * 2;
  const int64_t b_span = b_kc ? 256 * a.ldb * 2 : 64 * a.ldb * 2 + static_cast<int64_t>(a.N) * 2;
  a.ring = (a.K > 0 && a.K % GEMM_BK == 0 && vec == 8 && a_span < (int64_t{1} << 32) && b_span < (int64_t{1} << 32)) ? 1 : 0;
  // gelu and gelu' of the activation epilogues come from a table in LDS in the ring kernels (they have the LDS room)
  a.act_lut = (a.ring && (epi == EPI_ACT_FWD || epi == EPI_ACT_BWD)) ? 1 : 0;
  int bm, bn;
  tile_dims(tile, bm, bn);
  a.m_tiles = ceil_div(a.M, bm);
  a.n_tiles = ceil_div(a.N, bn);
  if (m_tiles_out) *m_tiles_out = a.m_tiles;
  if (static_cast<int64_t>(a.m_tiles) * a.n_tiles > 0x7fffffff || a.batch > 65535)
    return fail(NMTG_ERR_UNSUPPORTED, "gemm: grid too large (tiles %d x %d, batch %d)", a.m_tiles, a.n_tiles, a.batch);
  if (epi == EPI_SPLITK && a.ws == nullptr)
    return fail(NMTG_ERR_INVALID, "gemm: the split-K epilogue needs a workspace");
  a.tile_used = tile;
  if (epi != EPI_SPLITK) a.defer_reduce = 0;
  // riders travel with the kernels that ring_rider<> (gemm_inst.hip.h) names, and only in an unbatched launch
  const bool can_ride = tile == TILE_M && a.vec == 8 && a.ring && a.batch == 1 && layout == LAYOUT_NN && epi == EPI_PLAIN;
  a.riders_taken = (a.riders != nullptr && a.rider_blocks > 0 && can_ride) ? 1 : 0;
  if (!a.riders_taken) { a.riders = nullptr; a.rider_blocks = 0; }
  if (planned_out) *planned_out = a;
  int rc;
  if (layout == LAYOUT_NT) rc = gemm_launch_nt(dtype, tile, epi, a, st);
  else if (layout == LAYOUT_NN) rc = gemm_launch_nn(dtype, tile, epi, a, st);
  else rc = gemm_launch_tn(dtype, tile, epi, a, st);
  if (rc) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "gemm: launch failed: %s", hipGetErrorString(e));
  return 0;
}

namespace {
// Shared eligibility test and launch of the whole-row tile (128 x 512, N <= 512): 16-byte accesses everywhere.
int row_tile_try(int dtype, int epi, GemmArgs a, const void* extra_like_c, hipStream_t st) {
  if (a.M <= 0 || a.N <= 0 || a.batch <= 0) return 0;
  if (dtype != NMTG_F16 && dtype != NMTG_BF16) return 0;
  if (a.N > 512 || a.N % 8 != 0 || a.K <= 0 || a.K % 8 != 0 || a.batch > 65535 || !extra_like_c) return 0;
  auto ok16 = [](const void* p, int64_t ld, int64_t stride, int batch) { return vec_of(p, ld, stride, batch) == 8; };
  if (!ok16(a.A, a.lda, a.sA, a.batch) || !ok16(a.B, a.ldb, a.sB, a.batch) || !ok16(a.C, a.ldc, a.sC, a.batch) ||
      !ok16(extra_like_c, a.ldc, a.sC, a.batch) || (a.aux_out && !ok16(a.aux_out, a.ldc, a.sC, a.batch)))
    return 0;
  auto ok8 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 8 == 0; };
  if ((a.dmask && !ok8(a.dmask)) || (a.kmask && a.kmask_kind != 0 && !ok8(a.kmask))) return 0;
  a.vec = 8;
  a.ring = 0;
  a.splits = 1;
  a.k_per_split = ceil_div(a.K, GEMM_BK) * GEMM_BK;
  a.m_tiles = ceil_div(a.M, 128);
  a.n_tiles = 1;
  if (int rc = gemm_launch_nt(dtype, TILE_R, epi, a, st)) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NMTG_ERR_LAUNCH, "gemm: launch failed: %s", hipGetErrorString(e));
  return 1;
}
}  // namespace

int gemm_scores_softmax_try(int dtype, GemmArgs a, hipStream_t st) {
  return row_tile_try(dtype, (a.dmask != nullptr && a.rng) ? EPI_SCORES_SOFTMAX_RNG : EPI_SCORES_SOFTMAX, a, a.out2, st);
}

int gemm_dsoftmax_try(int dtype, GemmArgs a, hipStream_t st) {
  a.bias = nullptr;
  a.aux_out = nullptr;
  a.kmask = nullptr;
  a.kmask_kind = 0;
  return row_tile_try(dtype, EPI_DSOFTMAX, a, a.aux_in, st);
}

}  // namespace nmtg

using namespace nmtg;

extern "C" int64_t nmtg_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k, int64_t batch) {
  if (m <= 0 || n <= 0 || k <= 0 || batch <= 0 || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return 0;
  return static_cast<int64_t>(gemm_splitk_workspace_bytes(static_cast<int>(m), static_cast<int>(n), static_cast<int>(k),
                                                          static_cast<int>(batch)));
}

extern "C" int nmtg_gemm(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a, int64_t lda,
                         int64_t stride_a, const void* b, int64_t ldb, int64_t stride_b, void* c, int64_t ldc,
                         int64_t stride_c, int64_t batch, const void* bias, void* workspace, int64_t workspace_bytes,
                         int dtype, void* stream) {
  NMTG_REQUIRE(m >= 0 && n >= 0 && k >= 0 && batch >= 0 && m <= INT32_MAX && n <= INT32_MAX && k <= INT32_MAX &&
                   batch <= 65535,
               "gemm: bad shape m=%lld n=%lld k=%lld batch=%lld", (long long)m, (long long)n, (long long)k, (long long)batch);
  int layout;
  if (!trans_a && trans_b) layout = LAYOUT_NT;
  else if (!trans_a && !trans_b) layout = LAYOUT_NN;
  else if (trans_a && !trans_b) layout = LAYOUT_TN;
  else return fail(NMTG_ERR_UNSUPPORTED, "gemm: A^T B^T is not provided (no caller on this path needs it)");
  GemmArgs g{};
  g.A = a; g.B = b; g.C = c;
  g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.sA = stride_a; g.sB = stride_b; g.sC = stride_c;
  g.M = static_cast<int>(m); g.N = static_cast<int>(n); g.K = static_cast<int>(k);
  g.batch = static_cast<int>(batch);
  g.alpha = alpha;
  g.bias = bias;
  // leading dimensions must cover the contiguous extent
  NMTG_REQUIRE(lda >= (trans_a ? m : k) && ldb >= (trans_b ? k : n) && ldc >= n, "gemm: leading dimension too small");
  return gemm_run(dtype, layout, EPI_PLAIN, g, workspace, static_cast<size_t>(std::max<int64_t>(0, workspace_bytes)),
                  static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------------------------
// nmtg_gemm for callers that cannot allocate: the split-K partials go to a fixed array in device
// memory that belongs to the library (one copy per GPU, held until the process ends).
// ---------------------------------------------------------------------------------------------
namespace {
constexpr size_t STATIC_SCRATCH_BYTES = size_t{32} << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

// `scratch` names a host-side handle, not a device address: the address on the current device is asked for once per
// device and kept.
constexpr int SCRATCH_MAX_DEV = 64;
void* scratch_ptr[SCRATCH_MAX_DEV] = {nullptr};
std::mutex scratch_mutex;

int scratch_on_current_device(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= SCRATCH_MAX_DEV)
    return nmtg::fail(NMTG_ERR_LAUNCH, "gemm_static: cannot identify the current device: %s", hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return nmtg::fail(NMTG_ERR_LAUNCH, "gemm_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return 0;
}
}  // namespace

extern "C" int64_t nmtg_gemm_static_max_workspace_bytes(void) { return static_cast<int64_t>(STATIC_SCRATCH_BYTES); }

extern "C" int nmtg_gemm_static(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a, int64_t lda,
                                int64_t stride_a, const void* b, int64_t ldb, int64_t stride_b, void* c, int64_t ldc,
                                int64_t stride_c, int64_t batch, const void* bias, int dtype, void* stream) {
  const int64_t need = nmtg_gemm_workspace_bytes(m, n, k, batch);
  NMTG_REQUIRE(need <= static_cast<int64_t>(STATIC_SCRATCH_BYTES),
               "gemm_static: this shape splits K over %lld bytes of partial sums, the built-in scratch holds %lld; use nmtg_gemm "
               "with a workspace", (long long)need, (long long)STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0) {
    if (int rc = scratch_on_current_device(&ws)) return rc;
  }
  // every split writes its whole partial tile before the reduction reads it: nothing has to be cleared between calls
  return nmtg_gemm(trans_a, trans_b, m, n, k, alpha, a, lda, stride_a, b, ldb, stride_b, c, ldc, stride_c, batch, bias, ws, need,
                   dtype, stream);
}
