// Pieces of the library that the CPU build does not take from the kernel sources (per-kernel tracing counts launches
// by name and reports zero time), and C hooks for the reduction kernels, which the real library only reaches from
// inside its GEMM-based operators.
#include "reduce.hip.h"
#include "gemm.hip.h"
#include <algorithm>
#include <cstring>
#include <map>
#include <string>

namespace {
bool g_trace = false;
std::map<std::string, int> g_launches;
}  // namespace

namespace nmtg {
bool trace_on() { return g_trace; }
void trace_open(const char* name, hipStream_t, int* slot) {
  ++g_launches[name];
  *slot = -1;
}
void trace_close(hipStream_t, int) {}
}  // namespace nmtg

extern "C" int nmtg_trace_begin(void) {
  g_launches.clear();
  g_trace = true;
  return 0;
}

// same text format as the library's: "name launches total_ms\n" per kernel name; returns the bytes needed
extern "C" int64_t nmtg_trace_end(char* out, int64_t capacity) {
  g_trace = false;
  std::string text;
  for (const auto& kv : g_launches) text += kv.first + " " + std::to_string(kv.second) + " 0.0\n";
  if (out != nullptr && capacity > 0) {
    const size_t n = std::min(text.size(), static_cast<size_t>(capacity - 1));
    memcpy(out, text.data(), n);
    out[n] = 0;
  }
  return static_cast<int64_t>(text.size()) + 1;
}

using namespace nmtg;

extern "C" int hostsim_colsum_parts(int M) { return colsum_parts(M); }

extern "C" int hostsim_colsum(int dtype, const void* X, int64_t ld, int M, int N, float* part, void* out) {
  return colsum_run(dtype, X, ld, M, N, part, out, nullptr);
}

// Split-K reduction for the 128x128 tile (2 x 2 wavefronts) and the 256x256 tile (2 x 4), launched as gemm_inst.hip.h does.
template <typename T, int BM, int BN, int WM, int WN>
static int splitk(const float* ws, void* C, int64_t ldc, int M, int N, int m_tiles, int n_tiles, int batch, int64_t sC,
                  int splits, float alpha, int c_vec) {
  constexpr int per_blk = WM * WN * (BM / WM / 32) * (BN / WN / 32) * 4 * 64;
  const int64_t total = static_cast<int64_t>(batch) * m_tiles * n_tiles * per_blk;
  hipLaunchKernelGGL((splitk_reduce_kernel<T, BM, BN, WM, WN>), dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                     nullptr, ws, static_cast<T*>(C), ldc, M, N, m_tiles, n_tiles, batch, sC, splits, alpha, c_vec);
  return 0;
}

extern "C" int hostsim_splitk_reduce(int dtype, int tile, const float* ws, void* C, int64_t ldc, int M, int N, int m_tiles,
                                     int n_tiles, int batch, int64_t sC, int splits, float alpha, int c_vec) {
  if (tile == 1) {
    NMTG_DISPATCH_DTYPE(dtype, T, return (splitk<T, 128, 128, 2, 2>(ws, C, ldc, M, N, m_tiles, n_tiles, batch, sC, splits, alpha, c_vec)));
  }
  NMTG_DISPATCH_DTYPE(dtype, T, return (splitk<T, 256, 256, 2, 4>(ws, C, ldc, M, N, m_tiles, n_tiles, batch, sC, splits, alpha, c_vec)));
  return -1;
}

// gemm_run asked for the split-K epilogue directly (only internal callers can) without the fp32 workspace its partial
// tiles go to: the call must be refused before any launch. -> gemm_run's status
extern "C" int hostsim_gemm_splitk_without_workspace(int dtype, const void* a, const void* b, void* c, int m, int n, int k) {
  GemmArgs g{};
  g.A = a; g.B = b; g.C = c;
  g.lda = m; g.ldb = n; g.ldc = n;
  g.M = m; g.N = n; g.K = k;
  g.batch = 1; g.alpha = 1.f;
  return gemm_run(dtype, LAYOUT_TN, EPI_SPLITK, g, nullptr, 0, nullptr);
}
