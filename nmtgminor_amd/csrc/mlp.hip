// Fused multi-layer perceptron, forward and backward, on the MFMA GEMM core.
//
// Stands in for fused_mlp_{relu,gelu,silu,agelu}.forward / backward / backward_input_only and
// mlp_gelu_blaslt.* of the reference (onmt/modules/extensions/mlp/mlp_gelu.cpp:69-264,
// mlp_gelu_cuda.cu:1362-1826; mlp_relu.cpp:68-272; mlp_blaslt/mlp_gelu.cpp:75-242).
//
// Launch plan for n layers (n = 2 in the transformer feed-forward block):
//   forward : n GEMMs. Hidden layers run the bias + activation + dropout epilogue and write the
//             pre-activation and the dropped activation straight from the accumulators; the
//             last layer adds its bias.
//   backward: per layer one weight-gradient GEMM (token dimension split over the chip, fp32
//             partials) and one data-gradient GEMM whose epilogue applies act'(h) * mask / (1-p)
//             and produces the bias-gradient column sums; one column-sum kernel for the last
//             layer's bias.
// The reference runs a GEMM and then separate element-wise kernels over the [tokens, inner]
// tensors; here those tensors cross HBM once per direction.
#include "gemm.hip.h"
#include <algorithm>
#include <cstdlib>
#include <vector>

namespace nmtg {
namespace {

constexpr int MAX_LAYERS = 16;

size_t align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

struct BwdPlan {
  size_t dh_bytes;       // one dh buffer [batch, max hidden] (two are used, ping-pong)
  size_t colsum_bytes;   // fp32 partials for one layer's bias gradient
  size_t splitk_bytes;   // largest weight-gradient split-K workspace
  int layers;
  // one column-sum and one split-K region per layer: with the reductions deferred to one launch at the end
  // every layer's partials stay alive until then
  size_t total() const { return 2 * dh_bytes + layers * (colsum_bytes + splitk_bytes); }
};

BwdPlan plan_bwd(int num_layers, const int64_t* out_features, int64_t batch, int64_t in_features, size_t esz) {
  BwdPlan p{0, 0, 0, num_layers};
  int64_t max_hidden = 0, max_out = 0;
  for (int i = 0; i < num_layers; ++i) {
    if (i < num_layers - 1) max_hidden = std::max(max_hidden, out_features[i]);
    max_out = std::max(max_out, out_features[i]);
    const int64_t in_i = i == 0 ? in_features : out_features[i - 1];
    p.splitk_bytes = std::max(p.splitk_bytes, gemm_splitk_workspace_bytes(static_cast<int>(out_features[i]),
                                                                          static_cast<int>(in_i),
                                                                          static_cast<int>(batch), 1));
  }
  p.dh_bytes = align_up(static_cast<size_t>(batch) * max_hidden * esz);
  const size_t parts = static_cast<size_t>(std::max<int64_t>(colsum_parts(static_cast<int>(batch)), (batch + 127) / 128));
  p.colsum_bytes = align_up(parts * max_out * sizeof(float));
  p.splitk_bytes = align_up(p.splitk_bytes);
  return p;
}

int check_shapes(const char* who, int num_layers, const int64_t* out_features, int64_t batch, int64_t in_features,
                 int dtype, int act) {
  NMTG_REQUIRE(num_layers >= 1 && num_layers <= MAX_LAYERS, "%s: number of layers %d outside [1, %d]", who, num_layers,
               MAX_LAYERS);
  NMTG_REQUIRE(out_features != nullptr, "%s: out_features is null", who);
  NMTG_REQUIRE(batch >= 0 && batch <= INT32_MAX && in_features > 0 && in_features <= INT32_MAX, "%s: bad input shape", who);
  for (int i = 0; i < num_layers; ++i)
    NMTG_REQUIRE(out_features[i] > 0 && out_features[i] <= INT32_MAX, "%s: bad out_features[%d]", who, i);
  NMTG_REQUIRE(dtype == NMTG_F16 || dtype == NMTG_BF16 || dtype == NMTG_F32, "%s: dtype %d not supported (fp32, fp16 and bf16 are)", who, dtype);
  NMTG_REQUIRE(act >= NMTG_ACT_NONE && act <= NMTG_ACT_AGELU, "%s: unknown activation %d", who, act);
  return 0;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_mlp_fwd(int num_layers, const void* x, const void* const* weights, const void* const* biases,
                            const int64_t* out_features, int64_t batch, int64_t in_features, void* out,
                            void* post_acts, void* pre_acts, uint8_t* mask, int mask_mode, float p, uint64_t seed,
                            uint64_t offset, int act, int dtype, void* stream) {
  if (int rc = check_shapes("mlp_fwd", num_layers, out_features, batch, in_features, dtype, act)) return rc;
  NMTG_REQUIRE(weights != nullptr, "mlp_fwd: weights is null");
  NMTG_REQUIRE(mask_mode >= 0 && mask_mode <= 2, "mlp_fwd: bad mask_mode %d", mask_mode);
  NMTG_REQUIRE(mask_mode == 0 || (p >= 0.f && p < 1.f), "mlp_fwd: dropout probability %f outside [0, 1)", p);
  NMTG_REQUIRE(mask_mode == 0 || mask != nullptr || num_layers == 1, "mlp_fwd: mask buffer required when dropout is applied");
  NMTG_REQUIRE(num_layers == 1 || post_acts != nullptr, "mlp_fwd: post-activation buffer required");
  if (batch == 0) return 0;
  NMTG_REQUIRE(x && out, "mlp_fwd: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const void* in = x;
  int64_t in_f = in_features;
  const int64_t esz = dtype == NMTG_F32 ? 4 : 2;
  int64_t elt_off = 0;  // element offset into the concatenated hidden buffers
  for (int i = 0; i < num_layers; ++i) {
    NMTG_REQUIRE(weights[i] != nullptr, "mlp_fwd: weights[%d] is null", i);
    const bool last = i == num_layers - 1;
    GemmArgs g{};
    g.A = in; g.lda = in_f;
    g.B = weights[i]; g.ldb = in_f;
    g.M = static_cast<int>(batch); g.N = static_cast<int>(out_features[i]); g.K = static_cast<int>(in_f);
    g.batch = 1; g.alpha = 1.f;
    g.bias = biases ? biases[i] : nullptr;
    g.ldc = out_features[i];
    int rc;
    if (last) {
      g.C = out;
      rc = gemm_run(dtype, LAYOUT_NT, EPI_PLAIN, g, nullptr, 0, st);
    } else {
      g.C = static_cast<uint8_t*>(post_acts) + elt_off * esz;
      g.aux_out = pre_acts ? static_cast<uint8_t*>(pre_acts) + elt_off * esz : nullptr;
      g.act = act;
      if (mask_mode != 0) {
        g.dmask = mask + elt_off;
        g.dscale = 1.f / (1.f - p);
        g.keep_p = 1.f - p;
        g.rng = mask_mode == 2;
        g.seed = seed;
        g.offset = offset + static_cast<uint64_t>(elt_off);  // distinct counter range per layer
      }
      rc = gemm_run(dtype, LAYOUT_NT, EPI_ACT_FWD, g, nullptr, 0, st);
      in = g.C;
      in_f = out_features[i];
      elt_off += batch * out_features[i];
    }
    if (rc) return rc;
  }
  return 0;
}

extern "C" int64_t nmtg_mlp_bwd_workspace_bytes(int num_layers, const int64_t* out_features, int64_t batch,
                                                int64_t in_features) {
  if (num_layers < 1 || num_layers > MAX_LAYERS || !out_features || batch <= 0 || in_features <= 0) return 0;
  return static_cast<int64_t>(plan_bwd(num_layers, out_features, batch, in_features, 2).total());
}

extern "C" int64_t nmtg_mlp_bwd_dtype_workspace_bytes(int num_layers, const int64_t* out_features, int64_t batch,
                                                      int64_t in_features, int dtype) {
  if (num_layers < 1 || num_layers > MAX_LAYERS || !out_features || batch <= 0 || in_features <= 0) return 0;
  return static_cast<int64_t>(plan_bwd(num_layers, out_features, batch, in_features, dtype == NMTG_F32 ? 4 : 2).total());
}

extern "C" int nmtg_mlp_bwd(int num_layers, const void* x, const void* const* weights, const int64_t* out_features,
                            int64_t batch, int64_t in_features, const void* grad_out, const void* post_acts,
                            const void* pre_acts, const uint8_t* mask, float p, int act, void* grad_x,
                            void* const* grad_weights, void* const* grad_biases, void* workspace,
                            int64_t workspace_bytes, int dtype, void* stream) {
  if (int rc = check_shapes("mlp_bwd", num_layers, out_features, batch, in_features, dtype, act)) return rc;
  NMTG_REQUIRE(weights != nullptr, "mlp_bwd: weights is null");
  NMTG_REQUIRE(mask == nullptr || (p >= 0.f && p < 1.f), "mlp_bwd: dropout probability %f outside [0, 1)", p);
  NMTG_REQUIRE(num_layers == 1 || post_acts != nullptr, "mlp_bwd: post-activation buffer required");
  NMTG_REQUIRE(num_layers == 1 || pre_acts != nullptr || act == NMTG_ACT_RELU || act == NMTG_ACT_NONE,
               "mlp_bwd: pre-activation buffer required for this activation");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t esz = dtype == NMTG_F32 ? 4 : 2;
  const BwdPlan plan = plan_bwd(num_layers, out_features, std::max<int64_t>(batch, 1), in_features, static_cast<size_t>(esz));
  NMTG_REQUIRE(workspace != nullptr && static_cast<size_t>(std::max<int64_t>(workspace_bytes, 0)) >= plan.total() &&
                   (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
               "mlp_bwd: workspace of %zu bytes (256-byte aligned) required, got %lld", plan.total(),
               (long long)workspace_bytes);
  NMTG_REQUIRE(batch == 0 || (x && grad_out), "mlp_bwd: null pointer argument");
  uint8_t* wsb = static_cast<uint8_t*>(workspace);
  void* dh[2] = {wsb, wsb + plan.dh_bytes};
  // The split-K reductions and the final bias-gradient sums of all layers are collected as jobs of one reduction
  // (ReduceTail, up to its capacity; layers beyond that get launches of their own, with bit-identical results).
  ReduceTail tail;
  auto colsum_region = [&](int layer) {
    return reinterpret_cast<float*>(wsb + 2 * plan.dh_bytes + layer * plan.colsum_bytes);
  };
  auto splitk_region = [&](int layer) {
    return static_cast<void*>(wsb + 2 * plan.dh_bytes + plan.layers * plan.colsum_bytes + layer * plan.splitk_bytes);
  };

  // element offsets of each hidden layer inside the concatenated buffers
  int64_t offs[MAX_LAYERS] = {0};
  for (int i = 1; i < num_layers; ++i) offs[i] = offs[i - 1] + batch * out_features[i - 1];

  const void* g_cur = grad_out;      // gradient wrt layer i's linear output
  bool bias_from_parts = false;      // colsum_ws holds the partial column sums of g_cur
  int parts_rows = 0;
  // The final reductions (split-K sums, bias-gradient sums) ride along with the last data-gradient product, which
  // leaves room on the CUs (GemmArgs::riders); where there is no such product they are one launch at the end. The
  // partial column sums of the output gradient, which those read, are a launch of their own ahead of the GEMMs.
  const int max_riders = num_cus();   // one rider per CU, whatever the number of jobs' blocks
  ReduceTail head;                   // partial column sums of grad_out, owed before the tail's final sums
  bool head_pending = false;
  auto flush_head = [&]() -> int {
    if (!head_pending) return 0;
    head_pending = false;
    return tail_launch(head, dtype, st);
  };
  for (int i = num_layers - 1; i >= 0; --i) {
    const int64_t out_i = out_features[i];
    const int64_t in_i = i == 0 ? in_features : out_features[i - 1];
    const void* input_i = i == 0 ? x : static_cast<const uint8_t*>(post_acts) + offs[i - 1] * esz;
    int rc;
    // bias gradient (its partial rows: written by the data-gradient GEMM of the layer above, or by a kernel of its own)
    float* colsum_ws = colsum_region(i);
    if (grad_biases && grad_biases[i]) {
      if (!tail.full()) {
        int parts = parts_rows;
        rc = 0;
        if (!bias_from_parts) {
          parts = colsum_parts(static_cast<int>(batch));
          rc = tail_add_colsum_partial(head, dtype, g_cur, out_i, static_cast<int>(batch), static_cast<int>(out_i), colsum_ws);
          head_pending = !rc;
        }
        if (!rc) rc = tail_add_colsum(tail, colsum_ws, parts, static_cast<int>(out_i), grad_biases[i]);
      } else if (bias_from_parts) {
        rc = colsum_finish(dtype, colsum_ws, parts_rows, static_cast<int>(out_i), grad_biases[i], st);
      } else {
        rc = colsum_run(dtype, g_cur, out_i, static_cast<int>(batch), static_cast<int>(out_i), colsum_ws, grad_biases[i], st);
      }
      if (rc) return rc;
    }
    // weight gradient: dW_i [out_i, in_i] = g^T input
    if (grad_weights && grad_weights[i]) {
      GemmArgs g{};
      g.A = g_cur; g.lda = out_i;
      g.B = input_i; g.ldb = in_i;
      g.C = grad_weights[i]; g.ldc = in_i;
      g.M = static_cast<int>(out_i); g.N = static_cast<int>(in_i); g.K = static_cast<int>(batch);
      g.batch = 1; g.alpha = 1.f;
      g.defer_reduce = !tail.full() ? 1 : 0;
      // (the partial column sums do not ride with this product: a split-K launch repeats the rider blocks in every
      // split, and the tiles then share CUs unevenly; measured slower than the launch of their own)
      if (int rc2 = flush_head()) return rc2;
      GemmArgs planned{};
      rc = gemm_run(dtype, LAYOUT_TN, EPI_PLAIN, g, splitk_region(i), plan.splitk_bytes, st, nullptr, &planned);
      if (!rc && planned.defer_reduce && planned.splits > 1)
        rc = tail_add_splitk(tail, planned.tile_used, planned.ws, planned.C, planned.ldc, planned.M, planned.N, planned.m_tiles,
                             planned.n_tiles, planned.batch, planned.sC, planned.splits, planned.alpha, planned.vec);
      if (rc) return rc;
    }
    // data gradient
    if (i > 0) {
      GemmArgs g{};
      g.A = g_cur; g.lda = out_i;
      g.B = weights[i]; g.ldb = in_i;
      g.C = dh[i & 1]; g.ldc = in_i;
      g.M = static_cast<int>(batch); g.N = static_cast<int>(in_i); g.K = static_cast<int>(out_i);
      g.batch = 1; g.alpha = 1.f;
      g.act = act;
      const bool have_pre = pre_acts != nullptr;
      g.aux_in = have_pre ? static_cast<const uint8_t*>(pre_acts) + offs[i - 1] * esz
                          : static_cast<const uint8_t*>(post_acts) + offs[i - 1] * esz;
      g.ld_aux = in_i;
      g.dscale = 1.f;
      if (have_pre) {
        if (mask != nullptr && p > 0.f) { g.dmask = mask + offs[i - 1]; g.dscale = 1.f / (1.f - p); }
      } else if (p > 0.f) {
        g.dscale = 1.f / (1.f - p);  // relu from the dropped output: a > 0 iff kept and h > 0
      }
      // one partial row per row tile of the GEMM
      g.colsum_part = (grad_biases && grad_biases[i - 1]) ? colsum_region(i - 1) : nullptr;
      rc = gemm_run(dtype, LAYOUT_NN, EPI_ACT_BWD, g, nullptr, 0, st, &parts_rows);
      if (rc) return rc;
      bias_from_parts = g.colsum_part != nullptr;
      g_cur = dh[i & 1];
    } else if (grad_x != nullptr) {
      if (int rc2 = flush_head()) return rc2;     // the tail's final sums read what the head writes
      GemmArgs g{};
      g.A = g_cur; g.lda = out_i;
      g.B = weights[0]; g.ldb = in_i;
      g.C = grad_x; g.ldc = in_i;
      g.M = static_cast<int>(batch); g.N = static_cast<int>(in_i); g.K = static_cast<int>(out_i);
      g.batch = 1; g.alpha = 1.f;
      if (!tail.empty()) { g.riders = &tail.args; g.rider_blocks = max_riders; }
      GemmArgs planned{};
      rc = gemm_run(dtype, LAYOUT_NN, EPI_PLAIN, g, nullptr, 0, st, nullptr, &planned);
      if (rc) return rc;
      if (planned.riders_taken) return 0;        // every reduction has run beside this product
    }
  }
  if (int rc = flush_head()) return rc;
  return tail_launch(tail, dtype, st);
}
