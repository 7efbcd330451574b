// Multi-head attention (self and encoder-decoder), forward and backward, on the MFMA GEMM core
// and the row-softmax kernels.
//
// Stands in for self_multihead_attn_blaslt.{forward, backward, forward_compact, backward_compact}
// (onmt/modules/extensions/multihead_attn_blaslt/self_multihead_attn_cuda.cu:40-243 forward,
// :413-742 backward, :247-407 / :745-960 compact) and encdec_multihead_attn_bias_blaslt.*
// (encdec_multihead_attn_bias_cuda.cu:40-273 forward, :1089-1472 backward).
//
// Layouts are the reference's: activations are time-first [T, B, E]; the self-attention input
// projection yields [T, B*H, 3, D] (q, k, v interleaved per head), the encoder-decoder key/value
// projection [Tk, B*H, 2, D]; scores and probabilities are [B*H, Tq, Tk]. The per-head products
// read q / k / v through strided views of those buffers (no copies), and the context is written
// straight back in [Tq, B*H, D] = [Tq, B, E].
//
// Differences in structure from the reference's launch list (6 forward / 10 backward launches):
// the key-padding / time mask is applied in the epilogue of the Q K^T product (no separate
// masked_fill pass over the [B*H, Tq, Tk] tensor); bias gradients are column-sum kernels with a
// fixed reduction order; weight gradients split the token dimension over the chip.
#include "gemm.hip.h"
#include <cstdlib>
#include <algorithm>

// implemented in softmax_dropout.hip
extern "C" int nmtg_softmax_dropout_fwd(const void*, const uint8_t*, int, void*, void*, uint8_t*, int, float, uint64_t,
                                        uint64_t, int64_t, int64_t, int64_t, int64_t, int, void*);
extern "C" int nmtg_softmax_dropout_bwd(const void*, const void*, int, const uint8_t*, int, const uint8_t*, int, float,
                                        void*, int64_t, int64_t, int64_t, int64_t, int, void*);

namespace nmtg {
namespace {

size_t align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

// One (batch*head)-strided operand: element pointer of head 0, row pitch, per-head stride.
struct Strided {
  const void* p;
  int64_t ld, stride;
};
inline const void* offset16(const void* p, int64_t elems) { return static_cast<const uint8_t*>(p) + elems * 2; }
inline void* offset16(void* p, int64_t elems) { return static_cast<uint8_t*>(p) + elems * 2; }

struct Core {
  int tq, tk, d, bh, heads;
  float scale;
  int dtype;
  hipStream_t st;
};

// scores = scale * q k^T (+ mask -> -inf);  probabilities / dropout;  ctx = P v.
int core_fwd(const Core& c, Strided q, Strided k, Strided v, const uint8_t* mask, int mask_kind, void* scores,
             void* softmax_out, void* dropped, uint8_t* dmask, int dropout_mode, float p, uint64_t seed, uint64_t offset,
             void* ctx, int64_t ld_ctx, int64_t stride_ctx) {
  GemmArgs g{};
  g.A = q.p; g.lda = q.ld; g.sA = q.stride;
  g.B = k.p; g.ldb = k.ld; g.sB = k.stride;
  g.C = scores; g.ldc = c.tk; g.sC = static_cast<int64_t>(c.tq) * c.tk;
  g.M = c.tq; g.N = c.tk; g.K = c.d; g.batch = c.bh; g.alpha = c.scale;
  g.kmask = mask; g.kmask_kind = mask_kind; g.heads = c.heads;
  // Without a score buffer (inference: nothing will be back-propagated) the probabilities and the context come from one
  // kernel that never writes the scores.
  if (scores == nullptr) {
    AttnProbsCall a{};
    a.q = q.p; a.k = k.p; a.v = v.p; a.ctx = ctx; a.probs = dropped;
    a.q_st = q.ld; a.q_sh = q.stride; a.q_sb = q.stride * c.heads;
    a.k_st = k.ld; a.k_sh = k.stride; a.k_sb = k.stride * c.heads;
    a.v_st = v.ld; a.v_sh = v.stride; a.v_sb = v.stride * c.heads;
    a.c_st = ld_ctx; a.c_sh = stride_ctx; a.c_sb = stride_ctx * c.heads;
    a.mask = mask_kind != 0 ? mask : nullptr; a.mask_kind = mask_kind;
    a.batch = c.bh / c.heads; a.heads = c.heads; a.d = c.d; a.tq = c.tq; a.tk = c.tk; a.scale = c.scale; a.dtype = c.dtype;
    if (dropout_mode != 0 || softmax_out != nullptr || !attn_probs_ok(a))
      return fail(NMTG_ERR_INVALID, "attention forward: the score buffer may only be left out for an inference call (no dropout) "
                                    "with 16-bit tensors, head dimension 64 or 128 and a key count that is a multiple of 4");
    return attn_probs_run(a, c.st);
  }
  // Scores, softmax and dropout in one kernel where the call qualifies (rows of up to 512 keys, 16-byte aligned
  // operands); NMTG_ATTN_FUSED=0 always takes the two-kernel path.
  int fused = 0;
  if (!switched_off("NMTG_ATTN_FUSED")) {
    GemmArgs f = g;
    f.out2 = dropped;
    f.aux_out = softmax_out;
    if (dropout_mode != 0) {
      f.dmask = dmask;
      f.rng = dropout_mode == 2;
      f.keep_p = 1.f - p;
      f.dscale = 1.f / (1.f - p);
      f.seed = seed;
      f.offset = offset;
    }
    fused = gemm_scores_softmax_try(c.dtype, f, c.st);
    if (fused < 0) return fused;
  }
  if (!fused) {
    if (int rc = gemm_run(c.dtype, LAYOUT_NT, EPI_SCORES, g, nullptr, 0, c.st)) return rc;
    if (int rc = nmtg_softmax_dropout_fwd(scores, nullptr, 0, softmax_out, dropped, dmask, dropout_mode, p, seed, offset,
                                          static_cast<int64_t>(c.bh) * c.tq, c.tk, c.tq, c.heads, c.dtype, c.st))
      return rc;
  }
  GemmArgs h{};
  h.A = dropped; h.lda = c.tk; h.sA = static_cast<int64_t>(c.tq) * c.tk;
  h.B = v.p; h.ldb = v.ld; h.sB = v.stride;
  h.C = ctx; h.ldc = ld_ctx; h.sC = stride_ctx;
  h.M = c.tq; h.N = c.d; h.K = c.tk; h.batch = c.bh; h.alpha = 1.f;
  return gemm_run(c.dtype, LAYOUT_NN, EPI_PLAIN, h, nullptr, 0, c.st);
}

// From dctx: dv = Pd^T dctx;  dP = dctx v^T;  dS = softmax'(...);  dq = scale dS k;  dk = scale dS^T q.
// ds_buf [bh, tq, tk] is scratch.
// saved_probs: `scores` holds the softmax results instead of the masked scores (the bias-free reference extension saves
// those, encdec_multihead_attn_cuda: onmt/modules/optimized/encdec_attention_func.py:81-105); nothing is recomputed then.
int core_bwd(const Core& c, Strided q, Strided k, Strided v, Strided dctx, const void* scores, const void* dropped,
             const uint8_t* dmask, float p, void* ds_buf, void* dq, int64_t ld_dq, int64_t s_dq, void* dk, int64_t ld_dk,
             int64_t s_dk, void* dv, int64_t ld_dv, int64_t s_dv, bool saved_probs = false) {
  const int64_t tt = static_cast<int64_t>(c.tq) * c.tk;
  {  // dv [tk, d] = Pd^T [tk, tq] dctx [tq, d]
    GemmArgs g{};
    g.A = dropped; g.lda = c.tk; g.sA = tt;
    g.B = dctx.p; g.ldb = dctx.ld; g.sB = dctx.stride;
    g.C = dv; g.ldc = ld_dv; g.sC = s_dv;
    g.M = c.tk; g.N = c.d; g.K = c.tq; g.batch = c.bh; g.alpha = 1.f;
    if (int rc = gemm_run(c.dtype, LAYOUT_TN, EPI_PLAIN, g, nullptr, 0, c.st)) return rc;
  }
  const bool drop = dmask != nullptr && p > 0.f;
  {  // dP [tq, tk] = dctx [tq, d] v^T, then dS = softmax'(scores; g) in place
    GemmArgs g{};
    g.A = dctx.p; g.lda = dctx.ld; g.sA = dctx.stride;
    g.B = v.p; g.ldb = v.ld; g.sB = v.stride;
    g.C = ds_buf; g.ldc = c.tk; g.sC = tt;
    g.M = c.tq; g.N = c.tk; g.K = c.d; g.batch = c.bh; g.alpha = 1.f;
    int fused = 0;
    if (!saved_probs && !switched_off("NMTG_ATTN_FUSED")) {   // one-kernel form, see core_fwd
      GemmArgs f = g;
      f.aux_in = scores;
      f.dmask = drop ? dmask : nullptr;
      f.dscale = drop ? 1.f / (1.f - p) : 1.f;
      fused = gemm_dsoftmax_try(c.dtype, f, c.st);
      if (fused < 0) return fused;
    }
    if (!fused) {
      if (int rc = gemm_run(c.dtype, LAYOUT_NT, EPI_PLAIN, g, nullptr, 0, c.st)) return rc;
      if (int rc = nmtg_softmax_dropout_bwd(ds_buf, scores, saved_probs ? 0 : 1, nullptr, 0, drop ? dmask : nullptr, drop ? 1 : 0,
                                            drop ? p : 0.f, ds_buf, static_cast<int64_t>(c.bh) * c.tq, c.tk, c.tq, c.heads,
                                            c.dtype, c.st))
        return rc;
    }
  }
  {  // dq [tq, d] = scale dS [tq, tk] k [tk, d]
    GemmArgs g{};
    g.A = ds_buf; g.lda = c.tk; g.sA = tt;
    g.B = k.p; g.ldb = k.ld; g.sB = k.stride;
    g.C = dq; g.ldc = ld_dq; g.sC = s_dq;
    g.M = c.tq; g.N = c.d; g.K = c.tk; g.batch = c.bh; g.alpha = c.scale;
    if (int rc = gemm_run(c.dtype, LAYOUT_NN, EPI_PLAIN, g, nullptr, 0, c.st)) return rc;
  }
  {  // dk [tk, d] = scale dS^T [tk, tq] q [tq, d]
    GemmArgs g{};
    g.A = ds_buf; g.lda = c.tk; g.sA = tt;
    g.B = q.p; g.ldb = q.ld; g.sB = q.stride;
    g.C = dk; g.ldc = ld_dk; g.sC = s_dk;
    g.M = c.tk; g.N = c.d; g.K = c.tq; g.batch = c.bh; g.alpha = c.scale;
    if (int rc = gemm_run(c.dtype, LAYOUT_TN, EPI_PLAIN, g, nullptr, 0, c.st)) return rc;
  }
  return 0;
}

// y [rows, out] = x [rows, in] W^T (+ b)
int linear_fwd(int dtype, const void* x, const void* w, const void* b, void* y, int64_t rows, int64_t in_f, int64_t out_f,
               hipStream_t st) {
  GemmArgs g{};
  g.A = x; g.lda = in_f;
  g.B = w; g.ldb = in_f;
  g.C = y; g.ldc = out_f;
  g.M = static_cast<int>(rows); g.N = static_cast<int>(out_f); g.K = static_cast<int>(in_f);
  g.batch = 1; g.alpha = 1.f; g.bias = b;
  return gemm_run(dtype, LAYOUT_NT, EPI_PLAIN, g, nullptr, 0, st);
}

// dx = dy W (optional), dW = dy^T x (optional), db = colsum(dy) (optional)
int linear_bwd(int dtype, const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t rows,
               int64_t in_f, int64_t out_f, void* splitk_ws, size_t splitk_bytes, float* colsum_ws, hipStream_t st) {
  if (db) {
    if (int rc = colsum_run(dtype, dy, out_f, static_cast<int>(rows), static_cast<int>(out_f), colsum_ws, db, st)) return rc;
  }
  if (dw) {
    GemmArgs g{};
    g.A = dy; g.lda = out_f;
    g.B = x; g.ldb = in_f;
    g.C = dw; g.ldc = in_f;
    g.M = static_cast<int>(out_f); g.N = static_cast<int>(in_f); g.K = static_cast<int>(rows);
    g.batch = 1; g.alpha = 1.f;
    if (int rc = gemm_run(dtype, LAYOUT_TN, EPI_PLAIN, g, splitk_ws, splitk_bytes, st)) return rc;
  }
  if (dx) {
    GemmArgs g{};
    g.A = dy; g.lda = out_f;
    g.B = w; g.ldb = in_f;
    g.C = dx; g.ldc = in_f;
    g.M = static_cast<int>(rows); g.N = static_cast<int>(in_f); g.K = static_cast<int>(out_f);
    g.batch = 1; g.alpha = 1.f;
    if (int rc = gemm_run(dtype, LAYOUT_NN, EPI_PLAIN, g, nullptr, 0, st)) return rc;
  }
  return 0;
}

int check_attn(const char* who, int64_t tq, int64_t tk, int64_t b, int64_t e, int heads, int dtype) {
  NMTG_REQUIRE(dtype == NMTG_F16 || dtype == NMTG_BF16, "%s: dtype %d not supported (fp16 and bf16 run on MFMA)", who, dtype);
  NMTG_REQUIRE(tq > 0 && tk > 0 && b > 0 && e > 0 && heads > 0, "%s: bad shape", who);
  NMTG_REQUIRE(e % heads == 0, "%s: embed dim %lld not divisible by %d heads", who, (long long)e, heads);
  NMTG_REQUIRE(b * heads <= 65535, "%s: batch*heads %lld exceeds 65535", who, (long long)(b * heads));
  NMTG_REQUIRE(tq <= (1 << 20) && tk <= 4096 && tq * b <= INT32_MAX && tk * b <= INT32_MAX && e <= (1 << 20),
               "%s: sequence too long (tk <= 4096)", who);
  return 0;
}

struct BwdWs {
  size_t dctx, ds, dlin_a, dlin_b, colsum, splitk;
  size_t total() const { return dctx + ds + dlin_a + dlin_b + colsum + splitk; }
};

BwdWs plan_ws(int64_t tq, int64_t tk, int64_t b, int64_t e, int heads, bool self_attn) {
  BwdWs w{};
  w.dctx = align_up(static_cast<size_t>(tq) * b * e * 2);
  w.ds = align_up(static_cast<size_t>(b) * heads * tq * tk * 2);
  w.dlin_a = align_up(static_cast<size_t>(tq) * b * e * 2 * (self_attn ? 3 : 1));
  w.dlin_b = self_attn ? 0 : align_up(static_cast<size_t>(tk) * b * e * 2 * 2);
  const int64_t rows = std::max(tq, tk) * b;
  w.colsum = align_up(static_cast<size_t>(std::max<int64_t>(colsum_parts(static_cast<int>(rows)), 1)) * 3 * e * sizeof(float));
  size_t sk = gemm_splitk_workspace_bytes(static_cast<int>(e), static_cast<int>(e), static_cast<int>(tq * b), 1);
  if (self_attn) sk = std::max(sk, gemm_splitk_workspace_bytes(static_cast<int>(3 * e), static_cast<int>(e), static_cast<int>(tq * b), 1));
  else sk = std::max(sk, gemm_splitk_workspace_bytes(static_cast<int>(2 * e), static_cast<int>(e), static_cast<int>(tk * b), 1));
  w.splitk = align_up(sk);
  return w;
}

}  // namespace
}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_self_attn_fwd(const void* x, const void* w_in, const void* w_out, const void* b_in, const void* b_out,
                                  const uint8_t* mask, int mask_kind, void* lin, void* scores, void* softmax_out,
                                  void* dropped, uint8_t* dropout_mask, int dropout_mode, float p, uint64_t seed,
                                  uint64_t offset, void* ctx, void* out, int64_t t, int64_t b, int64_t e, int heads,
                                  int dtype, void* stream) {
  if (int rc = check_attn("self_attn_fwd", t, t, b, e, heads, dtype)) return rc;
  NMTG_REQUIRE(lin && ctx && (dropped || !scores), "self_attn_fwd: null buffer");
  NMTG_REQUIRE(mask_kind >= 0 && mask_kind <= 2 && (mask_kind == 0 || mask != nullptr), "self_attn_fwd: bad mask arguments");
  NMTG_REQUIRE((x == nullptr) == (w_in == nullptr), "self_attn_fwd: x and w_in go together (both NULL = compact form)");
  NMTG_REQUIRE((out == nullptr) == (w_out == nullptr), "self_attn_fwd: out and w_out go together (both NULL = compact form)");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t d = e / heads;
  if (x != nullptr) {
    if (int rc = linear_fwd(dtype, x, w_in, b_in, lin, t * b, e, 3 * e, st)) return rc;
  }
  Core c{static_cast<int>(t), static_cast<int>(t), static_cast<int>(d), static_cast<int>(b * heads), heads,
         1.f / sqrtf(static_cast<float>(d)), dtype, st};
  const int64_t ld = b * 3 * e;
  Strided q{lin, ld, 3 * d}, k{offset16(lin, d), ld, 3 * d}, v{offset16(lin, 2 * d), ld, 3 * d};
  if (int rc = core_fwd(c, q, k, v, mask, mask_kind, scores, softmax_out, dropped, dropout_mask, dropout_mode, p, seed, offset,
                        ctx, b * e, d))
    return rc;
  if (out != nullptr) return linear_fwd(dtype, ctx, w_out, b_out, out, t * b, e, e, st);
  return 0;
}

extern "C" int64_t nmtg_self_attn_bwd_workspace_bytes(int64_t t, int64_t b, int64_t e, int heads) {
  if (t <= 0 || b <= 0 || e <= 0 || heads <= 0) return 0;
  return static_cast<int64_t>(plan_ws(t, t, b, e, heads, true).total());
}

extern "C" int nmtg_self_attn_bwd(const void* grad_out, const void* ctx, const void* dropped, const void* scores,
                                  const void* lin, const void* x, const void* w_in, const void* w_out,
                                  const uint8_t* dropout_mask, float p, void* grad_x, void* grad_w_in, void* grad_w_out,
                                  void* grad_b_in, void* grad_b_out, void* grad_lin, void* workspace,
                                  int64_t workspace_bytes, int64_t t, int64_t b, int64_t e, int heads, int dtype,
                                  void* stream) {
  if (int rc = check_attn("self_attn_bwd", t, t, b, e, heads, dtype)) return rc;
  NMTG_REQUIRE(grad_out && dropped && scores && lin, "self_attn_bwd: null tensor");
  const bool compact = w_out == nullptr;  // grad_out is the context gradient, the projections are the caller's
  NMTG_REQUIRE(compact || (ctx && x && w_in), "self_attn_bwd: ctx, x and w_in are required with the projections");
  const BwdWs ws = plan_ws(t, t, b, e, heads, true);
  NMTG_REQUIRE(workspace && static_cast<size_t>(std::max<int64_t>(workspace_bytes, 0)) >= ws.total() &&
                   (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
               "self_attn_bwd: workspace of %zu bytes (256-byte aligned) required", ws.total());
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* base = static_cast<uint8_t*>(workspace);
  void* dctx = base;
  void* ds = base + ws.dctx;
  void* dlin = grad_lin ? grad_lin : static_cast<void*>(base + ws.dctx + ws.ds);
  float* colsum_ws = reinterpret_cast<float*>(base + ws.dctx + ws.ds + ws.dlin_a + ws.dlin_b);
  void* splitk_ws = base + ws.dctx + ws.ds + ws.dlin_a + ws.dlin_b + ws.colsum;
  const int64_t d = e / heads, rows = t * b;

  const void* dctx_src = grad_out;
  if (!compact) {
    if (int rc = linear_bwd(dtype, grad_out, ctx, w_out, dctx, grad_w_out, grad_b_out, rows, e, e, splitk_ws, ws.splitk,
                            colsum_ws, st))
      return rc;
    dctx_src = dctx;
  }
  Core c{static_cast<int>(t), static_cast<int>(t), static_cast<int>(d), static_cast<int>(b * heads), heads,
         1.f / sqrtf(static_cast<float>(d)), dtype, st};
  const int64_t ld = b * 3 * e;
  Strided q{lin, ld, 3 * d}, k{offset16(lin, d), ld, 3 * d}, v{offset16(lin, 2 * d), ld, 3 * d};
  Strided dc{dctx_src, b * e, d};
  if (int rc = core_bwd(c, q, k, v, dc, scores, dropped, dropout_mask, p, ds, dlin, ld, 3 * d, offset16(dlin, d), ld, 3 * d,
                        offset16(dlin, 2 * d), ld, 3 * d))
    return rc;
  if (compact) return 0;
  return linear_bwd(dtype, dlin, x, w_in, grad_x, grad_w_in, grad_b_in, rows, e, 3 * e, splitk_ws, ws.splitk, colsum_ws, st);
}

extern "C" int nmtg_encdec_attn_fwd(const void* x_q, const void* x_kv, const void* w_q, const void* w_kv, const void* w_out,
                                    const void* b_q, const void* b_kv, const void* b_out, const uint8_t* pad_mask,
                                    void* q_lin, void* kv_lin, void* scores, void* softmax_out, void* dropped,
                                    uint8_t* dropout_mask, int dropout_mode, float p, uint64_t seed, uint64_t offset,
                                    void* ctx, void* out, int64_t tq, int64_t tk, int64_t b, int64_t e, int heads,
                                    int dtype, void* stream) {
  if (int rc = check_attn("encdec_attn_fwd", tq, tk, b, e, heads, dtype)) return rc;
  NMTG_REQUIRE(q_lin && kv_lin && ctx && (dropped || !scores), "encdec_attn_fwd: null buffer");
  NMTG_REQUIRE((x_q == nullptr) == (w_q == nullptr) && (x_kv == nullptr) == (w_kv == nullptr),
               "encdec_attn_fwd: an input and its weight go together (both NULL = projection done by the caller)");
  NMTG_REQUIRE((out == nullptr) == (w_out == nullptr), "encdec_attn_fwd: out and w_out go together");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t d = e / heads;
  if (x_q != nullptr) {
    if (int rc = linear_fwd(dtype, x_q, w_q, b_q, q_lin, tq * b, e, e, st)) return rc;
  }
  if (x_kv != nullptr) {
    if (int rc = linear_fwd(dtype, x_kv, w_kv, b_kv, kv_lin, tk * b, e, 2 * e, st)) return rc;
  }
  Core c{static_cast<int>(tq), static_cast<int>(tk), static_cast<int>(d), static_cast<int>(b * heads), heads,
         1.f / sqrtf(static_cast<float>(d)), dtype, st};
  Strided q{q_lin, b * e, d}, k{kv_lin, b * 2 * e, 2 * d}, v{offset16(kv_lin, d), b * 2 * e, 2 * d};
  if (int rc = core_fwd(c, q, k, v, pad_mask, pad_mask ? 1 : 0, scores, softmax_out, dropped, dropout_mask, dropout_mode, p,
                        seed, offset, ctx, b * e, d))
    return rc;
  if (out != nullptr) return linear_fwd(dtype, ctx, w_out, b_out, out, tq * b, e, e, st);
  return 0;
}

extern "C" int64_t nmtg_encdec_attn_bwd_workspace_bytes(int64_t tq, int64_t tk, int64_t b, int64_t e, int heads) {
  if (tq <= 0 || tk <= 0 || b <= 0 || e <= 0 || heads <= 0) return 0;
  return static_cast<int64_t>(plan_ws(tq, tk, b, e, heads, false).total());
}

namespace {
int encdec_attn_bwd_run(bool saved_probs, const void* grad_out, const void* ctx, const void* dropped, const void* scores,
                        const void* q_lin, const void* kv_lin, const void* x_q, const void* x_kv,
                        const void* w_q, const void* w_kv, const void* w_out, const uint8_t* dropout_mask,
                        float p, void* grad_x_q, void* grad_x_kv, void* grad_w_q, void* grad_w_kv,
                        void* grad_w_out, void* grad_b_q, void* grad_b_kv, void* grad_b_out, void* grad_q_lin,
                        void* grad_kv_lin, void* workspace, int64_t workspace_bytes, int64_t tq, int64_t tk,
                        int64_t b, int64_t e, int heads, int dtype, void* stream) {
  if (int rc = check_attn("encdec_attn_bwd", tq, tk, b, e, heads, dtype)) return rc;
  NMTG_REQUIRE(grad_out && dropped && scores && q_lin && kv_lin, "encdec_attn_bwd: null tensor");
  const bool compact = w_out == nullptr;
  NMTG_REQUIRE(compact || (ctx && x_q && x_kv && w_q && w_kv), "encdec_attn_bwd: ctx, inputs and weights are required");
  const BwdWs ws = plan_ws(tq, tk, b, e, heads, false);
  NMTG_REQUIRE(workspace && static_cast<size_t>(std::max<int64_t>(workspace_bytes, 0)) >= ws.total() &&
                   (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
               "encdec_attn_bwd: workspace of %zu bytes (256-byte aligned) required", ws.total());
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* base = static_cast<uint8_t*>(workspace);
  void* dctx = base;
  void* ds = base + ws.dctx;
  void* dq = grad_q_lin ? grad_q_lin : static_cast<void*>(base + ws.dctx + ws.ds);
  void* dkv = grad_kv_lin ? grad_kv_lin : static_cast<void*>(base + ws.dctx + ws.ds + ws.dlin_a);
  float* colsum_ws = reinterpret_cast<float*>(base + ws.dctx + ws.ds + ws.dlin_a + ws.dlin_b);
  void* splitk_ws = base + ws.dctx + ws.ds + ws.dlin_a + ws.dlin_b + ws.colsum;
  const int64_t d = e / heads;

  const void* dctx_src = grad_out;
  if (!compact) {
    if (int rc = linear_bwd(dtype, grad_out, ctx, w_out, dctx, grad_w_out, grad_b_out, tq * b, e, e, splitk_ws, ws.splitk,
                            colsum_ws, st))
      return rc;
    dctx_src = dctx;
  }
  Core c{static_cast<int>(tq), static_cast<int>(tk), static_cast<int>(d), static_cast<int>(b * heads), heads,
         1.f / sqrtf(static_cast<float>(d)), dtype, st};
  Strided q{q_lin, b * e, d}, k{kv_lin, b * 2 * e, 2 * d}, v{offset16(kv_lin, d), b * 2 * e, 2 * d};
  Strided dc{dctx_src, b * e, d};
  if (int rc = core_bwd(c, q, k, v, dc, scores, dropped, dropout_mask, p, ds, dq, b * e, d, dkv, b * 2 * e, 2 * d,
                        offset16(dkv, d), b * 2 * e, 2 * d, saved_probs))
    return rc;
  if (compact) return 0;
  if (int rc = linear_bwd(dtype, dq, x_q, w_q, grad_x_q, grad_w_q, grad_b_q, tq * b, e, e, splitk_ws, ws.splitk, colsum_ws, st))
    return rc;
  return linear_bwd(dtype, dkv, x_kv, w_kv, grad_x_kv, grad_w_kv, grad_b_kv, tk * b, e, 2 * e, splitk_ws, ws.splitk, colsum_ws,
                    st);
}
}  // namespace

extern "C" int nmtg_encdec_attn_bwd(const void* grad_out, const void* ctx, const void* dropped, const void* scores,
                                    const void* q_lin, const void* kv_lin, const void* x_q, const void* x_kv,
                                    const void* w_q, const void* w_kv, const void* w_out, const uint8_t* dropout_mask,
                                    float p, void* grad_x_q, void* grad_x_kv, void* grad_w_q, void* grad_w_kv,
                                    void* grad_w_out, void* grad_b_q, void* grad_b_kv, void* grad_b_out, void* grad_q_lin,
                                    void* grad_kv_lin, void* workspace, int64_t workspace_bytes, int64_t tq, int64_t tk,
                                    int64_t b, int64_t e, int heads, int dtype, void* stream) {
  return encdec_attn_bwd_run(false, grad_out, ctx, dropped, scores, q_lin, kv_lin, x_q, x_kv, w_q, w_kv, w_out, dropout_mask, p,
                             grad_x_q, grad_x_kv, grad_w_q, grad_w_kv, grad_w_out, grad_b_q, grad_b_kv, grad_b_out, grad_q_lin,
                             grad_kv_lin, workspace, workspace_bytes, tq, tk, b, e, heads, dtype, stream);
}

extern "C" int nmtg_encdec_attn_bwd_from_probs(const void* grad_out, const void* ctx, const void* dropped,
                                               const void* softmax_results, const void* q_lin, const void* kv_lin,
                                               const void* x_q, const void* x_kv, const void* w_q, const void* w_kv,
                                               const void* w_out, const uint8_t* dropout_mask, float p, void* grad_x_q,
                                               void* grad_x_kv, void* grad_w_q, void* grad_w_kv, void* grad_w_out,
                                               void* grad_q_lin, void* grad_kv_lin, void* workspace, int64_t workspace_bytes,
                                               int64_t tq, int64_t tk, int64_t b, int64_t e, int heads, int dtype,
                                               void* stream) {
  return encdec_attn_bwd_run(true, grad_out, ctx, dropped, softmax_results, q_lin, kv_lin, x_q, x_kv, w_q, w_kv, w_out,
                             dropout_mask, p, grad_x_q, grad_x_kv, grad_w_q, grad_w_kv, grad_w_out, nullptr, nullptr, nullptr,
                             grad_q_lin, grad_kv_lin, workspace, workspace_bytes, tq, tk, b, e, heads, dtype, stream);
}
