/*
 * nmtg_hip.h — C ABI of libnmtg_hip.so: MI355X (gfx950) kernels for the fused transformer-layer
 * ops of NMTGMinor (LayerNorm, fused MLP, self / encoder-decoder attention, masked softmax +
 * dropout, dropout + residual add, label-smoothed softmax cross-entropy).
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers owned by the caller. The library never allocates, frees
 *     or keeps device memory, and holds no state between calls apart from the last error text.
 *   - Tensors are dense row-major unless a leading dimension / stride argument says otherwise.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream). Calls only enqueue
 *     work on that stream; they never synchronise the device.
 *   - Element types are named by nmtg_dtype codes.
 *   - Return value: 0 on success, a negative nmtg_status otherwise; nmtg_last_error() then
 *     returns a human-readable reason (thread-local). No entry point aborts or exits.
 *
 * Each declaration cites the interface of the reference tree (paths relative to the NMTGMinor
 * checkout) that it stands in for.
 */
#ifndef NMTG_HIP_H_
#define NMTG_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { NMTG_F32 = 0, NMTG_F16 = 1, NMTG_BF16 = 2 } nmtg_dtype;

typedef enum {
  NMTG_OK = 0,
  NMTG_ERR_INVALID = -1,     /* bad argument: shape, dtype, alignment, null pointer */
  NMTG_ERR_UNSUPPORTED = -2, /* valid request that this build has no kernel for */
  NMTG_ERR_LAUNCH = -3       /* HIP reported an error when the kernel was enqueued */
} nmtg_status;

/* Activation codes of the fused MLP. Reference: the per-activation extension modules
 * onmt/modules/extensions/mlp/mlp_{relu,gelu,silu,agelu}.cpp and the plain mlp.cpp. */
typedef enum {
  NMTG_ACT_NONE = 0,
  NMTG_ACT_RELU = 1,
  NMTG_ACT_GELU = 2,  /* exact erf form */
  NMTG_ACT_SILU = 3,
  NMTG_ACT_AGELU = 4  /* tanh approximation, 0.044715 */
} nmtg_act;

/* Library version (major*10000 + minor*100 + patch) and the last error of the calling thread. */
int nmtg_version(void);
const char* nmtg_last_error(void);

/* ------------------------------------------------------------------------------------------
 * LayerNorm.
 * Reference: fast_layer_norm_cuda.ln_fwd / ln_bwd,
 *   onmt/modules/extensions/layer_norm/ln_api.cpp:80-153 (ln_fwd), :156-249 (ln_bwd).
 *
 * x [rows, hidden] of in_dtype; gamma, beta [hidden] of w_dtype; z [rows, hidden] of w_dtype
 * (the reference forms the output in the weight dtype); mu, rsigma [rows] fp32.
 * Any hidden size is accepted (the reference registers 25 sizes, ln_fwd_cuda_kernel.cu:73-233).
 * ------------------------------------------------------------------------------------------ */
int nmtg_ln_fwd(const void* x, const void* gamma, const void* beta, void* z, float* mu,
                float* rsigma, int64_t rows, int64_t hidden, float eps, int in_dtype, int w_dtype,
                void* stream);

/* Number of partial rows ln_bwd writes: dgamma_part / dbeta_part are [n_part, hidden] fp32
 * (the reference's ctas_per_col, ln_api.cpp:214-215). */
int64_t nmtg_ln_bwd_parts(int64_t rows, int64_t hidden);

/* dz [rows, hidden] w_dtype; x_or_z [rows, hidden] in_dtype (x, or z when memory_efficient);
 * mu may be NULL and beta is required when memory_efficient != 0; dx [rows, hidden] in_dtype;
 * dgamma, dbeta [hidden] w_dtype; dgamma_part, dbeta_part [n_part, hidden] fp32 workspace that
 * is also an output, with n_part == nmtg_ln_bwd_parts(rows, hidden). */
int nmtg_ln_bwd(const void* dz, const void* x_or_z, const float* mu, const float* rsigma,
                const void* gamma, const void* beta, void* dx, void* dgamma, void* dbeta,
                float* dgamma_part, float* dbeta_part, int64_t n_part, int64_t rows,
                int64_t hidden, int memory_efficient, int in_dtype, int w_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NMTG_HIP_H_ */
