/* C ABI of the projection GEMMs around the decode path (exported by libonellm_gemm.so).
 *
 * Replaces launchLinearGemm (src/kernels/qkv_linear.cu:8-66, declared src/kernels/qkv_linear.h:9-14) and the
 * cublasWrapper::Gemm call under it (src/kernels/cublas_wrapper.cc:33-85).  The multiplication itself is a library
 * GEMM (hipBLASLt, fp32 accumulation); this entry point adds what the reference re-creates on every call: a handle
 * per device and a cached plan per (dtype, M, K, N, layout).  For the few rows of a decode step (fp16 or fp32, W as
 * [K, N], M <= 32, K a multiple of 64, rows of W in whole 16-byte pieces) the library also holds a kernel of its own
 * that streams the weights once through the matrix cores; onellm_linear_tune times it beside the library's
 * algorithms and onellm_linear runs whichever won.  Small shapes the library has no kernel for (unit-test and example-driver sizes, up to 2^24
 * multiply-adds) run a plain kernel in this library; a larger one returns ONELLM_ENOGEMMKERNEL unless the caller has
 * allowed the plain kernel, which is about a hundred times slower.
 *
 * Kept out of libonellm_hip.so so that the decode-path kernels do not pull in the BLAS library.
 */
#ifndef ONELLM_GEMM_H
#define ONELLM_GEMM_H
#include <stddef.h>
#include "onellm_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* y[M, N] = x[M, K] . W, row-major, fp32 accumulation, y rounded once to `dtype`.  x and W are contiguous; row m
 * of y starts at y + m * ldy elements (ldy >= N; 0 means N), so two projections can write the two halves of one
 * [M, 2, N] buffer — the layout the SwiGLU kernel reads (src/kernels/activation_kernel.cu:11-13).
 *   w_is_nk == 0:  W is [K, N]  (the layout of every BaseWeight the oneLLM layers hold: shape = {in, out},
 *                  src/weights/llama/layer_weights.cc:21-41)
 *   w_is_nk != 0:  W is [N, K]  (y = x . W^T; launchLinearGemm's trans_b)
 * workspace: device scratch for the library's split-K algorithms; may be NULL/0, then only algorithms that need
 * none are considered.  Returns 0, an ONELLM_E* code, or a hipError_t. */
int onellm_linear(int dtype, const void* x, const void* w, void* y, int M, int K, int N, int ldy, int w_is_nk,
                  void* workspace, size_t workspace_bytes, onellm_stream_t stream);

/* Optional, once per shape (for example when a model is loaded): times the library's candidate algorithms and, where
 * it applies, the configurations of this library's few-row kernel for this problem on stand-in operands it allocates
 * and frees itself, and makes onellm_linear use the fastest for this (dtype, M, K, N, ldy, w_is_nk, workspace or not)
 * from then on instead of the library's first suggestion.  The timing runs rotate over enough copies of W (640 MB, at
 * most 16) that every run meets its matrix cold, as a projection inside a model does.  Synchronises the stream.
 * best_us / first_us (either may be NULL) receive the time of the chosen algorithm and of the library's first
 * suggestion.  ONELLM_EUNSUPPORTED if nothing takes the problem. */
int onellm_linear_tune(int dtype, int M, int K, int N, int ldy, int w_is_nk, void* workspace, size_t workspace_bytes,
                       onellm_stream_t stream, float* best_us, float* first_us);

/* Two projections that share their input and shape - the gate and up projections of a feed-forward block
 * (src/layers/ffn/ffn.cpp:61-62 calls launchLinearGemm twice): y_first = x . w_first, y_second = x . w_second, both
 * with row stride ldy.  The result is that of two onellm_linear calls; where this library's few-row kernel takes the
 * problem and onellm_linear_pair_tune found it faster, both go out in one launch. */
int onellm_linear_pair(int dtype, const void* x, const void* w_first, const void* w_second, void* y_first, void* y_second,
                       int M, int K, int N, int ldy, int w_is_nk, void* workspace, size_t workspace_bytes,
                       onellm_stream_t stream);

/* Optional, once per shape: onellm_linear_tune for the single projection, then the one-launch forms of the pair
 * against two tuned calls, on stand-in operands as above.  best_us / two_calls_us (either may be NULL) receive the time
 * of what onellm_linear_pair will run from then on and of the two-call sequence. */
int onellm_linear_pair_tune(int dtype, int M, int K, int N, int ldy, int w_is_nk, void* workspace, size_t workspace_bytes,
                            onellm_stream_t stream, float* best_us, float* two_calls_us);

/* workspace size onellm_linear can make use of (a constant; any smaller size is valid too) */
size_t onellm_linear_workspace_bytes(void);

/* what the last onellm_linear / onellm_linear_pair call on this thread ran: 1 the library GEMM, 2 this library's
 * few-row kernel, 3 that kernel for both projections of a pair in one launch, 0 the plain fallback kernel; and, when
 * the tuned configuration cuts the problem along K but every arrival-counter set of this GPU belongs to another
 * workspace (onellm_hip.h, onellm_release_workspace): 4 the few-row kernel uncut, 5 the library GEMM - same results,
 * slower than the tuned form */
int onellm_linear_last_path(void);

/* allow != 0: problems of any size may run the plain kernel when the library declines them (process-wide; off by
 * default, so that a projection of a real model never becomes a hundred times slower without an error).  Returns
 * the previous setting. */
int onellm_linear_allow_plain(int allow);

#ifdef __cplusplus
}
#endif
#endif
