/* C surface of the decode-side layers (exported by libonellm_layers.so) for callers that cannot construct the C++
 * objects of onellm/layers.h — Python, C, other FFIs.  No counterpart in the reference, whose layers are only
 * reachable from C++ (examples/cpp/decoder/self_decoder_example.cpp builds the objects by hand); each call below does
 * what that driver does and then calls the C++ method named.  Return code 0 = ok, 1 = a C++ exception was caught and
 * its text is available from onellm_layers_last_error() (per thread).  All pointers are device pointers unless noted;
 * dtype is ONELLM_FP32 or ONELLM_FP16 for every tensor and weight of a call.
 */
#ifndef ONELLM_LAYERS_H
#define ONELLM_LAYERS_H
#include "onellm_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

const char* onellm_layers_last_error(void);

/* launchLinearGemm (src/kernels/qkv_linear.h:9-14): y = x[M, K] . W.  trans_b: W is [N, K] instead of [K, N].
 * pair: y is the {2, M, N} gate/up buffer of the FFN (rows interleaved as [M, 2, N]); second: write its second slot. */
int onellm_layers_linear(int dtype, void* x, void* w, void* y, int M, int K, int N, int trans_b, int pair, int second);

/* setLinearGemmPlainFallback / linearGemmWorkspaceCount of onellm/layers.h: whether a projection the GEMM library
 * declines may run the plain kernel whatever its size (off by default: a large one throws); how many GEMM workspaces
 * exist (one per device and launch stream that has run a projection). */
int onellm_layers_allow_plain_gemm(int allow);
int onellm_layers_gemm_workspace_count(void);
/* releaseLinearGemmWorkspace of onellm/layers.h: before a launch stream is destroyed, waits for it, frees the GEMM
 * workspace the current device keeps for it and gives its arrival-counter sets back.  1: freed, 0: the stream had
 * none, -1: error (onellm_layers_last_error). */
int onellm_layers_release_gemm_workspace(onellm_stream_t stream);

/* A LlamaSelfDecoder (src/layers/decoder/self_decoder.h:10-74) with its layer weights and an allocator.
 * The ten `void**` are host arrays of L device pointers, in the order of LlamaLayerWeight::loadWeights
 * (src/weights/llama/layer_weights.h:32-41); with attn_bias == 0 the qkv / output biases are ignored; bdown[l] may be
 * NULL.  Weights are [in, out] row-major.  The weight buffers must outlive the decoder.  stream: where every step of
 * this decoder is queued (NULL = the null stream).  Returns NULL on failure. */
void* onellm_decoder_create(int dtype, int B, int Hq, int Hkv, int D, int inter_size, int L, int S, int rotary_dim,
                            float rope_base, float rmsnorm_eps, int attn_bias, void** attn_norm, void** ffn_norm,
                            void** wqkv, void** bqkv, void** wo, void** bo, void** wdown, void** bdown, void** wgate,
                            void** wup, void* output_norm, onellm_stream_t stream);

/* LlamaSelfDecoder::forward for one step: decoder_input [B, Hq*D] is the residual stream (updated), decoder_output
 * [B, Hq*D] receives the final normalised activations, the caches are [L, B, Hkv, S, D] and get row step-1 of every
 * layer.  step = attended positions including the new token, the same for the whole batch.  Queued on the
 * decoder's stream; returns without synchronising.  After one ordinary step (which creates buffers and GEMM plans)
 * further steps allocate nothing and may be captured into a HIP graph on that stream. */
int onellm_decoder_forward(void* decoder, int step, void* decoder_input, void* decoder_output, void* k_cache, void* v_cache);

void onellm_decoder_destroy(void* decoder);

#ifdef __cplusplus
}
#endif
#endif
