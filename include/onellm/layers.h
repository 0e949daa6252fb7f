// The decode-side layers of oneLLM over this backend: launchLinearGemm, LLaMASelfAttentionLayer, LLaMAFFNLayer and
// LlamaSelfDecoder with the constructor and forward() signatures of
//   src/kernels/qkv_linear.h:9-14
//   src/layers/attention/masked_self_attention.h:13-55
//   src/layers/ffn/ffn.h
//   src/layers/decoder/self_decoder.h:10-74
// so that a driver written like examples/cpp/decoder/self_decoder_example.cpp builds against them.  They own no
// arithmetic: every step is one of the launch* functions of onellm/kernels.h or a library GEMM.
//
// One decode step (B sequences, one new token each), as LlamaSelfDecoder::forward runs it:
//   y <- RMSNorm(x, attn_norm[0])                                  x = "decoder_input" (the residual stream),
//   per layer l:                                                   y = "decoder_output"
//     qkv <- y . Wqkv ; a <- masked attention(qkv + bias, RoPE, cache slab l) ; y <- a . Wo
//     x <- x + y + bo ; y <- RMSNorm(x, ffn_norm[l])               (launchFusedAddBiasResidualRMSNorm)
//     y <- (silu(y . Wgate) * (y . Wup)) . Wdown
//     x <- x + y + bdown ; y <- RMSNorm(x, attn_norm[l+1] or output_norm_weight)
// Element type (FP32 or FP16) follows "decoder_input".  Everything is queued on one stream (see below);
// forward() returns without synchronising.
//
// Where this differs from the reference snapshot, on purpose (the snapshot cannot produce a decoder output):
//   * src/layers/decoder/self_decoder.cpp:19 normalises decoder_input in place and then uses it as the residual;
//     here the normalised copy goes to decoder_output and decoder_input stays the residual stream;
//   * src/layers/ffn/ffn.cpp:68 leaves the FFN result in a private buffer; here it is written to "ffn_output";
//   * src/kernels/qkv_linear.cu:35-38 computes the offset of the shared gate/up buffer into a shadowed variable,
//     so `up` overwrites `gate`; here shared_out_buf writes the second [M, N] half;
//   * src/layers/attention/masked_self_attention.cpp:72 always addresses cache layer 0; here layer l gets slab l;
//   * src/kernels/decoder_masked_attn.cu:186 rotates the new token as position `step`, one past the 0-based position
//     the context phase gave the cached rows (src/kernels/qkv_bias_and_RoPE.cu:140); the attention layer here rotates
//     it as position step - 1 by default, which is what a cache written by prefill (or by earlier decode steps of this
//     layer) needs; setRopePositionOffset(0) restores the kernel's own convention;
//   * no device synchronisation after each launch (src/layers/decoder/self_decoder.cpp:22,50,67).
#pragma once
#include <cstddef>
#include <vector>
#include "onellm/allocator.h"
#include "onellm/kernels.h"
#include "onellm/tensor_map.h"
#include "onellm/weights.h"

class cublasWrapper;   // carried for signature compatibility only; may be null, never dereferenced
// `stream` arguments: the attention and FFN layers queue where the launch* functions do (onellmSetLaunchStream, the
// null stream by default, as in the reference).  A LlamaSelfDecoder constructed with a non-null stream queues its
// whole step there, which is what makes a step capturable into a HIP graph: run one step first (buffers, the
// attention workspace and the GEMM plans are created on first use), then capture.

// output[M, N] = input[M, K] . weight, weight.shape = {K, N} (or {N, K} with trans_b); M = input->shape[0], K = the
// product of the remaining input dimensions.  shared_out_buf: write the second [M, N] half of a [2, M, N] output.
void launchLinearGemm(Tensor* input, BaseWeight& weight, Tensor* output, bool trans_a = false, bool trans_b = false,
                      bool shared_out_buf = false);

// Both projections of a feed-forward block that share their input (the reference calls launchLinearGemm twice,
// src/layers/ffn/ffn.cpp:61-62): output {2, M, N} holds first's result in its first half and second's in the other,
// rows interleaved as [M, 2, N], exactly as the two calls leave it; where the few-row kernel of the projection
// library takes the problem both go out in one launch.  The weights are {K, N} matrices of one shape.
void launchLinearGemmPair(Tensor* input, BaseWeight& first, BaseWeight& second, Tensor* output);

// launchLinearGemm times the GEMM library's candidate algorithms the first time it sees a shape and keeps the fastest;
// that first call synchronises the null stream.  Switch it off to keep every call asynchronous (for example before
// capturing a step into a graph; shapes tuned earlier stay tuned).
void setLinearGemmAutotune(bool on);
// A projection the GEMM library has no kernel for throws unless it is tiny (unit-test and example-driver sizes) or
// the plain kernel - about a hundred times slower - has been allowed here.
void setLinearGemmPlainFallback(bool allow);
// Number of GEMM workspaces alive: one per (device, launch stream) that has run a projection.
size_t linearGemmWorkspaceCount();
// Before a stream that ran projections is destroyed: waits for the stream, frees the GEMM workspace the current
// device keeps for it and gives the workspace's arrival-counter sets back (onellm_release_workspace).  Returns
// whether there was one.  Graphs captured on that stream must not be replayed afterwards.
bool releaseLinearGemmWorkspace(hipStream_t stream);

class LLaMASelfAttentionLayer {
public:
    LLaMASelfAttentionLayer(int head_num, int kv_head_num, int head_size, LLaMAAttentionStaticParams attn_params,
                            hipStream_t stream, cublasWrapper* cublas_wrapper, BaseAllocator* allocator,
                            bool is_free_buffer_after_fwd);
    ~LLaMASelfAttentionLayer();
    LLaMAAttentionStaticParams& GetAttnStaticParams() { return attn_static_params; }
    void setRopePositionOffset(int offset) { rope_pos_offset = offset; }
    template<typename T> void allocForForward(LLaMAAttentionDynParams& params);
    void free();
    // inputs: "attention_input" [B, hidden], "step" (host int), "finished" [B], "layer_id" (host int)
    // outputs: "attention_output" [B, hidden], "all_k_cache", "all_v_cache" [L, B, Hkv, S, D]
    void forward(TensorMap& inputs, TensorMap& outputs, LLaMAattentionWeights& weights, LLaMAAttentionDynParams& params);

private:
    const int  head_num;
    const int  head_size;
    const int  hidden_units;
    const int  kv_head_num;
    const bool is_free_buffer_after_fwd;
    LLaMAAttentionStaticParams attn_static_params;
    BaseAllocator* allocator;
    int rope_pos_offset = -1;
    Tensor* qkv_buf    = nullptr;
    Tensor* mha_output = nullptr;
};

class LLaMAFFNLayer {
public:
    LLaMAFFNLayer(int head_num, int head_size, int inter_size, hipStream_t stream, cublasWrapper* cublas_wrapper,
                  BaseAllocator* allocator, bool is_free_buffer_after_fwd);
    ~LLaMAFFNLayer();
    template<typename T> void allocForForward(LLaMAAttentionDynParams& params);
    template<typename T> void allocForForward(int batch_size);
    void free();
    // inputs: "ffn_input" [N, hidden]; outputs: "ffn_output" [N, hidden] (may be the same buffer)
    void forward(TensorMap& inputs, TensorMap& outputs, LLaMAFFNWeights& weights, LLaMAAttentionDynParams& params);

private:
    const int  inter_size;
    const int  hidden_units;
    const bool is_free_buffer_after_fwd;
    BaseAllocator* allocator;
    Tensor* SwiGLU_input    = nullptr;   // [2, N, inter]: gate rows, then up rows
    Tensor* down_proj_input = nullptr;   // [N, inter]
};

class LlamaSelfDecoder {
public:
    LlamaSelfDecoder(int head_num, int kv_head_num, int head_size, int inter_size, int num_layer,
                     const LLaMAAttentionStaticParams& attn_params, float rmsnorm_eps, hipStream_t stream,
                     cublasWrapper* cublas_wrapper, BaseAllocator* allocator, bool is_free_buffer_after_forward);
    ~LlamaSelfDecoder();
    template<typename T> void allocForForward(LLaMAAttentionDynParams& dyn_params);
    void free();
    LLaMASelfAttentionLayer* attention() { return selfAttn; }
    // input_tensors: "decoder_input" [B, hidden] (updated: the residual stream), "step", "finished",
    //                "output_norm_weight" [hidden]
    // output_tensors: "decoder_output" [B, hidden], "all_k_cache", "all_v_cache"
    void forward(TensorMap& input_tensors, const std::vector<LlamaLayerWeight*>& layerWeights, TensorMap& output_tensors,
                 LLaMAAttentionDynParams& dyn_params);

private:
    int   num_layer;
    int   hidden_units;
    float rmsnorm_eps;
    hipStream_t stream;
    LLaMASelfAttentionLayer* selfAttn;
    LLaMAFFNLayer*           ffn;
};
