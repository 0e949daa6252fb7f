// The six launcher functions of the decode hot path, with the signatures the oneLLM layers and
// unit tests call.  Each is a thin shim over the C ABI in onellm_hip.h: it unpacks shapes the
// way the reference launcher does and throws std::runtime_error on a non-zero return code.
#pragma once
#include <hip/hip_runtime_api.h>
#include "onellm/tensor.h"
#include "onellm/weights.h"
#include "onellm/params.h"

// Stream the launch* functions below queue on, per calling thread; the default is the null stream, which is where
// the reference launches everything.  No counterpart in the reference: it is for callers that own a stream, for
// example to capture a decode step into a HIP graph (the null stream cannot be captured).
void onellmSetLaunchStream(hipStream_t stream);
hipStream_t onellmGetLaunchStream();

// src/kernels/decoder_masked_attn.h:7-14
void launchDecoderMaskedMHA(Tensor* qkv_buf,
                            BaseWeight& qkv,
                            Tensor* k_cache,
                            Tensor* v_cache,
                            Tensor* finished,
                            Tensor* step,
                            Tensor* mha_output,
                            LLaMAAttentionStaticParams& static_params);

// The same with the RoPE position stated: the token at cache row step-1 is rotated as position
// step + rope_pos_offset.  The 8-argument form is offset 0 (src/kernels/decoder_masked_attn.cu:186 rotates with
// `step`); -1 is the 0-based position the context-phase kernel gives the same row
// (src/kernels/qkv_bias_and_RoPE.cu:140), i.e. what a cache filled by prefill needs.
void launchDecoderMaskedMHA(Tensor* qkv_buf,
                            BaseWeight& qkv,
                            Tensor* k_cache,
                            Tensor* v_cache,
                            Tensor* finished,
                            Tensor* step,
                            Tensor* mha_output,
                            LLaMAAttentionStaticParams& static_params,
                            int rope_pos_offset);

// src/kernels/rmsnorm_kernel.h:6-9
void launchRMSNorm(Tensor* decoder_out, LayerNormWeight& attn_norm_weight, float eps);

// src/kernels/fused_addresidual_norm.h:4-12 (float as in the reference, half added)
template<typename T>
void launchFusedAddBiasResidualRMSNorm(T* residual,
                                       T* decoder_out,
                                       const T* bias,
                                       const T* scale,
                                       float eps,
                                       int num_tokens,
                                       int hidden_units);

// src/kernels/append_to_kvcache.h:20-26
void launchAppendKVCache(Tensor* k_src,
                         Tensor* v_src,
                         Tensor* layer_id,
                         Tensor* cur_query_length,
                         Tensor* history_length,
                         Tensor* k_dst,
                         Tensor* v_dst);

// src/kernels/transpose_kernel.h:5-11
void launchTransposeKVCache(Tensor* k_cache_src,
                            Tensor* v_cache_src,
                            Tensor* context_length,
                            Tensor* layer_id,
                            Tensor* k_cache_dst,
                            Tensor* v_cache_dst);

// src/kernels/beamsearch_topK.h:35-38
void launchTopKforBeamSearch(const float* probs,
                             const int batch_size,
                             const int vocab_size,
                             float* topk_workspace);

// src/kernels/qkv_bias_and_RoPE.h (context phase; produces the K/V the decode step reads)
void launchAddFusedQKVBiasTransposeAndRoPE(Tensor* q_buf,
                                           Tensor* k_buf,
                                           Tensor* v_buf,
                                           Tensor* QKV,
                                           BaseWeight& qkv,
                                           Tensor* padding_offset,
                                           Tensor* history_length,
                                           Tensor* input_length,
                                           LLaMAAttentionStaticParams& params);

// src/kernels/activation_kernel.h (float as in the reference, half added)
template<typename T>
void launchAct(const T* input, T* out, const int batch_size, const int intermedia_size);

// src/kernels/topK_sampling.h
void launchSampling(Tensor* topk_id,
                    Tensor* topk_val,
                    Tensor* seqlen,
                    Tensor* is_finished,
                    Tensor* output_id,
                    IntDict& params);
