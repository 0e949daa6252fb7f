// The six launch* functions of oneLLM's decode path, with oneLLM's own signatures, as shims over
// the C ABI.  Each unpacks shapes the way the reference launcher does (cited per function), calls
// the C entry point on the null stream (the reference launches everything there; onellmSetLaunchStream names
// another one for the calling thread) and throws
// std::runtime_error when the entry point reports an error.  No printing, no device sync.
#include <map>
#include <mutex>
#include <utility>
#include <stdexcept>
#include <string>
#include <hip/hip_runtime_api.h>
#include "onellm/kernels.h"
#include "onellm_hip.h"

namespace {
thread_local hipStream_t t_launch_stream = nullptr;
void* launch_stream() { return t_launch_stream; }
}  // namespace

void onellmSetLaunchStream(hipStream_t stream) { t_launch_stream = stream; }
hipStream_t onellmGetLaunchStream() { return t_launch_stream; }

namespace {

void throw_on_error(int rc, const char* what)
{
    if (rc != 0) {
        throw std::runtime_error(std::string("[TM][ERROR] ") + what + ": " + onellm_error_string(rc) + " \n");
    }
}

int abi_dtype(const Tensor* t, const char* what)
{
    if (t->dtype == FP32) return ONELLM_FP32;
    if (t->dtype == FP16) return ONELLM_FP16;
    throw std::runtime_error(std::string("[oneLLM][ERROR] ") + what + ": only FP32 and FP16 tensors are supported \n");
}

// The reference signature of the attention launcher has no workspace parameter, so the shim owns
// grow-only device buffers (freed at exit by the runtime): one per (device, launch stream), so
// that steps queued on different streams or devices never share scratch.
struct Workspace {
    struct Buffer {
        void* ptr = nullptr;
        size_t bytes = 0;
    };
    std::mutex mu;
    std::map<std::pair<int, hipStream_t>, Buffer> buffers;
    void* get(size_t need, hipStream_t stream)
    {
        int device = 0;
        throw_on_error((int)hipGetDevice(&device), "workspace device");
        std::lock_guard<std::mutex> g(mu);
        Buffer& b = buffers[std::make_pair(device, stream)];
        if (need > b.bytes) {
            // creating (or growing) the buffer synchronises, allocates and clears: none of that may be recorded
            // into a graph, so a stream that is being captured is refused - run one ordinary step first
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) (void)hipGetLastError();
            if (capturing != hipStreamCaptureStatusNone)
                throw std::runtime_error("[oneLLM][ERROR] launchDecoderMaskedMHA: this step needs the attention workspace to be "
                                         "created or grown, which cannot be done while the launch stream is being captured; "
                                         "run one ordinary step on this stream first \n");
            // the old buffer may still be in use by work queued earlier on its stream
            if (b.ptr) {
                throw_on_error((int)hipStreamSynchronize(stream), "workspace sync");
                throw_on_error((int)hipFree(b.ptr), "workspace free");
                b.ptr = nullptr;
                b.bytes = 0;
            }
            throw_on_error((int)hipMalloc(&b.ptr, need), "workspace alloc");
            // zero-filled once: the attention entry point may then finish split sequences in one launch
            // (ONELLM_ATTN_ZEROED_WORKSPACE); only that entry point ever writes the buffer
            throw_on_error((int)hipMemsetAsync(b.ptr, 0, need, stream), "workspace clear");
            b.bytes = need;
        }
        return b.ptr;
    }
};
Workspace g_attn_ws;

// A cache tensor is either the 5-D [num_layers, B, Hkv, S, D] the layers allocate
// (examples/cpp/decoder/self_decoder_example.cpp:186-187) or the 4-D [B, Hkv, S, D] the kernel
// unit tests build (tests/unittests/test_append_kvcache.cu:74).
struct CacheShape {
    int layers, B, Hkv, S, D;
};
CacheShape cache_shape(const Tensor* c, const char* what)
{
    const auto& s = c->shape;
    if (s.size() == 5) return {s[0], s[1], s[2], s[3], s[4]};
    if (s.size() == 4) return {1, s[0], s[1], s[2], s[3]};
    throw std::runtime_error(std::string("[oneLLM][ERROR] ") + what + ": KV cache must be 4-D or 5-D \n");
}

// layer_id is used only when it is host-resident; a device tensor is never dereferenced on the
// host (the reference warns about exactly that, src/kernels/transpose_kernel.cu:60) and means 0.
int host_layer_id(const Tensor* layer_id)
{
    if (layer_id && layer_id->data && layer_id->location != GPU && layer_id->dtype == INT32) return *(const int*)layer_id->data;
    return 0;
}

}  // namespace

// src/kernels/decoder_masked_attn.cu:280-327
void launchDecoderMaskedMHA(Tensor* qkv_buf, BaseWeight& qkv, Tensor* k_cache, Tensor* v_cache, Tensor* finished,
                            Tensor* step, Tensor* mha_output, LLaMAAttentionStaticParams& static_params)
{
    launchDecoderMaskedMHA(qkv_buf, qkv, k_cache, v_cache, finished, step, mha_output, static_params, /*rope_pos_offset=*/0);
}

void launchDecoderMaskedMHA(Tensor* qkv_buf, BaseWeight& qkv, Tensor* k_cache, Tensor* v_cache, Tensor* finished,
                            Tensor* step, Tensor* mha_output, LLaMAAttentionStaticParams& static_params, int rope_pos_offset)
{
    (void)finished;   // unused by the reference as well (:284)
    ONELLM_CHECK_WITH_INFO(qkv_buf && k_cache && v_cache && step && mha_output, "null tensor");
    ONELLM_CHECK_WITH_INFO(qkv_buf->shape.size() == 3, "qkv_buf must be [B, Hq+2Hkv, D]");
    ONELLM_CHECK_WITH_INFO(step->location != GPU && step->data, "step must be a host tensor");
    const int dtype = abi_dtype(qkv_buf, "launchDecoderMaskedMHA");
    const int batch_size = qkv_buf->shape[0];          // :289
    const int qkv_head_num = qkv_buf->shape[1];        // :290
    const int head_size = qkv_buf->shape[2];           // :293
    const CacheShape cs = cache_shape(k_cache, "launchDecoderMaskedMHA");
    const int kv_head_num = cs.Hkv;                    // :291 (shape[2] of the 5-D tensor)
    const int head_num = qkv_head_num - 2 * kv_head_num;   // :292
    const int cur_step = *(const int*)step->data;      // :294
    ONELLM_CHECK_WITH_INFO(cs.B == batch_size && cs.D == head_size, "KV cache does not match qkv_buf");
    ONELLM_CHECK_WITH_INFO(head_num > 0 && cur_step >= 1 && cur_step <= cs.S, "step outside [1, max_seq_len]");
    // Most shapes need no scratch (a single sequence split); the buffer is only created when the
    // entry point asks for one.
    auto call = [&](void* ws, size_t ws_bytes) {
        return onellm_decode_attn(dtype, qkv_buf->data, qkv.bias, k_cache->data, v_cache->data, mha_output->data,
                                  batch_size, head_num, kv_head_num, head_size, cs.S, /*layer=*/0, cs.layers,
                                  cur_step, nullptr, cur_step,
                                  static_params.rotary_embedding_dim, static_params.rotary_embedding_base,
                                  rope_pos_offset, ONELLM_ATTN_ZEROED_WORKSPACE, ws, ws_bytes, launch_stream());
    };
    int rc = call(nullptr, 0);
    if (rc == ONELLM_EWORKSPACE) {
        // sized for the cache's whole length, so that it is created once and not regrown as the step advances
        const size_t ws_bytes = onellm_decode_attn_workspace_bytes(batch_size, head_num, kv_head_num, head_size, cs.S);
        rc = call(g_attn_ws.get(ws_bytes, t_launch_stream), ws_bytes);
    }
    throw_on_error(rc, "launchDecoderMaskedMHA");
}

// src/kernels/rmsnorm_kernel.cu:85-103.  LayerNormWeight carries `float* gamma`; for an FP16
// tensor the same field is taken to point at fp16 values.
void launchRMSNorm(Tensor* decoder_out, LayerNormWeight& attn_norm_weight, float eps)
{
    ONELLM_CHECK_WITH_INFO(decoder_out && decoder_out->shape.size() == 2, "decoder_out must be [num_tokens, hidden]");
    const int num_tokens = decoder_out->shape[0];      // :90
    const int hidden_units = decoder_out->shape[1];    // :91
    const int rc = onellm_rmsnorm(abi_dtype(decoder_out, "launchRMSNorm"), decoder_out->data, attn_norm_weight.gamma,
                                  eps, num_tokens, hidden_units, launch_stream());
    throw_on_error(rc, "launchRMSNorm");
}

// src/kernels/fused_addresidual_norm.cu:109-141
template <typename T>
void launchFusedAddBiasResidualRMSNorm(T* residual, T* decoder_out, const T* bias, const T* scale, float eps,
                                       int num_tokens, int hidden_units)
{
    const int dtype = std::is_same<T, half>::value ? ONELLM_FP16 : ONELLM_FP32;
    const int rc = onellm_fused_add_bias_residual_rmsnorm(dtype, residual, decoder_out, bias, scale, eps, num_tokens,
                                                          hidden_units, launch_stream());
    throw_on_error(rc, "launchFusedAddBiasResidualRMSNorm");
}
template void launchFusedAddBiasResidualRMSNorm(float*, float*, const float*, const float*, float, int, int);
template void launchFusedAddBiasResidualRMSNorm(half*, half*, const half*, const half*, float, int, int);

// src/kernels/append_to_kvcache.cu:73-114
void launchAppendKVCache(Tensor* k_src, Tensor* v_src, Tensor* layer_id, Tensor* cur_query_length,
                         Tensor* history_length, Tensor* k_dst, Tensor* v_dst)
{
    ONELLM_CHECK_WITH_INFO(k_src && v_src && cur_query_length && history_length && k_dst && v_dst, "null tensor");
    ONELLM_CHECK_WITH_INFO(k_src->shape.size() == 4, "k_src must be [B, Hkv, max_q_len, D]");
    const int batch_size = k_src->shape[0];            // :81
    const int kv_head_num = k_src->shape[1];           // :83
    const int max_q_len = k_src->shape[2];             // :84
    const int head_size = k_src->shape[3];             // :85
    const CacheShape cs = cache_shape(k_dst, "launchAppendKVCache");
    ONELLM_CHECK_WITH_INFO(cs.B == batch_size && cs.Hkv == kv_head_num && cs.D == head_size, "cache does not match k_src");
    const int rc = onellm_kv_append(abi_dtype(k_src, "launchAppendKVCache"), k_src->data, v_src->data, k_dst->data,
                                    v_dst->data, (const int*)cur_query_length->data, (const int*)history_length->data,
                                    batch_size, kv_head_num, max_q_len, cs.S, head_size, host_layer_id(layer_id),
                                    cs.layers, launch_stream());
    throw_on_error(rc, "launchAppendKVCache");
}

// src/kernels/transpose_kernel.cu:45-88
void launchTransposeKVCache(Tensor* k_cache_src, Tensor* v_cache_src, Tensor* context_length, Tensor* layer_id,
                            Tensor* k_cache_dst, Tensor* v_cache_dst)
{
    ONELLM_CHECK_WITH_INFO(k_cache_src && v_cache_src && context_length && k_cache_dst && v_cache_dst, "null tensor");
    ONELLM_CHECK_WITH_INFO(k_cache_dst->shape.size() == 4, "k_cache_dst must be [B, Hq, max_k_len, D]");
    const int batch_size = context_length->shape[0];   // :53
    const CacheShape cs = cache_shape(k_cache_src, "launchTransposeKVCache");
    const int head_num = k_cache_dst->shape[1];        // :56
    const int max_k_len = k_cache_dst->shape[2];       // :58
    const int head_size = k_cache_dst->shape[3];       // :59
    ONELLM_CHECK_WITH_INFO(cs.B == batch_size && cs.D == head_size, "cache does not match destination");
    const int rc = onellm_kv_repeat(abi_dtype(k_cache_src, "launchTransposeKVCache"), k_cache_src->data,
                                    v_cache_src->data, k_cache_dst->data, v_cache_dst->data,
                                    (const int*)context_length->data, batch_size, head_num, cs.Hkv, cs.S, max_k_len,
                                    head_size, host_layer_id(layer_id), cs.layers, launch_stream());
    throw_on_error(rc, "launchTransposeKVCache");
}

// src/kernels/beamsearch_topK.cu:85-119: K = beamwidth = 2 and 8 blocks per row are fixed there
// (:89-90,105), which also fixes where the caller finds the results inside the workspace.
void launchTopKforBeamSearch(const float* probs, const int batch_size, const int vocab_size, float* topk_workspace)
{
    constexpr int beamwidth = 2;
    const int rc = onellm_beam_topk(probs, batch_size, beamwidth, vocab_size, beamwidth, topk_workspace, launch_stream());
    throw_on_error(rc, "launchTopKforBeamSearch");
}

// src/kernels/qkv_bias_and_RoPE.cu:167-207
void launchAddFusedQKVBiasTransposeAndRoPE(Tensor* q_buf, Tensor* k_buf, Tensor* v_buf, Tensor* QKV, BaseWeight& qkv,
                                           Tensor* padding_offset, Tensor* history_length, Tensor* input_length,
                                           LLaMAAttentionStaticParams& params)
{
    (void)input_length;   // the reference only forms an unused value from it (:139)
    ONELLM_CHECK_WITH_INFO(q_buf && k_buf && v_buf && QKV && padding_offset && history_length, "null tensor");
    ONELLM_CHECK_WITH_INFO(QKV->shape.size() == 3 && q_buf->shape.size() == 4, "QKV must be [tokens, heads, D], q_buf [B, Hq, S, D]");
    const int token_num = QKV->shape[0];               // :177
    const int qkv_head_num = QKV->shape[1];            // :178
    const int head_size = QKV->shape[2];               // :179
    const int batch_size = q_buf->shape[0];            // :180
    const int head_num = q_buf->shape[1];              // :181
    const int seq_len = q_buf->shape[2];               // :182
    const int kv_head_num = (qkv_head_num - head_num) / 2;   // :183
    const int rc = onellm_qkv_bias_rope_transpose(abi_dtype(QKV, "launchAddFusedQKVBiasTransposeAndRoPE"), q_buf->data,
                                                  k_buf->data, v_buf->data, QKV->data, qkv.bias,
                                                  (const int*)padding_offset->data, (const int*)history_length->data,
                                                  batch_size, seq_len, token_num, head_num, kv_head_num, head_size,
                                                  params.rotary_embedding_dim, params.rotary_embedding_base, launch_stream());
    throw_on_error(rc, "launchAddFusedQKVBiasTransposeAndRoPE");
}

// src/kernels/activation_kernel.cu:24-34
template <typename T>
void launchAct(const T* input, T* out, const int batch_size, const int intermedia_size)
{
    const int dtype = std::is_same<T, half>::value ? ONELLM_FP16 : ONELLM_FP32;
    throw_on_error(onellm_silu_and_mul(dtype, input, out, batch_size, intermedia_size, launch_stream()), "launchAct");
}
template void launchAct(const float*, float*, const int, const int);
template void launchAct(const half*, half*, const int, const int);

// src/kernels/topK_sampling.cu:43-70
void launchSampling(Tensor* topk_id, Tensor* topk_val, Tensor* seqlen, Tensor* is_finished, Tensor* output_id, IntDict& params)
{
    ONELLM_CHECK_WITH_INFO(topk_id && topk_val && seqlen && is_finished && output_id, "null tensor");
    ONELLM_CHECK_WITH_INFO(topk_id->shape.size() == 2, "topk_id must be [batch, K]");
    ONELLM_CHECK_WITH_INFO(params.count("vocab_size") && params.count("step") && params.count("end_id"),
                           "params need vocab_size, step and end_id");
    const int batch_size = topk_id->shape[0];          // :49
    const int K = topk_id->shape[1];                   // :50
    const int rc = onellm_topk_sample((const int*)topk_id->data, (const float*)topk_val->data, (int*)output_id->data,
                                      (int*)seqlen->data, (unsigned char*)is_finished->data, batch_size, K,
                                      (unsigned long long)(unsigned)params["step"], params["end_id"], params["vocab_size"],
                                      launch_stream());
    throw_on_error(rc, "launchSampling");
}
