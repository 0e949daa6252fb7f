// Test harness for the launcher shims: builds oneLLM-style Tensor / BaseWeight / LayerNormWeight
// objects around raw pointers handed in from Python and calls the six launch* functions exactly as
// the oneLLM layers and unit tests do.  C++ exceptions are turned into return code 1 + a message.
#include <cstring>
#include <exception>
#include <string>
#include "onellm/kernels.h"
#include "onellm/tensor_map.h"
#include "counter_sets.hpp"

namespace {
std::string g_last_error;

template <typename F>
int guarded(F&& f)
{
    try {
        f();
        g_last_error.clear();
        return 0;
    } catch (const std::exception& e) {
        g_last_error = e.what();
        return 1;
    }
}

DataType dt(int dtype) { return dtype == 1 ? FP16 : (dtype == 0 ? FP32 : INT8); }

Tensor cache_tensor(int dtype, void* p, int L, int B, int Hkv, int S, int D)
{
    if (L <= 0) return Tensor(GPU, dt(dtype), {B, Hkv, S, D}, p);        // 4-D, as the kernel unit tests build it
    return Tensor(GPU, dt(dtype), {L, B, Hkv, S, D}, p);                 // 5-D, as the layers allocate it
}
}  // namespace

extern "C" {

const char* h_last_error() { return g_last_error.c_str(); }

int h_decode_mha(int dtype, void* qkv, void* bias, void* kc, void* vc, void* out, int B, int Hq, int Hkv, int D, int S,
                 int L, int step_value, int step_on_gpu, int rotary_dim, float base)
{
    return guarded([&] {
        Tensor qkv_buf(GPU, dt(dtype), {B, Hq + 2 * Hkv, D}, qkv);
        BaseWeight w;
        w.data = nullptr;
        w.type = dtype == 1 ? WeightType::FP16_W : WeightType::FP32_W;
        w.bias = bias;
        Tensor k_cache = cache_tensor(dtype, kc, L, B, Hkv, S, D);
        Tensor v_cache = cache_tensor(dtype, vc, L, B, Hkv, S, D);
        bool fin = false;
        Tensor finished(GPU, BOOL, {B}, &fin);
        int h_step = step_value;
        Tensor step(step_on_gpu ? GPU : CPU, INT32, {1}, &h_step);
        Tensor mha_output(GPU, dt(dtype), {B, Hq * D}, out);
        LLaMAAttentionStaticParams params;
        params.rotary_embedding_dim = rotary_dim;
        params.rotary_embedding_base = base;
        params.max_position_embeddings = 2048;
        params.use_dynamic_ntk = false;
        launchDecoderMaskedMHA(&qkv_buf, w, &k_cache, &v_cache, &finished, &step, &mha_output, params);
    });
}

int h_rmsnorm(int dtype, void* x, void* gamma, int N, int H, float eps)
{
    return guarded([&] {
        Tensor t(GPU, dt(dtype), {N, H}, x);
        LayerNormWeight w;
        w.gamma = (float*)gamma;
        launchRMSNorm(&t, w, eps);
    });
}

int h_fused_norm(int dtype, void* residual, void* out, void* bias, void* gamma, int N, int H, float eps)
{
    return guarded([&] {
        if (dtype == 1)
            launchFusedAddBiasResidualRMSNorm<half>((half*)residual, (half*)out, (const half*)bias, (const half*)gamma, eps, N, H);
        else
            launchFusedAddBiasResidualRMSNorm<float>((float*)residual, (float*)out, (const float*)bias, (const float*)gamma, eps, N, H);
    });
}

int h_append(int dtype, void* ks, void* vs, void* kc, void* vc, void* cur, void* hist, int B, int Hkv, int Q, int S, int D,
             int L, int host_layer_id)
{
    return guarded([&] {
        Tensor k_src(GPU, dt(dtype), {B, Hkv, Q, D}, ks), v_src(GPU, dt(dtype), {B, Hkv, Q, D}, vs);
        Tensor k_dst = cache_tensor(dtype, kc, L, B, Hkv, S, D), v_dst = cache_tensor(dtype, vc, L, B, Hkv, S, D);
        Tensor cur_len(GPU, INT32, {B}, cur), history(GPU, INT32, {B}, hist);
        int lid = host_layer_id;
        Tensor layer_id(CPU, INT32, {1}, &lid);
        launchAppendKVCache(&k_src, &v_src, host_layer_id >= 0 ? &layer_id : nullptr, &cur_len, &history, &k_dst, &v_dst);
    });
}

int h_repeat(int dtype, void* kc, void* vc, void* kd, void* vd, void* ctx, int B, int Hq, int Hkv, int S, int MK, int D, int L,
             int host_layer_id)
{
    return guarded([&] {
        Tensor k_src = cache_tensor(dtype, kc, L, B, Hkv, S, D), v_src = cache_tensor(dtype, vc, L, B, Hkv, S, D);
        Tensor k_dst(GPU, dt(dtype), {B, Hq, MK, D}, kd), v_dst(GPU, dt(dtype), {B, Hq, MK, D}, vd);
        Tensor ctx_len(GPU, INT32, {B}, ctx);
        int lid = host_layer_id;
        Tensor layer_id(CPU, INT32, {1}, &lid);
        launchTransposeKVCache(&k_src, &v_src, &ctx_len, host_layer_id >= 0 ? &layer_id : nullptr, &k_dst, &v_dst);
    });
}

int h_topk(const float* probs, int B, int V, float* ws)
{
    return guarded([&] { launchTopKforBeamSearch(probs, B, V, ws); });
}

int h_prefill_rope(int dtype, void* q, void* k, void* v, void* qkv, void* bias, void* padding_offset, void* history, void* input_len,
                   int B, int S, int tokens, int Hq, int Hkv, int D, int rotary_dim, float base)
{
    return guarded([&] {
        Tensor q_buf(GPU, dt(dtype), {B, Hq, S, D}, q), k_buf(GPU, dt(dtype), {B, Hkv, S, D}, k), v_buf(GPU, dt(dtype), {B, Hkv, S, D}, v);
        Tensor QKV(GPU, dt(dtype), {tokens, Hq + 2 * Hkv, D}, qkv);
        BaseWeight w;
        w.data = nullptr;
        w.type = dtype == 1 ? WeightType::FP16_W : WeightType::FP32_W;
        w.bias = bias;
        Tensor po(GPU, INT32, {B, S}, padding_offset), hist(GPU, INT32, {B}, history), in_len(GPU, INT32, {B}, input_len);
        LLaMAAttentionStaticParams params{rotary_dim, base, 2048, false};
        launchAddFusedQKVBiasTransposeAndRoPE(&q_buf, &k_buf, &v_buf, &QKV, w, &po, &hist, &in_len, params);
    });
}

int h_act(int dtype, const void* input, void* out, int B, int I)
{
    return guarded([&] {
        if (dtype == 1) launchAct<half>((const half*)input, (half*)out, B, I);
        else launchAct<float>((const float*)input, (float*)out, B, I);
    });
}

int h_sampling(void* topk_id, void* topk_val, void* seqlen, void* finished, void* out, int B, int K, int step, int end_id, int vocab)
{
    return guarded([&] {
        Tensor id(GPU, INT32, {B, K}, topk_id), val(GPU, FP32, {B, K}, topk_val), sl(GPU, INT32, {B}, seqlen);
        Tensor fin(GPU, BOOL, {B}, finished), o(GPU, INT32, {B}, out);
        IntDict params;
        params.insert({"step", step});
        params.insert({"vocab_size", vocab});
        params.insert({"end_id", end_id});
        launchSampling(&id, &val, &sl, &fin, &o, params);
    });
}

// the callers' pattern after every launch (src/layers/attention/masked_self_attention.cpp:73 in oneLLM)
// onellmSetLaunchStream for the calling thread (NULL restores the null stream)
void h_set_launch_stream(void* stream) { onellmSetLaunchStream(static_cast<hipStream_t>(stream)); }

int h_sync_and_check()
{
    return guarded([] { DeviceSyncAndCheckCudaError(); });
}

// host-only behaviour of the carrier types
int h_getval_requires_cpu_tensor()
{
    int v = 7;
    Tensor on_cpu(CPU, INT32, {1}, &v), on_gpu(GPU, INT32, {1}, &v);
    if (on_cpu.getVal<int>() != 7) return 2;
    return guarded([&] { (void)on_gpu.getVal<int>(); });   // must throw -> 1
}

int h_tensor_size(int a, int b, int c)
{
    int dummy;
    Tensor t(CPU, FP32, {a, b, c}, &dummy);
    Tensor empty(CPU, FP32, {a, b, c});
    return empty.size() == 0 ? t.size() : -1;
}

int h_type_tags()
{
    return (getTensorType<float>() == FP32) + 2 * (getTensorType<half>() == FP16) + 4 * (getTensorType<int>() == INT32)
           + 8 * (getTensorType<const float>() == FP32) + 16 * (getWeightType<half>() == WeightType::FP16_W)
           + 32 * (getBitNum(WeightType::INT8_W) == 8);
}

// Tensor == Tensor (src/utils/tensor.h:146-160) and CHECK_CUBLAS (src/utils/macro.h:59-70): a bit per check that holds
int h_equality_and_status_checks()
{
    float a[4] = {1.f, 2.f, 3.f, 4.f}, b[4] = {1.f, 2.f, 3.f, 4.f}, c[4] = {1.f, 2.f, 3.f, 5.f}, d[2] = {1.f, 2.f};
    Tensor ta(CPU, FP32, {2, 2}, a), tb(CPU, FP32, {4}, b), tc(CPU, FP32, {2, 2}, c), td(CPU, FP32, {2}, d), empty(CPU, FP32, {2, 2});
    int ok = 0;
    ok |= (ta == tb) << 0;                        // same count, same values (shapes are not compared, as in the reference)
    ok |= (!(ta == tc)) << 1;
    ok |= (!(ta == td)) << 2;
    ok |= (!(ta == empty)) << 3;
    const int fine = guarded([] { CHECK_CUBLAS(0); });
    const int threw = guarded([] { CHECK_CUBLAS(3); });
    ok |= (fine == 0 && threw == 1 && g_last_error.find("[TM][ERROR]") != std::string::npos) << 4;
    return ok;
}

// TensorMap as the layers use it (src/utils/tensor.h:160-296): returns a bit per check that holds
int h_tensor_map_checks()
{
    int v = 5, w = 9;
    Tensor good(CPU, INT32, {1}, &v), other(CPU, INT32, {1}, &w), no_data(CPU, INT32, {1}), no_shape(CPU, INT32, {}, &v);
    TensorMap m{{"step", good}, {"dropped_a", no_data}, {"dropped_b", no_shape}};
    int ok = 0;
    ok |= (m.size() == 1) << 0;                                  // tensors without data or shape are not inserted
    ok |= (m.isExist("step") && !m.isExist("dropped_a")) << 1;
    ok |= (m["step"].getVal<int>() == 5 && m.getVal<int>("step") == 5) << 2;
    m.insert("other", other);
    m["step"] = other;                                           // entries are assignable views
    ok |= (m.size() == 2 && m.at("step").getVal<int>() == 9 && m.getPtr<int>("other") == &w) << 3;
    const int threw = guarded([&] { (void)m["missing"]; });
    ok |= (threw == 1 && g_last_error.find("missing") != std::string::npos && g_last_error.find("other") != std::string::npos) << 4;
    ok |= (m.keys().size() == 2) << 5;
    return ok;
}

// LlamaLayerWeight records the shapes of src/weights/llama/layer_weights.cc:21-41 and only views the pointers
int h_layer_weight_checks(int head_num, int kv_head_num, int head_size, int inter_size, int attn_bias)
{
    LlamaLayerWeight lw(head_num, kv_head_num, head_size, inter_size, WeightType::FP16_W, attn_bias != 0);
    const int hidden = head_num * head_size;
    float buf[10];
    lw.loadWeights<float>(buf + 0, buf + 1, buf + 2, buf + 3, buf + 4, buf + 5, buf + 6, buf + 7, buf + 8, buf + 9);
    int ok = 0;
    ok |= (lw.self_attn_weight.qkv.shape == std::vector<int>{hidden, (head_num + 2 * kv_head_num) * head_size}) << 0;
    ok |= (lw.self_attn_weight.output.shape == std::vector<int>{hidden, hidden}) << 1;
    ok |= (lw.ffn_weight.gate.shape == std::vector<int>{hidden, inter_size} && lw.ffn_weight.up.shape == lw.ffn_weight.gate.shape) << 2;
    ok |= (lw.ffn_weight.down.shape == std::vector<int>{inter_size, hidden}) << 3;
    ok |= (lw.attn_norm_weight.gamma == buf + 0 && lw.ffn_norm_weight.gamma == buf + 1 && lw.self_attn_weight.qkv.data == buf + 2
           && lw.self_attn_weight.output.data == buf + 4 && lw.ffn_weight.down.data == buf + 6 && lw.ffn_weight.down.bias == buf + 7
           && lw.ffn_weight.gate.data == buf + 8 && lw.ffn_weight.up.data == buf + 9) << 4;
    const bool biases = lw.self_attn_weight.qkv.bias == buf + 3 && lw.self_attn_weight.output.bias == buf + 5;
    const bool none = lw.self_attn_weight.qkv.bias == nullptr && lw.self_attn_weight.output.bias == nullptr;
    ok |= (attn_bias ? biases : none) << 5;
    ok |= (lw.self_attn_weight.qkv.type == WeightType::FP16_W && lw.ffn_weight.down.type == WeightType::FP16_W) << 6;
    return ok;
}

// ---- the table of arrival-counter sets (csrc/counter_sets.hpp): plain host logic, driven from Python
void* h_counter_table_new(int sets_per_device, int listed) { return new onellm::CounterSets("test table", sets_per_device, listed != 0); }
void h_counter_table_delete(void* t) { delete static_cast<onellm::CounterSets*>(t); }
int h_counter_table_acquire(void* t, int device, void* workspace, int capturing)
{
    return static_cast<onellm::CounterSets*>(t)->acquire(device, workspace, capturing != 0);
}
int h_counter_table_release(void* t, void* workspace) { return static_cast<onellm::CounterSets*>(t)->release(workspace); }
void h_counter_table_stats(void* t, int device, int* owned, int* captured, long* fallbacks)
{
    const onellm::CounterSets::Stats s = static_cast<onellm::CounterSets*>(t)->stats(device);
    *owned = s.owned;
    *captured = s.captured;
    *fallbacks = s.fallbacks;
}

}  // extern "C"
