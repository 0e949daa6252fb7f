// A stand-alone C++ driver of one decode step, written against include/onellm/layers.h the way a oneLLM user writes
// one against src/layers/decoder/self_decoder.h: same shapes and constants as
// examples/cpp/decoder/self_decoder_example.cpp:10-27,40-140 (step 3, 4 query / 2 kv heads of size 8, inter size 12,
// 2 layers, cache of 12 rows, batch 2; inputs and caches 1, norm scales 1 / 2, projection weights 1 / 2, biases 2 / 0),
// same TensorMap keys, same constructor and forward() calls.  Prints decoder_output, the residual stream and the
// appended K rows so that a test can compare them with the CPU oracle on the same constants.
#include <cstdio>
#include <vector>
#include <hip/hip_runtime.h>
#include "onellm/layers.h"

namespace {
std::vector<void*> g_owned;

float* device_filled(size_t n, float value)
{
    std::vector<float> h(n, value);
    float* d = nullptr;
    CHECK(hipMalloc((void**)&d, n * sizeof(float)));
    CHECK(hipMemcpy(d, h.data(), n * sizeof(float), hipMemcpyHostToDevice));
    g_owned.push_back(d);
    return d;
}
void print_row(const char* name, const float* d, size_t n)
{
    std::vector<float> h(n);
    CHECK(hipMemcpy(h.data(), d, n * sizeof(float), hipMemcpyDeviceToHost));
    std::printf("%s", name);
    for (float v : h) std::printf(" %.9g", v);
    std::printf("\n");
}
}  // namespace

int main()
{
    int h_step = 3;
    const int head_num = 4, kv_head_num = 2, head_size = 8, inter_size = 12, num_layers = 2, max_seq_len = 12;
    const int qkv_units = (head_num + 2 * kv_head_num) * head_size, hidden = head_num * head_size;
    const float rmsnorm_eps = 1e-16f;
    LLaMAAttentionStaticParams attn_static_params{128, 10000.f, 2048, false};
    LLaMAAttentionDynParams attn_dyn_params{};
    attn_dyn_params.batch_size = 2;
    const int B = attn_dyn_params.batch_size;
    HipAllocator allocator;

    float* d_decoder_input = device_filled((size_t)B * hidden, 1.f);
    float* d_decoder_output = device_filled((size_t)B * hidden, 0.f);
    const size_t cache_elems = (size_t)num_layers * B * kv_head_num * max_seq_len * head_size;
    float* d_all_k_cache = device_filled(cache_elems, 1.f);
    float* d_all_v_cache = device_filled(cache_elems, 1.f);
    bool* d_finished = nullptr;
    CHECK(hipMalloc((void**)&d_finished, B * sizeof(bool)));
    CHECK(hipMemset(d_finished, 0, B * sizeof(bool)));
    g_owned.push_back(d_finished);

    float* d_output_norm_weight = device_filled(hidden, 2.f);
    float* d_attn_norm_weight = device_filled(hidden, 1.f);
    float* d_ffn_norm_weight = device_filled(hidden, 1.f);
    float* d_qkv_weights = device_filled((size_t)hidden * qkv_units, 1.f);
    float* d_qkv_bias = device_filled(qkv_units, 2.f);
    float* d_output_weights = device_filled((size_t)hidden * hidden, 1.f);
    float* d_out_bias = device_filled(hidden, 2.f);
    float* d_ffn_gate = device_filled((size_t)hidden * inter_size, 2.f);
    float* d_ffn_up = device_filled((size_t)hidden * inter_size, 1.f);
    float* d_ffn_down = device_filled((size_t)hidden * inter_size, 2.f);
    float* d_ffn_down_bias = device_filled(hidden, 0.f);

    const DataType type = getTensorType<float>(), type_int = getTensorType<int>(), type_bool = getTensorType<bool>();
    std::vector<LlamaLayerWeight*> layerWeights;
    for (int i = 0; i < num_layers; i++) {
        layerWeights.push_back(new LlamaLayerWeight(head_num, kv_head_num, head_size, inter_size, getWeightType<float>(),
                                                    /*attn_bias=*/true));
        layerWeights.back()->loadWeights<float>(d_attn_norm_weight, d_ffn_norm_weight, d_qkv_weights, d_qkv_bias,
                                                d_output_weights, d_out_bias, d_ffn_down, d_ffn_down_bias, d_ffn_gate, d_ffn_up);
    }

    TensorMap decoder_inputs{
        {"decoder_input", Tensor(GPU, type, {B, hidden}, d_decoder_input)},
        {"step", Tensor(CPU, type_int, {1}, &h_step)},
        {"finished", Tensor(GPU, type_bool, {B}, d_finished)},
        {"output_norm_weight", Tensor(GPU, type, {hidden}, d_output_norm_weight)}};
    TensorMap decoder_outputs{
        {"decoder_output", Tensor(GPU, type, {B, hidden}, d_decoder_output)},
        {"all_k_cache", Tensor(GPU, type, {num_layers, B, kv_head_num, max_seq_len, head_size}, d_all_k_cache)},
        {"all_v_cache", Tensor(GPU, type, {num_layers, B, kv_head_num, max_seq_len, head_size}, d_all_v_cache)}};

    LlamaSelfDecoder* selfDecoder = new LlamaSelfDecoder(head_num, kv_head_num, head_size, inter_size, num_layers,
                                                         attn_static_params, rmsnorm_eps, /*stream=*/nullptr,
                                                         /*cublas_wrapper=*/nullptr, &allocator,
                                                         /*is_free_buffer_after_forward=*/true);
    selfDecoder->forward(decoder_inputs, layerWeights, decoder_outputs, attn_dyn_params);
    DeviceSyncAndCheckCudaError();

    print_row("decoder_output", d_decoder_output, (size_t)B * hidden);
    print_row("residual", d_decoder_input, (size_t)B * hidden);
    for (int l = 0; l < num_layers; l++) {
        const size_t row = (((size_t)l * B + 0) * kv_head_num + 0) * max_seq_len + (h_step - 1);
        print_row("k_row", d_all_k_cache + row * head_size, head_size);
        print_row("v_row", d_all_v_cache + row * head_size, head_size);
    }

    delete selfDecoder;
    for (LlamaLayerWeight* w : layerWeights) delete w;
    for (void* p : g_owned) CHECK(hipFree(p));
    return 0;
}
