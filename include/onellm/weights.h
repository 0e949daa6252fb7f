// Weight carriers of the decode path, with the member names, order and types the oneLLM layers fill
// in, so that code written against them compiles unchanged:
//   WeightType, getBitNum, getWeightType<T>, BaseWeight   <- src/weights/base_weights.h:5-49
//   LayerNormWeight                                         <- src/weights/llama/norm_weights.h:2-4
// A BaseWeight never owns `data` or `bias`; both are device pointers (bias may be null).
#pragma once
#include <cstdint>
#include <type_traits>
#include <vector>
#include <hip/hip_fp16.h>

enum class WeightType { FP32_W, FP16_W, INT8_W, UNSUPPORTED_W };

// storage bits of one weight element; 0 for an unsupported type
inline int getBitNum(WeightType type)
{
    return type == WeightType::FP32_W ? 32 : type == WeightType::FP16_W ? 16 : type == WeightType::INT8_W ? 8 : 0;
}

template<typename T>
inline WeightType getWeightType()
{
    using U = typename std::remove_const<T>::type;
    return std::is_same<U, float>::value    ? WeightType::FP32_W
           : std::is_same<U, half>::value   ? WeightType::FP16_W
           : std::is_same<U, int8_t>::value ? WeightType::INT8_W
                                            : WeightType::UNSUPPORTED_W;
}

// one projection: `data` is the matrix (used by the GEMMs, never by this backend), `bias` the fused
// bias vector the attention kernels read
struct BaseWeight {
    std::vector<int> shape;
    void*            data;
    WeightType       type;
    void*            bias;
};

// RMSNorm scale.  The field is `float*` in oneLLM; for FP16 activations the launcher reads fp16
// values behind the same pointer.
struct LayerNormWeight {
    float* gamma;
};

// Per-layer weight bundles as the decoder layers receive them:
//   LLaMAattentionWeights <- src/weights/llama/attention_weights.h:4-10
//   LLaMAFFNWeights       <- src/weights/llama/ffn_weights.h:4-8
//   LlamaLayerWeight      <- src/weights/llama/layer_weights.h:7-47
// Every matrix is row-major [in, out] (shape = {in, out}, src/weights/llama/layer_weights.cc:21-41), y = x . W.
struct LLaMAattentionWeights {
    BaseWeight q;
    BaseWeight k;
    BaseWeight v;
    BaseWeight qkv;      // [hidden, (Hq + 2 Hkv) * D], bias [(Hq + 2 Hkv) * D]
    BaseWeight output;   // [hidden, hidden], bias [hidden]
};

struct LLaMAFFNWeights {
    BaseWeight gate;     // [hidden, inter]
    BaseWeight up;       // [hidden, inter]
    BaseWeight down;     // [inter, hidden], bias [hidden] (may be null)
};

// A view: the constructor records the shapes, loadWeights() the device pointers; nothing is allocated or freed
// here (the reference allocates in the constructor, then overwrites those pointers in loadWeights and frees the
// caller's buffers in its destructor — src/weights/llama/layer_weights.cc:18-41,75-84,105-117).
struct LlamaLayerWeight {
    LlamaLayerWeight() = delete;
    LlamaLayerWeight(int head_num, int kv_head_num, int head_size, int inter_size, WeightType weight_type, bool attn_bias):
        attn_bias(attn_bias)
    {
        const int hidden_units = head_num * head_size;
        const int qkv_out = (head_num + 2 * kv_head_num) * head_size;
        attn_norm_weight.gamma = nullptr;
        ffn_norm_weight.gamma  = nullptr;
        self_attn_weight.qkv    = BaseWeight{{hidden_units, qkv_out}, nullptr, weight_type, nullptr};
        self_attn_weight.output = BaseWeight{{hidden_units, hidden_units}, nullptr, weight_type, nullptr};
        self_attn_weight.q = self_attn_weight.k = self_attn_weight.v = BaseWeight{{}, nullptr, weight_type, nullptr};
        ffn_weight.gate = BaseWeight{{hidden_units, inter_size}, nullptr, weight_type, nullptr};
        ffn_weight.up   = BaseWeight{{hidden_units, inter_size}, nullptr, weight_type, nullptr};
        ffn_weight.down = BaseWeight{{inter_size, hidden_units}, nullptr, weight_type, nullptr};
    }

    // argument order of src/weights/llama/layer_weights.h:32-41
    template<typename T>
    void loadWeights(T* d_attn_norm_weight, T* d_ffn_norm_weight, T* d_qkv_weights, T* d_qkv_bias, T* d_output_weights,
                     T* d_out_bias, T* d_ffn_down, T* d_ffn_down_bias, T* d_ffn_gate, T* d_ffn_up)
    {
        attn_norm_weight.gamma       = (float*)d_attn_norm_weight;
        ffn_norm_weight.gamma        = (float*)d_ffn_norm_weight;
        self_attn_weight.qkv.data    = d_qkv_weights;
        self_attn_weight.qkv.bias    = attn_bias ? (void*)d_qkv_bias : nullptr;
        self_attn_weight.output.data = d_output_weights;
        self_attn_weight.output.bias = attn_bias ? (void*)d_out_bias : nullptr;
        ffn_weight.down.data         = d_ffn_down;
        ffn_weight.down.bias         = d_ffn_down_bias;
        ffn_weight.gate.data         = d_ffn_gate;
        ffn_weight.up.data           = d_ffn_up;
    }

    LayerNormWeight       attn_norm_weight;
    LayerNormWeight       ffn_norm_weight;
    LLaMAattentionWeights self_attn_weight;
    LLaMAFFNWeights       ffn_weight;

private:
    bool attn_bias;
};
