// C surface over LlamaSelfDecoder / launchLinearGemm (declared in onellm_layers.h) for callers that cannot build
// C++ objects: it assembles the Tensor, TensorMap and LlamaLayerWeight objects the way
// examples/cpp/decoder/self_decoder_example.cpp does, from raw device pointers.  C++ exceptions become return code 1 +
// a message.
#include <exception>
#include <memory>
#include <string>
#include <vector>
#include "onellm/layers.h"
#include "onellm_layers.h"

namespace {
thread_local std::string g_last_error;

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
DataType dt(int dtype) { return dtype == 1 ? FP16 : FP32; }
WeightType wt(int dtype) { return dtype == 1 ? WeightType::FP16_W : WeightType::FP32_W; }

struct Decoder {
    int dtype, B, Hq, Hkv, D, I, L, S;
    HipAllocator allocator;
    std::vector<std::unique_ptr<LlamaLayerWeight>> weights;
    std::vector<LlamaLayerWeight*> weight_ptrs;
    std::unique_ptr<LlamaSelfDecoder> decoder;
    void* output_norm = nullptr;
};
}  // namespace

extern "C" {

const char* onellm_layers_last_error() { return g_last_error.c_str(); }

// pair: y is the {2, M, N} gate/up buffer; second: write its second slot (shared_out_buf)
int onellm_layers_linear(int dtype, void* x, void* w, void* y, int M, int K, int N, int trans_b, int pair, int second)
{
    return guarded([&] {
        Tensor in(GPU, dt(dtype), {M, K}, x);
        BaseWeight weight;
        weight.shape = trans_b ? std::vector<int>{N, K} : std::vector<int>{K, N};
        weight.data = w;
        weight.type = wt(dtype);
        weight.bias = nullptr;
        Tensor out = pair ? Tensor(GPU, dt(dtype), {2, M, N}, y) : Tensor(GPU, dt(dtype), {M, N}, y);
        launchLinearGemm(&in, weight, &out, false, trans_b != 0, second != 0);
    });
}

int onellm_layers_allow_plain_gemm(int allow)
{
    setLinearGemmPlainFallback(allow != 0);
    return 0;
}

int onellm_layers_gemm_workspace_count(void) { return (int)linearGemmWorkspaceCount(); }

int onellm_layers_release_gemm_workspace(onellm_stream_t stream)
{
    int had = 0;
    const int rc = guarded([&] { had = releaseLinearGemmWorkspace(static_cast<hipStream_t>(stream)) ? 1 : 0; });
    return rc == 0 ? had : -1;
}

// per-layer pointer arrays of length L, in the argument order of LlamaLayerWeight::loadWeights
void* onellm_decoder_create(int dtype, int B, int Hq, int Hkv, int D, int I, int L, int S, int rotary_dim, float rope_base,
                        float eps, int attn_bias, void** attn_norm, void** ffn_norm, void** wqkv, void** bqkv, void** wo,
                        void** bo, void** wdown, void** bdown, void** wgate, void** wup, void* output_norm,
                        onellm_stream_t stream)
{
    Decoder* d = nullptr;
    const int rc = guarded([&] {
        d = new Decoder{dtype, B, Hq, Hkv, D, I, L, S};
        for (int l = 0; l < L; ++l) {
            d->weights.emplace_back(new LlamaLayerWeight(Hq, Hkv, D, I, wt(dtype), attn_bias != 0));
            d->weights.back()->loadWeights<void>(attn_norm[l], ffn_norm[l], wqkv[l], bqkv[l], wo[l], bo[l], wdown[l], bdown[l],
                                                 wgate[l], wup[l]);
            d->weight_ptrs.push_back(d->weights.back().get());
        }
        d->output_norm = output_norm;
        LLaMAAttentionStaticParams sp;
        sp.rotary_embedding_dim = rotary_dim;
        sp.rotary_embedding_base = rope_base;
        sp.max_position_embeddings = 2048;
        sp.use_dynamic_ntk = false;
        d->decoder.reset(new LlamaSelfDecoder(Hq, Hkv, D, I, L, sp, eps, static_cast<hipStream_t>(stream), nullptr, &d->allocator,
                                              /*is_free_buffer_after_forward=*/false));
    });
    if (rc != 0) {
        delete d;
        return nullptr;
    }
    return d;
}

int onellm_decoder_forward(void* handle, int step_value, void* decoder_input, void* decoder_output, void* k_cache, void* v_cache)
{
    return guarded([&] {
        Decoder* d = static_cast<Decoder*>(handle);
        const int hidden = d->Hq * d->D;
        int h_step = step_value;
        bool fin = false;
        LLaMAAttentionDynParams dyn{};
        dyn.batch_size = d->B;
        dyn.num_layers = d->L;
        TensorMap inputs{{"decoder_input", Tensor(GPU, dt(d->dtype), {d->B, hidden}, decoder_input)},
                         {"step", Tensor(CPU, getTensorType<int>(), {1}, &h_step)},
                         {"finished", Tensor(GPU, getTensorType<bool>(), {d->B}, &fin)},
                         {"output_norm_weight", Tensor(GPU, dt(d->dtype), {hidden}, d->output_norm)}};
        TensorMap outputs{{"decoder_output", Tensor(GPU, dt(d->dtype), {d->B, hidden}, decoder_output)},
                          {"all_k_cache", Tensor(GPU, dt(d->dtype), {d->L, d->B, d->Hkv, d->S, d->D}, k_cache)},
                          {"all_v_cache", Tensor(GPU, dt(d->dtype), {d->L, d->B, d->Hkv, d->S, d->D}, v_cache)}};
        d->decoder->forward(inputs, d->weight_ptrs, outputs, dyn);
    });
}

void onellm_decoder_destroy(void* handle) { delete static_cast<Decoder*>(handle); }

}  // extern "C"
