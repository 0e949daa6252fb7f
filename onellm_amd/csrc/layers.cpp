// Decode-side layers of oneLLM over this backend (declared in onellm/layers.h): they sequence the launch*
// functions and the projection GEMMs for one decode step and own no arithmetic of their own.
#include <map>
#include <mutex>
#include <set>
#include <tuple>
#include <utility>
#include <stdexcept>
#include <string>
#include <hip/hip_runtime_api.h>
#include "onellm/layers.h"
#include "onellm_gemm.h"

namespace {

void require(bool ok, const std::string& what)
{
    if (!ok) throw std::runtime_error("[oneLLM][ERROR] " + what + " \n");
}
void hip_ok(hipError_t e, const char* what)
{
    if (e != hipSuccess) throw std::runtime_error(std::string("[TM][ERROR] ") + what + ": " + hipGetErrorString(e) + " \n");
}
size_t elt_bytes(DataType t)
{
    require(t == FP32 || t == FP16, "the decode layers run FP32 or FP16 tensors");
    return t == FP32 ? 4 : 2;
}
int rows_of(const Tensor* t) { return t->shape.empty() ? 0 : t->shape[0]; }
int cols_of(const Tensor* t)
{
    int n = 1;
    for (size_t i = 1; i < t->shape.size(); ++i) n *= t->shape[i];
    return n;
}

bool stream_is_capturing(hipStream_t stream)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return status != hipStreamCaptureStatusNone;
}

// Scratch for the GEMM library's split-K algorithms: one buffer per (device, launch stream), created on first use
// there - steps queued on different streams of one GPU (two decoders, two threads) must not share split-K
// partials.  Creating one allocates, so a stream that is being captured is refused.
struct GemmWorkspace {
    struct Buffer {
        void* ptr = nullptr;
        size_t bytes = 0;
    };
    std::mutex mu;
    std::map<std::pair<int, hipStream_t>, Buffer> buffers;
    Buffer get(hipStream_t stream)
    {
        int device = 0;
        hip_ok(hipGetDevice(&device), "gemm workspace device");
        std::lock_guard<std::mutex> g(mu);
        const auto key = std::make_pair(device, stream);
        auto it = buffers.find(key);
        if (it != buffers.end()) return it->second;
        require(!stream_is_capturing(stream), "launchLinearGemm: the first call on a stream creates its GEMM workspace, which "
                                              "cannot be done while the stream is being captured; run one ordinary step first");
        Buffer b;
        const size_t want = onellm_linear_workspace_bytes();
        if (hipMalloc(&b.ptr, want) == hipSuccess) b.bytes = want;
        else { b.ptr = nullptr; (void)hipGetLastError(); }      // the library then keeps to algorithms that need none
        buffers[key] = b;
        return b;
    }
    bool drop(hipStream_t stream)
    {
        int device = 0;
        hip_ok(hipGetDevice(&device), "gemm workspace device");
        Buffer b;
        {
            std::lock_guard<std::mutex> g(mu);
            auto it = buffers.find(std::make_pair(device, stream));
            if (it == buffers.end()) return false;
            b = it->second;
            buffers.erase(it);
        }
        if (b.ptr) {
            hip_ok(hipStreamSynchronize(stream), "gemm workspace sync");
            (void)onellm_release_workspace(b.ptr);
            hip_ok(hipFree(b.ptr), "gemm workspace free");
        }
        return true;
    }
    size_t count()
    {
        std::lock_guard<std::mutex> g(mu);
        return buffers.size();
    }
};
GemmWorkspace g_gemm_ws;

// The first time a projection shape is seen, the library's candidate algorithms are timed once and the fastest is
// kept (the first suggestion is up to 1.7x slower on the skinny decode shapes).  That one call synchronises the
// stream; setLinearGemmAutotune(false) keeps every call asynchronous.
std::mutex g_tuned_mu;
std::set<std::tuple<int, int, int, int, int, int>> g_tuned;
bool g_autotune = true;

void tune_once(int dtype, int M, int K, int N, int ldy, int w_is_nk, void* ws, size_t ws_bytes)
{
    {
        std::lock_guard<std::mutex> g(g_tuned_mu);
        if (!g_autotune || g_tuned.count(std::make_tuple(dtype, M, K, N, ldy, w_is_nk))) return;
        // a shape first seen under capture is not timed now (that would allocate and synchronise) and stays
        // unmarked, so that the next ordinary call tunes it; the captured call uses the library's first suggestion
        if (stream_is_capturing(onellmGetLaunchStream())) return;
        g_tuned.insert(std::make_tuple(dtype, M, K, N, ldy, w_is_nk));
    }
    (void)onellm_linear_tune(dtype, M, K, N, ldy, w_is_nk, ws, ws_bytes, onellmGetLaunchStream(), nullptr, nullptr);   // best effort
}

// the same for the one-launch forms of a pair of projections (the key's last element tells the two tables apart)
void tune_pair_once(int dtype, int M, int K, int N, int ldy, int w_is_nk, void* ws, size_t ws_bytes)
{
    {
        std::lock_guard<std::mutex> g(g_tuned_mu);
        const auto key = std::make_tuple(dtype, M, K, N, ldy, w_is_nk + 2);
        if (!g_autotune || g_tuned.count(key)) return;
        if (stream_is_capturing(onellmGetLaunchStream())) return;
        g_tuned.insert(key);
        g_tuned.insert(std::make_tuple(dtype, M, K, N, ldy, w_is_nk));    // (the pair's tuning run covers the single projection)
    }
    (void)onellm_linear_pair_tune(dtype, M, K, N, ldy, w_is_nk, ws, ws_bytes, onellmGetLaunchStream(), nullptr, nullptr);   // best effort
}

Tensor* new_buffer(BaseAllocator* a, DataType t, std::vector<int> shape)
{
    size_t n = elt_bytes(t);
    for (int d : shape) n *= (size_t)d;
    Tensor* buf = new Tensor(Device::GPU, t, std::move(shape));
    buf->data = a->Malloc(buf->data, n, false);
    return buf;
}
void drop_buffer(BaseAllocator* a, Tensor*& buf)
{
    if (!buf) return;
    a->deviceFree(buf->data);
    delete buf;
    buf = nullptr;
}

}  // namespace

void setLinearGemmAutotune(bool on)
{
    std::lock_guard<std::mutex> g(g_tuned_mu);
    g_autotune = on;
}

void setLinearGemmPlainFallback(bool allow) { (void)onellm_linear_allow_plain(allow ? 1 : 0); }

size_t linearGemmWorkspaceCount() { return g_gemm_ws.count(); }

bool releaseLinearGemmWorkspace(hipStream_t stream) { return g_gemm_ws.drop(stream); }

// src/kernels/qkv_linear.cu:8-66
void launchLinearGemm(Tensor* input, BaseWeight& weight, Tensor* output, bool trans_a, bool trans_b, bool shared_out_buf)
{
    require(input && output && input->data && output->data && weight.data, "launchLinearGemm: null tensor or weight");
    require(!trans_a, "launchLinearGemm: a transposed input is not supported");
    require(input->dtype == output->dtype, "launchLinearGemm: input and output element types differ");
    require(weight.shape.size() == 2, "launchLinearGemm: weight must be a matrix");
    const size_t e = elt_bytes(input->dtype);
    const WeightType want = input->dtype == FP32 ? WeightType::FP32_W : WeightType::FP16_W;
    require(weight.type == want, "launchLinearGemm: weight element type does not match the activations");
    const int M = rows_of(input), K = cols_of(input);
    const int wk = trans_b ? weight.shape[1] : weight.shape[0];
    const int N = trans_b ? weight.shape[0] : weight.shape[1];
    require(wk == K, "launchLinearGemm: inner sizes differ (" + std::to_string(K) + " vs " + std::to_string(wk) + ")");
    // a {2, M, N} output is the gate/up pair buffer of the SwiGLU kernel, rows interleaved as [M, 2, N]
    // (told apart from an ordinary [M, a, b] output by its shape: there N = a * b, here N = b)
    const bool pair = output->shape.size() == 3 && output->shape[0] == 2 && output->shape[1] == M && output->shape[2] == N;
    int ldy = N;
    char* y = static_cast<char*>(output->data);
    if (pair) {
        ldy = 2 * N;
        if (shared_out_buf) y += (size_t)N * e;
    } else {
        require(!shared_out_buf, "launchLinearGemm: shared_out_buf needs a {2, M, N} output");
        require(rows_of(output) == M && cols_of(output) == N, "launchLinearGemm: output shape");
    }
    const GemmWorkspace::Buffer ws = g_gemm_ws.get(onellmGetLaunchStream());
    const int dtype_code = input->dtype == FP32 ? ONELLM_FP32 : ONELLM_FP16;
    tune_once(dtype_code, M, K, N, ldy, trans_b ? 1 : 0, ws.ptr, ws.bytes);
    const int rc = onellm_linear(dtype_code, input->data, weight.data, y, M, K, N, ldy, trans_b ? 1 : 0, ws.ptr, ws.bytes,
                                 onellmGetLaunchStream());
    if (rc != 0) throw std::runtime_error(std::string("[TM][ERROR] launchLinearGemm: ") + onellm_error_string(rc) + " \n");
}

// the two launchLinearGemm calls of src/layers/ffn/ffn.cpp:61-62 (gate, then up with shared_out_buf) as one
void launchLinearGemmPair(Tensor* input, BaseWeight& first, BaseWeight& second, Tensor* output)
{
    require(input && output && input->data && output->data && first.data && second.data, "launchLinearGemmPair: null tensor or weight");
    require(input->dtype == output->dtype, "launchLinearGemmPair: input and output element types differ");
    require(first.shape.size() == 2 && second.shape == first.shape, "launchLinearGemmPair: the weights must be two matrices of one shape");
    const size_t e = elt_bytes(input->dtype);
    const WeightType want = input->dtype == FP32 ? WeightType::FP32_W : WeightType::FP16_W;
    require(first.type == want && second.type == want, "launchLinearGemmPair: weight element type does not match the activations");
    const int M = rows_of(input), K = cols_of(input), N = first.shape[1];
    require(first.shape[0] == K, "launchLinearGemmPair: inner sizes differ (" + std::to_string(K) + " vs " + std::to_string(first.shape[0]) + ")");
    require(output->shape.size() == 3 && output->shape[0] == 2 && output->shape[1] == M && output->shape[2] == N,
            "launchLinearGemmPair: the output must be the {2, M, N} pair buffer");
    const int ldy = 2 * N;
    char* y = static_cast<char*>(output->data);
    const GemmWorkspace::Buffer ws = g_gemm_ws.get(onellmGetLaunchStream());
    const int dtype_code = input->dtype == FP32 ? ONELLM_FP32 : ONELLM_FP16;
    tune_pair_once(dtype_code, M, K, N, ldy, 0, ws.ptr, ws.bytes);
    const int rc = onellm_linear_pair(dtype_code, input->data, first.data, second.data, y, y + (size_t)N * e, M, K, N, ldy, 0, ws.ptr,
                                      ws.bytes, onellmGetLaunchStream());
    if (rc != 0) throw std::runtime_error(std::string("[TM][ERROR] launchLinearGemmPair: ") + onellm_error_string(rc) + " \n");
}

// ------------------------------------------------------------------------------------------- attention layer
LLaMASelfAttentionLayer::LLaMASelfAttentionLayer(int head_num, int kv_head_num, int head_size,
                                                 LLaMAAttentionStaticParams attn_params, hipStream_t stream,
                                                 cublasWrapper* cublas_wrapper, BaseAllocator* allocator,
                                                 bool is_free_buffer_after_fwd):
    head_num(head_num), head_size(head_size), hidden_units(head_num * head_size), kv_head_num(kv_head_num),
    is_free_buffer_after_fwd(is_free_buffer_after_fwd), attn_static_params(attn_params), allocator(allocator)
{
    (void)stream;
    (void)cublas_wrapper;
    require(kv_head_num > 0 && head_num % kv_head_num == 0, "query heads must be a multiple of kv heads");
    require(allocator != nullptr, "the attention layer needs an allocator");
}
LLaMASelfAttentionLayer::~LLaMASelfAttentionLayer() { free(); }

template<typename T>
void LLaMASelfAttentionLayer::allocForForward(LLaMAAttentionDynParams& params)
{
    const DataType t = getTensorType<T>();
    const int B = params.batch_size;
    if (qkv_buf && qkv_buf->shape[0] == B && qkv_buf->dtype == t) return;
    free();
    qkv_buf = new_buffer(allocator, t, {B, head_num + 2 * kv_head_num, head_size});
    mha_output = new_buffer(allocator, t, {B, hidden_units});
}
void LLaMASelfAttentionLayer::free()
{
    drop_buffer(allocator, qkv_buf);
    drop_buffer(allocator, mha_output);
}

// src/layers/attention/masked_self_attention.cpp:51-82
void LLaMASelfAttentionLayer::forward(TensorMap& inputs, TensorMap& outputs, LLaMAattentionWeights& weights,
                                      LLaMAAttentionDynParams& params)
{
    Tensor attention_input = inputs["attention_input"];
    Tensor attention_output = outputs["attention_output"];
    if (attention_input.dtype == FP16) allocForForward<half>(params);
    else allocForForward<float>(params);

    launchLinearGemm(&attention_input, weights.qkv, qkv_buf);

    // the launcher addresses layer 0 of whatever cache tensor it is given: hand it this layer's slab
    Tensor k_all = outputs["all_k_cache"], v_all = outputs["all_v_cache"];
    int layer = 0;
    if (inputs.isExist("layer_id")) layer = inputs["layer_id"].getVal<int>();
    Tensor k_slab = k_all, v_slab = v_all;
    if (k_all.shape.size() == 5) {
        require(layer >= 0 && layer < k_all.shape[0], "layer_id outside the cache");
        const std::vector<int> s4(k_all.shape.begin() + 1, k_all.shape.end());
        size_t slab = elt_bytes(k_all.dtype);
        for (int d : s4) slab *= (size_t)d;
        k_slab = Tensor(k_all.location, k_all.dtype, s4, static_cast<char*>(k_all.data) + slab * layer);
        v_slab = Tensor(v_all.location, v_all.dtype, s4, static_cast<char*>(v_all.data) + slab * layer);
    }
    Tensor finished = inputs["finished"];
    Tensor step = inputs["step"];
    launchDecoderMaskedMHA(qkv_buf, weights.qkv, &k_slab, &v_slab, &finished, &step, mha_output, attn_static_params,
                           rope_pos_offset);

    launchLinearGemm(mha_output, weights.output, &attention_output);
    if (is_free_buffer_after_fwd) free();
}

// ------------------------------------------------------------------------------------------------- FFN layer
LLaMAFFNLayer::LLaMAFFNLayer(int head_num, int head_size, int inter_size, hipStream_t stream, cublasWrapper* cublas_wrapper,
                             BaseAllocator* allocator, bool is_free_buffer_after_fwd):
    inter_size(inter_size), hidden_units(head_num * head_size), is_free_buffer_after_fwd(is_free_buffer_after_fwd),
    allocator(allocator)
{
    (void)stream;
    (void)cublas_wrapper;
    require(allocator != nullptr, "the FFN layer needs an allocator");
}
LLaMAFFNLayer::~LLaMAFFNLayer() { free(); }

template<typename T>
void LLaMAFFNLayer::allocForForward(int rows)
{
    const DataType t = getTensorType<T>();
    if (SwiGLU_input && SwiGLU_input->shape[1] == rows && SwiGLU_input->dtype == t) return;
    free();
    SwiGLU_input = new_buffer(allocator, t, {2, rows, inter_size});
    down_proj_input = new_buffer(allocator, t, {rows, inter_size});
}
template<typename T>
void LLaMAFFNLayer::allocForForward(LLaMAAttentionDynParams& params)
{
    allocForForward<T>(params.num_tokens > 0 ? params.num_tokens : params.batch_size);
}
void LLaMAFFNLayer::free()
{
    drop_buffer(allocator, SwiGLU_input);
    drop_buffer(allocator, down_proj_input);
}

// src/layers/ffn/ffn.cpp:53-73
void LLaMAFFNLayer::forward(TensorMap& inputs, TensorMap& outputs, LLaMAFFNWeights& weights, LLaMAAttentionDynParams& params)
{
    Tensor ffn_input = inputs["ffn_input"];
    Tensor ffn_output = outputs["ffn_output"];
    const int rows = rows_of(&ffn_input);
    require(cols_of(&ffn_input) == hidden_units && ffn_output.size() == ffn_input.size(), "ffn tensors are not [rows, hidden]");
    (void)params;
    if (ffn_input.dtype == FP16) allocForForward<half>(rows);
    else allocForForward<float>(rows);

    launchLinearGemmPair(&ffn_input, weights.gate, weights.up, SwiGLU_input);
    if (ffn_input.dtype == FP16)
        launchAct(static_cast<const half*>(SwiGLU_input->data), static_cast<half*>(down_proj_input->data), rows, inter_size);
    else
        launchAct(static_cast<const float*>(SwiGLU_input->data), static_cast<float*>(down_proj_input->data), rows, inter_size);
    launchLinearGemm(down_proj_input, weights.down, &ffn_output);
    if (is_free_buffer_after_fwd) free();
}

// --------------------------------------------------------------------------------------------------- decoder
LlamaSelfDecoder::LlamaSelfDecoder(int head_num, int kv_head_num, int head_size, int inter_size, int num_layer,
                                   const LLaMAAttentionStaticParams& attn_params, float rmsnorm_eps, hipStream_t stream,
                                   cublasWrapper* cublas_wrapper, BaseAllocator* allocator, bool is_free_buffer_after_forward):
    num_layer(num_layer), hidden_units(head_num * head_size), rmsnorm_eps(rmsnorm_eps), stream(stream),
    selfAttn(new LLaMASelfAttentionLayer(head_num, kv_head_num, head_size, attn_params, stream, cublas_wrapper, allocator,
                                         is_free_buffer_after_forward)),
    ffn(new LLaMAFFNLayer(head_num, head_size, inter_size, stream, cublas_wrapper, allocator, is_free_buffer_after_forward))
{
}
LlamaSelfDecoder::~LlamaSelfDecoder()
{
    delete selfAttn;
    delete ffn;
}
template<typename T>
void LlamaSelfDecoder::allocForForward(LLaMAAttentionDynParams&) {}   // no buffer of its own
void LlamaSelfDecoder::free() {}

namespace {
void fused_norm(Tensor& residual, Tensor& out, const void* bias, const void* gamma, float eps, int rows, int hidden)
{
    if (out.dtype == FP16)
        launchFusedAddBiasResidualRMSNorm(static_cast<half*>(residual.data), static_cast<half*>(out.data),
                                          static_cast<const half*>(bias), static_cast<const half*>(gamma), eps, rows, hidden);
    else
        launchFusedAddBiasResidualRMSNorm(static_cast<float*>(residual.data), static_cast<float*>(out.data),
                                          static_cast<const float*>(bias), static_cast<const float*>(gamma), eps, rows, hidden);
}
}  // namespace

// src/layers/decoder/self_decoder.cpp:15-78
void LlamaSelfDecoder::forward(TensorMap& input_tensors, const std::vector<LlamaLayerWeight*>& layerWeights,
                               TensorMap& output_tensors, LLaMAAttentionDynParams& dyn_params)
{
    require((int)layerWeights.size() >= num_layer, "fewer layer weights than layers");
    // a decoder constructed with a stream queues this step there; otherwise wherever the calling thread's launches go
    struct StreamScope {
        hipStream_t saved;
        bool active;
        StreamScope(hipStream_t s): saved(onellmGetLaunchStream()), active(s != nullptr) { if (active) onellmSetLaunchStream(s); }
        ~StreamScope() { if (active) onellmSetLaunchStream(saved); }
    } scope(stream);
    Tensor x = input_tensors["decoder_input"];      // residual stream
    Tensor y = output_tensors["decoder_output"];    // normalised activations / sub-layer results
    require(x.dtype == y.dtype && x.size() == y.size() && x.data != y.data, "decoder_input and decoder_output must be two buffers of one shape");
    const int rows = rows_of(&x);
    require(cols_of(&x) == hidden_units, "decoder_input is not [rows, head_num * head_size]");

    hip_ok(hipMemcpyAsync(y.data, x.data, (size_t)x.size() * elt_bytes(x.dtype), hipMemcpyDeviceToDevice, onellmGetLaunchStream()), "decoder copy");
    launchRMSNorm(&y, layerWeights[0]->attn_norm_weight, rmsnorm_eps);

    int layer_id = 0;
    TensorMap attn_in{{"attention_input", y},
                      {"layer_id", Tensor(Device::CPU, getTensorType<int>(), {1}, &layer_id)},
                      {"step", input_tensors["step"]},
                      {"finished", input_tensors["finished"]}};
    TensorMap attn_out{{"attention_output", y},
                       {"all_k_cache", output_tensors["all_k_cache"]},
                       {"all_v_cache", output_tensors["all_v_cache"]}};
    TensorMap ffn_in{{"ffn_input", y}};
    TensorMap ffn_out{{"ffn_output", y}};
    for (layer_id = 0; layer_id < num_layer; ++layer_id) {
        LlamaLayerWeight* w = layerWeights[layer_id];
        selfAttn->forward(attn_in, attn_out, w->self_attn_weight, dyn_params);
        fused_norm(x, y, w->self_attn_weight.output.bias, w->ffn_norm_weight.gamma, rmsnorm_eps, rows, hidden_units);
        ffn->forward(ffn_in, ffn_out, w->ffn_weight, dyn_params);
        const void* next_gamma = layer_id + 1 < num_layer ? (const void*)layerWeights[layer_id + 1]->attn_norm_weight.gamma
                                                          : (const void*)input_tensors["output_norm_weight"].data;
        fused_norm(x, y, w->ffn_weight.down.bias, next_gamma, rmsnorm_eps, rows, hidden_units);
    }
    hip_ok(hipGetLastError(), "decoder step");
}

template void LLaMASelfAttentionLayer::allocForForward<float>(LLaMAAttentionDynParams&);
template void LLaMASelfAttentionLayer::allocForForward<half>(LLaMAAttentionDynParams&);
template void LLaMAFFNLayer::allocForForward<float>(LLaMAAttentionDynParams&);
template void LLaMAFFNLayer::allocForForward<half>(LLaMAAttentionDynParams&);
template void LLaMAFFNLayer::allocForForward<float>(int);
template void LLaMAFFNLayer::allocForForward<half>(int);
template void LlamaSelfDecoder::allocForForward<float>(LLaMAAttentionDynParams&);
template void LlamaSelfDecoder::allocForForward<half>(LLaMAAttentionDynParams&);
