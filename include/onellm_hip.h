/*
 * onellm_hip.h — C ABI of the MI355X (gfx950) backend for oneLLM's per-token
 * decode hot path.
 *
 * Every entry point takes raw device pointers, plain ints/floats and a stream
 * handle, and returns an int: 0 on success, a positive hipError_t value when
 * the HIP runtime reported an error, or a negative ONELLM_E* code when an
 * argument is rejected before anything is launched.  Nothing here allocates
 * or frees device memory and nothing synchronises the device; the caller owns
 * all buffers.  `stream` is a hipStream_t passed as void* (NULL = the null
 * stream) so that a binder needs no HIP header.
 *
 * Each function names the reference interface it stands in for (paths are
 * relative to the oneLLM tree).
 */
#ifndef ONELLM_HIP_H
#define ONELLM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of activations / KV cache; values equal the reference's
 * `enum DataType` (src/utils/tensor.h:19-28): FP32 = 0, FP16 = 1. */
#define ONELLM_FP32 0
#define ONELLM_FP16 1

/* argument-rejection codes (negative so they never collide with hipError_t) */
#define ONELLM_EINVAL      (-1)  /* null pointer, non-positive size, bad enum  */
#define ONELLM_EUNSUPPORTED (-2) /* shape outside what the kernels are built for */
#define ONELLM_EWORKSPACE  (-3)  /* workspace missing or too small              */
#define ONELLM_ESCRATCH    (-4)  /* onellm_decode_attn_static: the step needs more than the built-in scratch */
#define ONELLM_ENOGEMMKERNEL (-5) /* onellm_linear (onellm_gemm.h): the GEMM library has no kernel for this problem and
                                     the plain kernel was not allowed                                          */
#define ONELLM_ECAPTURING  (-6)  /* the call would have to allocate or synchronise, and its stream is being captured */

/* flags for onellm_decode_attn */
#define ONELLM_ATTN_NO_V_BIAS     0x1u /* skip the v-bias add (reference decode kernel behaviour,
                                          src/kernels/decoder_masked_attn.cu:257-258)            */
#define ONELLM_ATTN_NO_CACHE_WRITE 0x2u /* do not store the new k/v row (read-only caches)        */
#define ONELLM_ATTN_ZEROED_WORKSPACE 0x4u /* the caller zero-filled the whole workspace once, after
                                          allocating it, and nothing but onellm_decode_attn has written
                                          it since.  A split sequence is then finished inside the one
                                          kernel (per-unit arrival counters at the front of the workspace,
                                          left at zero by every call) instead of by a second launch.
                                          Calls that share a workspace must not overlap.              */

typedef void* onellm_stream_t;

/* Library/ABI version: major*1000 + minor (1001: ONELLM_ATTN_ZEROED_WORKSPACE and the larger attention workspace). */
int onellm_hip_version(void);

/* Human-readable text for any code returned by this library.  Never NULL. */
const char* onellm_error_string(int code);

/*
 * Sets a launch-selection key for benchmarks and sweeps (for instance "attn_nsplit", "attn_balanced",
 * "attn_balanced_wgs", "attn_balanced_cost", "attn_fused_finish", "attn_turns", "attn_target_wgs",
 * "attn_gqa_valu", "norm_tpr", "prefill_generic"); value -1 hands the choice back to the launcher.
 * Process-wide, read at launch time.  The keys are not part of the stable interface: no caller
 * needs them, results never depend on them beyond rounding, and an unknown key returns
 * ONELLM_EINVAL.  No counterpart in the reference.
 */
int onellm_tune_set(const char* key, int value);

/*
 * Fused masked decoder self-attention for ONE new token per sequence.
 * Replaces launchDecoderMaskedMHA + masked_MHA_kernel
 * (src/kernels/decoder_masked_attn.h:7-14, src/kernels/decoder_masked_attn.cu:136-327).
 *
 *   qkv        [B, Hq+2*Hkv, D]   fused projection output, q|k|v head-major per token
 *   qkv_bias   [(Hq+2*Hkv)*D] or NULL (treated as zeros); q at h*D, k at Hq*D+kvh*D,
 *              v at (Hq+Hkv)*D+kvh*D (src/kernels/qkv_bias_and_RoPE.cu:116,125,131)
 *   k_cache,
 *   v_cache    [num_layers, B, Hkv, S, D]; slab `layer` is used; rows 0..t-2 are history
 *              and row t-1 is written by this call (roped+biased k, biased v)
 *   out        [B, Hq*D]
 *   t_host     number of attended positions (the reference's `step`,
 *              decoder_masked_attn.cu:294) used for every sequence when t_dev == NULL
 *   t_dev      optional device int32[B]: per-sequence t (1 <= t_dev[b] <= max_t)
 *   max_t      upper bound of all t (<= S); sizes the sequence split.  With t_dev == NULL
 *              pass t_host.
 *   rotary_dim, rope_base   LLaMAAttentionStaticParams (src/models/llama/llama_params.h:2-7),
 *              in the declared order; pairs (2i,2i+1) with 2i < rotary_dim are rotated by
 *              angle = pos / base^(2i/rotary_dim), pos = t + rope_pos_offset
 *              (offset 0 reproduces decoder_masked_attn.cu:186; -1 is the 0-based position
 *              that the prefill kernel uses, qkv_bias_and_RoPE.cu:140)
 *   workspace  device scratch of at least onellm_decode_attn_workspace_bytes() bytes, 256-byte
 *              aligned; contents on entry are irrelevant and nothing is carried between calls
 *              (unless ONELLM_ATTN_ZEROED_WORKSPACE says otherwise)
 *
 * Arithmetic is fp32 throughout; with ONELLM_FP16 the cache, qkv, bias and out are fp16 and the
 * new k/v rows are rounded to fp16 before they take part in this step's scores.
 * Shapes: Hq % Hkv == 0, 1 <= t <= S, D <= 512, B <= 65535.  Head sizes whose rows are a power of
 * two number of bytes (16..1024), or 10, 12, 20, 24, 40 or 48 16-byte pieces (D = 80, 96, 160, 192,
 * 320, 384 in fp16), in 16-byte aligned caches run the tiled kernels; anything else (odd D,
 * D = 72, 100, ..., unaligned caches) runs a slower scalar kernel with the same results.
 */
int onellm_decode_attn(int dtype,
                       const void* qkv, const void* qkv_bias,
                       void* k_cache, void* v_cache, void* out,
                       int B, int Hq, int Hkv, int D, int S,
                       int layer, int num_layers,
                       int t_host, const int* t_dev, int max_t,
                       int rotary_dim, float rope_base, int rope_pos_offset,
                       unsigned flags,
                       void* workspace, size_t workspace_bytes,
                       onellm_stream_t stream);

/* Bytes of workspace onellm_decode_attn needs for these sizes (0 never; at least 256). */
size_t onellm_decode_attn_workspace_bytes(int B, int Hq, int Hkv, int D, int max_t);

/*
 * onellm_decode_attn for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, results and kernels as onellm_decode_attn, minus the workspace: split partials and
 * arrival counters live in a fixed device array inside the library,
 * ONELLM_DECODE_ATTN_STATIC_SCRATCH_BYTES (16 MiB) per GPU, held from library load to process exit.
 * The call allocates, frees and synchronises nothing and launches only the attention kernel (the array is
 * zero when the library is loaded and every call leaves its counters at zero), so it can be the first call
 * on a stream that is being captured.  A step whose partials do not fit returns
 * ONELLM_ESCRATCH before anything is launched (onellm_decode_attn_workspace_bytes() is an upper bound
 * of what a step may need; steps that are not split need nothing).  All calls on one GPU share the
 * array, so calls that overlap in time on one GPU (two streams, two threads) race: serialise them.
 */
#define ONELLM_DECODE_ATTN_STATIC_SCRATCH_BYTES (16u << 20)
int onellm_decode_attn_static(int dtype,
                              const void* qkv, const void* qkv_bias,
                              void* k_cache, void* v_cache, void* out,
                              int B, int Hq, int Hkv, int D, int S,
                              int layer, int num_layers,
                              int t_host, const int* t_dev, int max_t,
                              int rotary_dim, float rope_base, int rope_pos_offset,
                              unsigned flags, onellm_stream_t stream);

/*
 * In-place RMSNorm over rows: x <- gamma * x * rsqrt(mean(x^2) + eps).
 * Replaces launchRMSNorm + RMSNorm (src/kernels/rmsnorm_kernel.h:6-9,
 * src/kernels/rmsnorm_kernel.cu:47-103).  x [N, H], gamma [H], both of `dtype`.
 */
int onellm_rmsnorm(int dtype, void* x, const void* gamma, float eps,
                   int N, int H, onellm_stream_t stream);

/*
 * Fused add-bias-residual + RMSNorm.  Replaces launchFusedAddBiasResidualRMSNorm
 * (src/kernels/fused_addresidual_norm.h:4-12, src/kernels/fused_addresidual_norm.cu:51-132):
 *   r = out + residual + bias;  residual <- r;  out <- gamma * r * rsqrt(mean(r^2) + eps)
 * residual, out [N, H]; bias [H] or NULL; gamma [H]; all of `dtype`.
 */
int onellm_fused_add_bias_residual_rmsnorm(int dtype, void* residual, void* out,
                                           const void* bias, const void* gamma, float eps,
                                           int N, int H, onellm_stream_t stream);

/*
 * KV-cache concat.  Replaces launchAppendKVCache (src/kernels/append_to_kvcache.h:20-26,
 * src/kernels/append_to_kvcache.cu:8-114):
 *   cache[layer, b, kvh, history_len[b] + tau, :] = src[b, kvh, tau, :]   for tau < cur_len[b]
 * k_src, v_src [B, Hkv, max_q_len, D]; caches [num_layers, B, Hkv, S, D];
 * cur_len, history_len device int32[B].  Rows that would land at or beyond S are dropped.
 */
int onellm_kv_append(int dtype, const void* k_src, const void* v_src,
                     void* k_cache, void* v_cache,
                     const int* cur_len, const int* history_len,
                     int B, int Hkv, int max_q_len, int S, int D,
                     int layer, int num_layers, onellm_stream_t stream);

/*
 * KV repeat (broadcast of KV heads to query heads).  Replaces launchTransposeKVCache
 * (src/kernels/transpose_kernel.h:5-11, src/kernels/transpose_kernel.cu:7-88):
 *   dst[b, h, s, :] = cache[layer, b, h / (Hq/Hkv), s, :]   for s < min(context_len[b], max_k_len)
 * caches [num_layers, B, Hkv, S, D]; k_dst, v_dst [B, Hq, max_k_len, D];
 * context_len device int32[B].  Rows at or beyond the length are left untouched.
 */
int onellm_kv_repeat(int dtype, const void* k_cache, const void* v_cache,
                     void* k_dst, void* v_dst, const int* context_len,
                     int B, int Hq, int Hkv, int S, int max_k_len, int D,
                     int layer, int num_layers, onellm_stream_t stream);

/*
 * Beam-search top-K.  Replaces launchTopKforBeamSearch (src/kernels/beamsearch_topK.h:35-38,
 * src/kernels/beamsearch_topK.cu:20-119).  logits [B*beam, V] fp32.
 * Order: larger value first; equal values: smaller global flat index (row*V + token) first.
 * Stage 1 keeps the K best of every (row, block) pair, stage 2 the K best of each batch entry.
 * workspace (fp32 words), the reference's layout generalised:
 *   vals[B*beam*nblk*K] | ids[B*beam*nblk*K] (int32) | final_vals[B*K] | final_ids[B*K] (int32)
 * nblk = ONELLM_TOPK_BLOCKS_PER_ROW (8, the reference's BlockPerBeam, beamsearch_topK.cu:105), so
 * with K = beam = 2 the final results sit exactly where the reference's unit test reads them
 * (tests/unittests/test_beamsearch_topK.cu:33-35).
 * 1 <= K <= 8.  Slots with no candidate hold value -inf and id -1.
 * On a stream that is not being captured both stages run in one kernel launch (the workgroup of a batch entry that
 * stores its survivors last merges them), for up to 1024 batch entries, with arrival counters the library keeps per
 * (GPU, workspace pointer): 64 sets per GPU, owned from a workspace's first call until onellm_release_workspace().
 * Beyond either limit, and on a stream under capture, stage 2 is a second launch (a launch less is worth more to the
 * host than the 1.5 us the longer kernel costs the device; a replayed graph has no host in it).  Same results either
 * way; onellm_beam_topk_last_path() tells which ran and why.  Two calls that may overlap in time need two
 * workspaces, as in the reference.
 */
#define ONELLM_TOPK_BLOCKS_PER_ROW 8
int onellm_beam_topk(const float* logits, int B, int beam, int V, int K,
                     float* workspace, onellm_stream_t stream);
size_t onellm_beam_topk_workspace_bytes(int B, int beam, int K);
/* kernel launches the last onellm_beam_topk call of this thread queued: 1 or 2 (0 before the first call or after
 * a refused one).  No counterpart in the reference; for tests and profiles. */
int onellm_beam_topk_last_launches(void);
/* which form the last onellm_beam_topk call of this thread took (0 before the first call or after a refused one).
 * No counterpart in the reference. */
#define ONELLM_TOPK_PATH_ONE_LAUNCH     1 /* both stages in one launch                                            */
#define ONELLM_TOPK_PATH_TWO_LAUNCHES   2 /* by design: stream under capture, more than 1024 batch entries, or the
                                             topk_two_launches tuning key                                          */
#define ONELLM_TOPK_PATH_NO_COUNTER_SET 3 /* two launches because every counter set of this GPU belongs to another
                                             workspace: release the ones no longer used                            */
int onellm_beam_topk_last_path(void);

/*
 * Arrival-counter sets.  Kernels that finish split work in one launch (the one-launch beam top-K here, the few-row
 * projection kernel of onellm_gemm.h when it cuts a problem along K) count arrivals in static device memory of the
 * library, one set of counters per (GPU, workspace pointer).  A set is owned from the first call that passes the
 * workspace and is never handed to another workspace behind the caller's back - a launch recorded into a graph keeps
 * its counters for as long as the graph lives.  A caller that frees or stops using a workspace gives its sets back:
 *   onellm_release_workspace(ptr)  returns how many sets (over all GPUs and kernel families) were freed.  The caller
 *       states that no launch that was handed `ptr` is queued, running, or recorded in a graph that will be replayed.
 * When every set of a GPU is owned, a call with a new workspace runs the form that needs no counters (a second
 * launch, an uncut run or the GEMM library): same results, slower, reported by the call's *_last_path query, counted
 * process-wide by onellm_counter_set_fallbacks() and announced once on stderr.  No counterpart in the reference
 * (its top-K always takes two launches, src/kernels/beamsearch_topK.cu:85-119).
 */
int onellm_release_workspace(const void* workspace);
long onellm_counter_set_fallbacks(void);

/* ------------------------------------------------------------------------------------------------
 * The callers either side of the decode path (built after the six entry points above).
 * ---------------------------------------------------------------------------------------------- */

/*
 * Context-phase fused QKV bias + RoPE + un-pad transpose: produces the K/V rows the decode step
 * streams.  Replaces launchAddFusedQKVBiasTransposeAndRoPE (src/kernels/qkv_bias_and_RoPE.h,
 * src/kernels/qkv_bias_and_RoPE.cu:74-207).  For each packed token tok:
 *   dst = tok + padding_offset[tok]; b = dst / seq_len; s = dst % seq_len; pos = history_length[b] + s
 *   q_buf[b, h, s, :] = RoPE(qkv[tok, h] + bias, pos);  k_buf[b, kvh, s, :] likewise;
 *   v_buf[b, kvh, s, :] = qkv[tok, Hq+Hkv+kvh] + bias
 * qkv [token_num, Hq+2*Hkv, D]; q_buf [B, Hq, seq_len, D]; k_buf, v_buf [B, Hkv, seq_len, D];
 * padding_offset device int32[token_num]; history_length device int32[B]; qkv_bias may be NULL.
 * Bias layout, RoPE arithmetic and rotary parameters are those of onellm_decode_attn; a decode step
 * with rope_pos_offset = -1 continues the positions this function writes.  D even, D <= 512.
 */
int onellm_qkv_bias_rope_transpose(int dtype, void* q_buf, void* k_buf, void* v_buf,
                                   const void* qkv, const void* qkv_bias,
                                   const int* padding_offset, const int* history_length,
                                   int B, int seq_len, int token_num, int Hq, int Hkv, int D,
                                   int rotary_dim, float rope_base, onellm_stream_t stream);

/*
 * SwiGLU gate.  Replaces launchAct<T> (src/kernels/activation_kernel.h, src/kernels/activation_kernel.cu:5-32):
 *   out[b, i] = silu(input[b, 0, i]) * input[b, 1, i],  silu(x) = x / (1 + exp(-x)) in fp32.
 * input [B, 2, I], out [B, I].
 */
int onellm_silu_and_mul(int dtype, const void* input, void* out, int B, int I, onellm_stream_t stream);

/*
 * Top-K sampling: the consumer of the beam top-K output.  Replaces launchSampling
 * (src/kernels/topK_sampling.h, src/kernels/topK_sampling.cu:6-70).  Per batch row, with the K
 * (value, id) pairs sorted best-first:  w_i = exp(val_i - val_0);  thr = u * sum(w);  the first i whose
 * running subtraction takes thr below 0 wins (the last one if rounding never does);
 *   output_id = topk_id[i] % vocab_size;  seqlen += 1 unless is_finished;  is_finished = (output_id == end_id).
 * topk_id int32 [B, K], topk_val fp32 [B, K] (not modified), output_id / seqlen int32 [B],
 * is_finished one byte per row (C++ bool).  u comes from Philox4x32-10 with key = seed (the reference
 * passes the step) and counter = (row, 0, 0, 0): reproducible on a CPU, but NOT the stream cuRAND's
 * XORWOW would give the reference.
 */
int onellm_topk_sample(const int* topk_id, const float* topk_val, int* output_id, int* seqlen,
                       unsigned char* is_finished, int B, int K, unsigned long long seed, int end_id,
                       int vocab_size, onellm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ONELLM_HIP_H */
