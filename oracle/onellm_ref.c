/*
 * onellm_ref.c — CPU oracle for the decode hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only the test-suite, the smoke check and the
 * benchmark's CPU-baseline leg may build, load or call it.  The HIP library does not link it
 * and has no CPU fallback.
 *
 * It restates, in plain C, what the oneLLM decode-path kernels are meant to compute.  Each
 * function cites the reference lines it follows (paths relative to the oneLLM tree).  Where the
 * reference snapshot contradicts itself the choice made is written beside the citation.
 *
 * Numeric model (all functions): element-wise work (bias add, RoPE, exp, scale, gamma) is done
 * in fp32 exactly as written; dot products and running sums are accumulated in double so that
 * the oracle is the value the fp32 inputs define, not one particular summation order.  With
 * dtype FP16 the buffers hold IEEE binary16 and every load widens / every store rounds once
 * (round-to-nearest-even).
 *
 * The RoPE sine/cosine are NOT libm's: they are a fixed sequence of IEEE fp32 operations
 * (3-term Cody-Waite reduction + degree-7/8 polynomials) so that a GPU kernel performing the
 * same sequence produces the same bits; onellm_ref_sincosf is pinned against double-precision
 * sin/cos in the test-suite.
 *
 * Parity status: every function below is pinned by known-answer tests taken from the reference's
 * own unit tests and by independent float64 formulations (tests/test_oracle_*.py), with one
 * exception.  onellm_ref_topk_sample: the random draw is "parity unpinned" against the reference,
 * whose uniform comes from cuRAND's XORWOW generator (a CUDA-toolkit library, not vendored, no
 * version pinned, absent here); everything around the draw (weights, threshold walk, id % vocab,
 * seqlen / finished bookkeeping) and the Philox generator used instead are pinned.
 * Tie order of the beam top-K is fixed by the task statement (lower index wins), not by a
 * reference test.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <immintrin.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* Number of host threads the loops below may use; returns the previous setting (1 without OpenMP).  Only the
 * benchmark's single-thread baseline changes it. */
int onellm_ref_set_threads(int n)
{
#ifdef _OPENMP
    const int before = omp_get_max_threads();
    if (n > 0) omp_set_num_threads(n);
    return before;
#else
    (void)n;
    return 1;
#endif
}

#define REF_FP32 0
#define REF_FP16 1

#define REF_ATTN_NO_V_BIAS      0x1u
#define REF_ATTN_NO_CACHE_WRITE 0x2u

/* ---------------------------------------------------------------- fp16 <-> fp32 */

static inline float h2f(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

static inline float ld(const void* p, size_t i, int dtype)
{
    return dtype == REF_FP16 ? h2f(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
static inline void st(void* p, size_t i, int dtype, float v)
{
    if (dtype == REF_FP16) ((uint16_t*)p)[i] = f2h(v);
    else ((float*)p)[i] = v;
}
/* value after one round trip through the storage type */
static inline float rnd(float v, int dtype) { return dtype == REF_FP16 ? h2f(f2h(v)) : v; }

static void ld_row(float* dst, const void* p, size_t off, int n, int dtype)
{
    if (dtype == REF_FP16) {
        const uint16_t* s = (const uint16_t*)p + off;
        int i = 0;
        for (; i + 8 <= n; i += 8)
            _mm256_storeu_ps(dst + i, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(s + i))));
        for (; i < n; ++i) dst[i] = h2f(s[i]);
    } else {
        memcpy(dst, (const float*)p + off, (size_t)n * sizeof(float));
    }
}

/* ---------------------------------------------------------------- deterministic sin/cos */

/*
 * sin and cos of an fp32 angle as a fixed sequence of fp32 IEEE operations.
 * Reduction: j = rint(x * 2/pi); r = x - j*pi/2 with pi/2 split in three fp32 terms, each
 * step one fused multiply-add.  Polynomials: the classic single-precision minimax pair on
 * [-pi/4, pi/4].  Quadrant from j & 3.  Valid for |x| < ~1e5 (positions of any KV cache).
 */
void onellm_ref_sincosf(float x, float* s_out, float* c_out)
{
    const float TWO_OVER_PI = 0x1.45f306p-1f;
    const float PIO2_HI = 0x1.921fb6p+0f;
    const float PIO2_MID = -0x1.777a5cp-25f;
    const float PIO2_LO = -0x1.0p-49f;
    float j = rintf(x * TWO_OVER_PI);
    float r = fmaf(-j, PIO2_HI, x);
    r = fmaf(-j, PIO2_MID, r);
    r = fmaf(-j, PIO2_LO, r);
    float r2 = r * r;
    float ps = fmaf(-1.9515295891e-4f, r2, 8.3321608736e-3f);
    ps = fmaf(ps, r2, -1.6666654611e-1f);
    float sr = fmaf(r * r2, ps, r);
    float pc = fmaf(2.443315711809948e-5f, r2, -1.388731625493765e-3f);
    pc = fmaf(pc, r2, 4.166664568298827e-2f);
    float cr = fmaf(r2 * r2, pc, fmaf(-0.5f, r2, 1.0f));
    int q = (int)j & 3;
    float s = (q & 1) ? cr : sr;
    float c = (q & 1) ? sr : cr;
    if (q & 2) s = -s;
    if ((q + 1) & 2) c = -c;
    *s_out = s;
    *c_out = c;
}

/*
 * Rotation frequencies of RoPE: freq[i] = base^(2i/rotary_dim), 2i < min(rotary_dim, D), and the angle
 * of pair i at position p is p / freq[i]  (src/kernels/decoder_masked_attn.cu:95-99 `GetRoPEfreq`:
 * `t_step / powf(base, zid / (float)rot_embed_dim)` with zid = 2i;
 * restated independently at tests/unittests/test_qkv_bias_and_rope.cu:56-66).
 */
void onellm_ref_rope_freqs(float* freq, int D, int rotary_dim, float base)
{
    /* rotary_dim may exceed D (the example drivers run rotary_dim 128 with D 8): the exponent
       keeps rotary_dim in the denominator and only the pairs that exist are rotated. */
    for (int i = 0; 2 * i < rotary_dim && 2 * i + 1 < D; ++i)
        freq[i] = powf(base, (float)(2 * i) / (float)rotary_dim);
}

/*
 * Rotate adjacent pairs (x[2i], x[2i+1]), 2i < rotary_dim, in place
 * (src/kernels/decoder_masked_attn.cu:102-131 `GetRoPEres` / `apply_RoPE`):
 *   x'[2i]   = cos*x[2i]   - sin*x[2i+1]
 *   x'[2i+1] = cos*x[2i+1] + sin*x[2i]
 * written as fma(x0, c, -(x1*s)) and fma(x1, c, x0*s) so the rounding sequence is fixed.
 */
void onellm_ref_rope_row(float* x, int D, int rotary_dim, const float* freq, int pos)
{
    for (int i = 0; 2 * i + 1 < D && 2 * i < rotary_dim; ++i) {
        float ang = (float)pos / freq[i];
        float s, c;
        onellm_ref_sincosf(ang, &s, &c);
        float x0 = x[2 * i], x1 = x[2 * i + 1];
        x[2 * i]     = fmaf(x0, c, -(x1 * s));
        x[2 * i + 1] = fmaf(x1, c, x0 * s);
    }
}

/* ---------------------------------------------------------------- decode attention */

/*
 * One decode step of fused masked self-attention
 * (src/kernels/decoder_masked_attn.cu:136-268 kernel, :280-327 launcher).
 *
 * Flow per (b, q-head h), kvh = h / (Hq/Hkv):
 *   q = qkv[b, h] + bias[h*D..]                      (:175-180)
 *   k = qkv[b, Hq+kvh] + bias[Hq*D + kvh*D..]        (:181-185)
 *   v = qkv[b, Hq+Hkv+kvh] + bias[(Hq+Hkv)*D+kvh*D..]  (v bias as the prefill kernel adds it,
 *        src/kernels/qkv_bias_and_RoPE.cu:130-134; the decode kernel as written skips it,
 *        :257-258 — flag REF_ATTN_NO_V_BIAS reproduces that)
 *   RoPE(q), RoPE(k) at position pos = t + rope_pos_offset   (:186 uses `step`, i.e. offset 0)
 *   cache row t-1 <- k, v (rounded to the storage type)      (:208-214, :255-259)
 *   s_j = (q . K_j) / sqrt(D), j < t                          (:218-224, scale :301)
 *   p = softmax(s) with the true row maximum                  (:228-244; the kernel as written
 *        is only valid for t <= D — not reproduced)
 *   out[b, h*D + d] = sum_j p_j V_j[d]                        (:247-267)
 *
 * Layout choices where the snapshot disagrees with itself: the fused buffer has batch stride
 * (Hq+2Hkv)*D (:296-299 slices one [B, Hq+2Hkv, D] buffer); the cache is
 * [num_layers, B, Hkv, S, D] as the layer allocates it (examples/cpp/decoder/self_decoder_example.cpp:186-187)
 * and as the concat kernel writes it (src/kernels/append_to_kvcache.cu:32-34); GQA maps q-head h
 * to kv-head h/G as the repeat kernel does (src/kernels/transpose_kernel.cu:32).
 *
 * t_arr (host int[B]) gives a per-sequence t; NULL means t_host for all.
 */
int onellm_ref_decode_attn(int dtype, const void* qkv, const void* qkv_bias,
                           void* k_cache, void* v_cache, void* out,
                           int B, int Hq, int Hkv, int D, int S, int layer, int num_layers,
                           int t_host, const int* t_arr,
                           int rotary_dim, float rope_base, int rope_pos_offset, unsigned flags)
{
    if (!qkv || !k_cache || !v_cache || !out || B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || S <= 0) return -1;
    if (Hq % Hkv || layer < 0 || layer >= num_layers) return -1;
    const int G = Hq / Hkv;
    const int QKVH = Hq + 2 * Hkv;
    const float scale = 1.0f / sqrtf((float)D);
    float* freq = (float*)malloc(sizeof(float) * (size_t)(D / 2 + 1));
    onellm_ref_rope_freqs(freq, D, rotary_dim, rope_base);
    const size_t slab = (size_t)layer * B * Hkv * S * D;
    int bad = 0;

#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b) {
        for (int kvh = 0; kvh < Hkv; ++kvh) {
            const int t = t_arr ? t_arr[b] : t_host;
            if (t < 1 || t > S) {
#pragma omp atomic write
                bad = 1;
                continue;
            }
            const int pos = t + rope_pos_offset;
            float* kn = (float*)malloc(sizeof(float) * (size_t)D * 4);
            float* vn = kn + D;
            float* q = vn + D;
            float* row = q + D;
            float* sc = (float*)malloc(sizeof(float) * (size_t)t);
            double* acc = (double*)malloc(sizeof(double) * (size_t)D);
            const size_t tok = (size_t)b * QKVH * D;
            /* new k / v rows */
            for (int d = 0; d < D; ++d) {
                kn[d] = ld(qkv, tok + (size_t)(Hq + kvh) * D + d, dtype);
                vn[d] = ld(qkv, tok + (size_t)(Hq + Hkv + kvh) * D + d, dtype);
                if (qkv_bias) kn[d] += ld(qkv_bias, (size_t)(Hq + kvh) * D + d, dtype);
                if (qkv_bias && !(flags & REF_ATTN_NO_V_BIAS)) vn[d] += ld(qkv_bias, (size_t)(Hq + Hkv + kvh) * D + d, dtype);
            }
            onellm_ref_rope_row(kn, D, rotary_dim, freq, pos);
            for (int d = 0; d < D; ++d) {
                kn[d] = rnd(kn[d], dtype);
                vn[d] = rnd(vn[d], dtype);
            }
            const size_t base = slab + ((size_t)b * Hkv + kvh) * (size_t)S * D;
            if (!(flags & REF_ATTN_NO_CACHE_WRITE)) {
                for (int d = 0; d < D; ++d) {
                    st(k_cache, base + (size_t)(t - 1) * D + d, dtype, kn[d]);
                    st(v_cache, base + (size_t)(t - 1) * D + d, dtype, vn[d]);
                }
            }
            for (int g = 0; g < G; ++g) {
                const int h = kvh * G + g;
                for (int d = 0; d < D; ++d) {
                    q[d] = ld(qkv, tok + (size_t)h * D + d, dtype);
                    if (qkv_bias) q[d] += ld(qkv_bias, (size_t)h * D + d, dtype);
                }
                onellm_ref_rope_row(q, D, rotary_dim, freq, pos);
                float smax = -INFINITY;
                for (int j = 0; j < t; ++j) {
                    const float* kr;
                    if (j == t - 1) kr = kn;
                    else { ld_row(row, k_cache, base + (size_t)j * D, D, dtype); kr = row; }
                    double a0 = 0, a1 = 0, a2 = 0, a3 = 0;
                    int d = 0;
                    for (; d + 4 <= D; d += 4) {
                        a0 += (double)q[d] * kr[d];
                        a1 += (double)q[d + 1] * kr[d + 1];
                        a2 += (double)q[d + 2] * kr[d + 2];
                        a3 += (double)q[d + 3] * kr[d + 3];
                    }
                    for (; d < D; ++d) a0 += (double)q[d] * kr[d];
                    sc[j] = (float)((a0 + a1) + (a2 + a3)) * scale;
                    if (sc[j] > smax) smax = sc[j];
                }
                double denom = 0;
                for (int d = 0; d < D; ++d) acc[d] = 0;
                for (int j = 0; j < t; ++j) {
                    const float p = expf(sc[j] - smax);
                    denom += p;
                    const float* vr;
                    if (j == t - 1) vr = vn;
                    else { ld_row(row, v_cache, base + (size_t)j * D, D, dtype); vr = row; }
                    for (int d = 0; d < D; ++d) acc[d] += (double)p * vr[d];
                }
                for (int d = 0; d < D; ++d)
                    st(out, (size_t)b * Hq * D + (size_t)h * D + d, dtype, (float)(acc[d] / denom));
            }
            free(acc);
            free(sc);
            free(kn);
        }
    }
    free(freq);
    return bad ? -1 : 0;
}

/* ---------------------------------------------------------------- norms */

/*
 * In-place RMSNorm (src/kernels/rmsnorm_kernel.cu:47-83): per row
 *   inv = rsqrt(sum(x^2)/H + eps)   (:61-72)      x <- gamma * x * inv   (:76-82)
 * The multiplication order gamma*x then *inv follows :78-81.
 */
int onellm_ref_rmsnorm(int dtype, void* x, const void* gamma, float eps, int N, int H)
{
    if (!x || !gamma || N < 0 || H <= 0) return -1;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const size_t o = (size_t)n * H;
        double ss = 0;
        for (int i = 0; i < H; ++i) {
            float v = ld(x, o + i, dtype);
            ss += (double)v * v;
        }
        const float inv = (float)(1.0 / sqrt(ss / H + (double)eps));
        for (int i = 0; i < H; ++i)
            st(x, o + i, dtype, ld(gamma, i, dtype) * ld(x, o + i, dtype) * inv);
    }
    return 0;
}

/*
 * Fused add-bias-residual-RMSNorm (src/kernels/fused_addresidual_norm.cu:51-107).
 * Intended semantics (what the calling layer relies on, src/layers/decoder/self_decoder.cpp:49-56
 * "decoder_output += decoder_input", and what the kernel's first loop computes, :78-82):
 *   r = out + residual + bias;  residual <- r (rounded to storage);
 *   out <- gamma * r * rsqrt(mean(r^2) + eps), r taken un-rounded.
 * as_written != 0 reproduces the snapshot instead (:99-105): the sum is used only for the
 * mean, `out` is scaled from its un-added value and residual is left alone.
 */
int onellm_ref_fused_add_bias_residual_rmsnorm(int dtype, void* residual, void* out,
                                               const void* bias, const void* gamma, float eps,
                                               int N, int H, int as_written)
{
    if (!residual || !out || !gamma || N < 0 || H <= 0) return -1;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const size_t o = (size_t)n * H;
        float* r = (float*)malloc(sizeof(float) * (size_t)H);
        double ss = 0;
        for (int i = 0; i < H; ++i) {
            r[i] = ld(out, o + i, dtype) + ld(residual, o + i, dtype);
            if (bias) r[i] += ld(bias, i, dtype);          /* no "+ 0" when absent: keeps -0 */
            ss += (double)r[i] * r[i];
        }
        const float inv = (float)(1.0 / sqrt(ss / H + (double)eps));
        for (int i = 0; i < H; ++i) {
            if (as_written) {
                st(out, o + i, dtype, ld(gamma, i, dtype) * ld(out, o + i, dtype) * inv);
            } else {
                st(residual, o + i, dtype, r[i]);
                st(out, o + i, dtype, ld(gamma, i, dtype) * r[i] * inv);
            }
        }
        free(r);
    }
    return 0;
}

/* ---------------------------------------------------------------- KV cache concat / repeat */

static size_t esize(int dtype) { return dtype == REF_FP16 ? 2 : 4; }

/*
 * KV concat (src/kernels/append_to_kvcache.cu:27-36 index math, :81-87 shapes):
 *   cache[layer, b, kvh, history[b]+tau, :] = src[b, kvh, tau, :]   for tau < cur_len[b]
 * The layer slab offset is the one the launcher comment gives (:75) and hard-codes to 0 (:87).
 * Rows that would fall outside [0, S) are dropped (the reference has no guard).
 */
int onellm_ref_kv_append(int dtype, const void* k_src, const void* v_src, void* k_cache, void* v_cache,
                         const int* cur_len, const int* history_len,
                         int B, int Hkv, int max_q_len, int S, int D, int layer, int num_layers)
{
    if (!k_src || !v_src || !k_cache || !v_cache || !cur_len || !history_len) return -1;
    if (B <= 0 || Hkv <= 0 || max_q_len <= 0 || S <= 0 || D <= 0 || layer < 0 || layer >= num_layers) return -1;
    const size_t e = esize(dtype), rowb = (size_t)D * e;
    const size_t slab = (size_t)layer * B * Hkv * S * D;
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < Hkv; ++h)
            for (int tau = 0; tau < max_q_len && tau < cur_len[b]; ++tau) {
                const long drow = (long)history_len[b] + tau;
                if (drow < 0 || drow >= S) continue;
                const size_t so = (((size_t)b * Hkv + h) * max_q_len + tau) * D;
                const size_t d_o = slab + (((size_t)b * Hkv + h) * S + (size_t)drow) * D;
                memcpy((char*)k_cache + d_o * e, (const char*)k_src + so * e, rowb);
                memcpy((char*)v_cache + d_o * e, (const char*)v_src + so * e, rowb);
            }
    return 0;
}

/*
 * KV repeat for grouped-query heads (src/kernels/transpose_kernel.cu:30-41 index math,
 * :53-62 shapes):  dst[b, h, s, :] = cache[layer, b, h/G, s, :]  for s < context_len[b];
 * dst is [B, Hq, max_k_len, D]; rows >= length are not written.  Lengths above max_k_len are
 * clipped (the reference grid simply has no threads there, :65).
 */
int onellm_ref_kv_repeat(int dtype, const void* k_cache, const void* v_cache, void* k_dst, void* v_dst,
                         const int* context_len, int B, int Hq, int Hkv, int S, int max_k_len, int D,
                         int layer, int num_layers)
{
    if (!k_cache || !v_cache || !k_dst || !v_dst || !context_len) return -1;
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || S <= 0 || max_k_len <= 0 || D <= 0) return -1;
    if (layer < 0 || layer >= num_layers) return -1;
    const int G = Hq / Hkv;
    const size_t e = esize(dtype), rowb = (size_t)D * e;
    const size_t slab = (size_t)layer * B * Hkv * S * D;
    for (int b = 0; b < B; ++b) {
        int len = context_len[b];
        if (len > max_k_len) len = max_k_len;
        if (len > S) len = S;
        for (int h = 0; h < Hq; ++h)
            for (int s = 0; s < len; ++s) {
                const size_t so = slab + (((size_t)b * Hkv + h / G) * S + s) * D;
                const size_t d_o = (((size_t)b * Hq + h) * max_k_len + s) * D;
                memcpy((char*)k_dst + d_o * e, (const char*)k_cache + so * e, rowb);
                memcpy((char*)v_dst + d_o * e, (const char*)v_cache + so * e, rowb);
            }
    }
    return 0;
}

/* ---------------------------------------------------------------- beam-search top-K */

/* candidate order: larger value first, then smaller id (global flat index) */
static inline int better(float v1, int i1, float v2, int i2)
{
    return v1 > v2 || (v1 == v2 && (unsigned)i1 < (unsigned)i2);
}

/*
 * Sorted-K insertion list (src/kernels/beamsearch_topK.h:3-33 `topK<K>::insertHeap`): the
 * candidate replaces the last slot when it is better, then one bubble pass restores order.
 * Unlike the reference's strict `>` on values alone (:16-31), the comparison is the total
 * order above, so the result does not depend on insertion order.  Empty slots are id -1.
 */
static void topk_insert(float* val, int* id, int K, float v, int i)
{
    if (id[K - 1] != -1 && !better(v, i, val[K - 1], id[K - 1])) return;
    val[K - 1] = v;
    id[K - 1] = i;
    for (int s = K - 2; s >= 0; --s) {
        if (id[s] == -1 || better(val[s + 1], id[s + 1], val[s], id[s])) {
            float tv = val[s]; val[s] = val[s + 1]; val[s + 1] = tv;
            int ti = id[s]; id[s] = id[s + 1]; id[s + 1] = ti;
        } else break;
    }
}

/*
 * Two-round beam top-K (src/kernels/beamsearch_topK.cu:20-52 round 1, :57-83 round 2,
 * :85-119 launcher and workspace plan).
 * Round 1: row r = [b, beam] is scanned by nblk blocks of 256 lanes; block `lane` owns tokens
 *   tid + lane*256 + m*nblk*256 (:35); candidate id = global flat index r*V + token (:36-38);
 *   output [B*beam, nblk, K] (:45-49).
 * Round 2: the beam*nblk*K candidates of each batch entry are merged into [B, K] (:70-81).
 * Workspace (fp32 words): vals | ids | final_vals | final_ids (:92-99).
 * Empty slots: value -inf, id -1.
 */
int onellm_ref_beam_topk(const float* logits, int B, int beam, int V, int K, int nblk, float* workspace)
{
    if (!logits || !workspace || B <= 0 || beam <= 0 || V <= 0 || K <= 0 || K > 64 || nblk <= 0) return -1;
    const size_t n1 = (size_t)B * beam * nblk * K;
    float* vals = workspace;
    int* ids = (int*)(vals + n1);
    float* fvals = (float*)(ids + n1);
    int* fids = (int*)(fvals + (size_t)B * K);
    const int rows = B * beam;
#pragma omp parallel for collapse(2) schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int lane = 0; lane < nblk; ++lane) {
            float v[64]; int id[64];
            for (int k = 0; k < K; ++k) { v[k] = -INFINITY; id[k] = -1; }
            for (int base = lane * 256; base < V; base += nblk * 256)
                for (int tok = base; tok < base + 256 && tok < V; ++tok)
                    topk_insert(v, id, K, logits[(size_t)r * V + tok], r * V + tok);
            for (int k = 0; k < K; ++k) {
                vals[((size_t)r * nblk + lane) * K + k] = v[k];
                ids[((size_t)r * nblk + lane) * K + k] = id[k];
            }
        }
    for (int b = 0; b < B; ++b) {
        float v[64]; int id[64];
        for (int k = 0; k < K; ++k) { v[k] = -INFINITY; id[k] = -1; }
        const size_t n = (size_t)beam * nblk * K;
        for (size_t i = 0; i < n; ++i) {
            const int cid = ids[(size_t)b * n + i];
            if (cid != -1) topk_insert(v, id, K, vals[(size_t)b * n + i], cid);
        }
        for (int k = 0; k < K; ++k) {
            fvals[(size_t)b * K + k] = v[k];
            fids[(size_t)b * K + k] = id[k];
        }
    }
    return 0;
}

/* ---------------------------------------------------------------- prefill: fused QKV bias + RoPE + un-pad transpose */

/*
 * Context-phase companion of the decode kernel (src/kernels/qkv_bias_and_RoPE.cu:74-161 kernel,
 * :167-207 launcher).  For every packed token `tok` (no padding between sequences):
 *   dst = tok + padding_offset[tok];  b = dst / seq_len;  s = dst % seq_len          (:97-104)
 *   q[h]   = QKV[tok, h]          + bias[h*D..]                                      (:115-119)
 *   k[kvh] = QKV[tok, Hq+kvh]     + bias[Hq*D + kvh*D..]                             (:123-128)
 *   v[kvh] = QKV[tok, Hq+Hkv+kvh] + bias[(Hq+Hkv)*D + kvh*D..]                       (:130-134)
 *   RoPE(q), RoPE(k) at the 0-based position history_length[b] + s                   (:138-143)
 *   q_buf[b, h, s, :] = q;  k_buf[b, kvh, s, :] = k;  v_buf[b, kvh, s, :] = v        (:147-159)
 * q_buf is [B, Hq, seq_len, D], k_buf/v_buf [B, Hkv, seq_len, D]; padded positions are not written.
 * input_length is read by the reference only to form an unused value (:139) and is not needed.
 * Same bias/RoPE arithmetic as the decode step above, so prefill and decode agree bit for bit.
 */
int onellm_ref_qkv_bias_rope_transpose(int dtype, void* q_buf, void* k_buf, void* v_buf, const void* qkv,
                                       const void* qkv_bias, const int* padding_offset, const int* history_length,
                                       int B, int seq_len, int token_num, int Hq, int Hkv, int D,
                                       int rotary_dim, float rope_base)
{
    if (!q_buf || !k_buf || !v_buf || !qkv || !padding_offset || !history_length) return -1;
    if (B <= 0 || seq_len <= 0 || token_num < 0 || Hq <= 0 || Hkv <= 0 || D <= 0) return -1;
    const int QKVH = Hq + 2 * Hkv;
    float* freq = (float*)malloc(sizeof(float) * (size_t)(D / 2 + 1));
    onellm_ref_rope_freqs(freq, D, rotary_dim, rope_base);
    int bad = 0;
#pragma omp parallel for schedule(static)
    for (int tok = 0; tok < token_num; ++tok) {
        const long dst = (long)tok + padding_offset[tok];
        const long b = dst / seq_len, s = dst % seq_len;
        if (dst < 0 || b >= B) {
#pragma omp atomic write
            bad = 1;
            continue;
        }
        const int pos = history_length[b] + (int)s;
        float* row = (float*)malloc(sizeof(float) * (size_t)D);
        for (int h = 0; h < QKVH; ++h) {
            for (int d = 0; d < D; ++d) {
                row[d] = ld(qkv, ((size_t)tok * QKVH + h) * D + d, dtype);
                if (qkv_bias) row[d] += ld(qkv_bias, (size_t)h * D + d, dtype);
            }
            void* out;
            size_t o;
            if (h < Hq) {
                onellm_ref_rope_row(row, D, rotary_dim, freq, pos);
                out = q_buf;
                o = (((size_t)b * Hq + h) * seq_len + (size_t)s) * D;
            } else if (h < Hq + Hkv) {
                onellm_ref_rope_row(row, D, rotary_dim, freq, pos);
                out = k_buf;
                o = (((size_t)b * Hkv + (h - Hq)) * seq_len + (size_t)s) * D;
            } else {
                out = v_buf;
                o = (((size_t)b * Hkv + (h - Hq - Hkv)) * seq_len + (size_t)s) * D;
            }
            for (int d = 0; d < D; ++d) st(out, o + d, dtype, row[d]);
        }
        free(row);
    }
    free(freq);
    return bad ? -1 : 0;
}

/* ---------------------------------------------------------------- SwiGLU */

/*
 * silu(x) * y over [B, 2, I] -> [B, I]  (src/kernels/activation_kernel.cu:5-22; CPU checker
 * tests/unittests/test_activation.cu:12-22): silu(x) = x / (1 + expf(-x)) in fp32.
 */
int onellm_ref_silu_and_mul(int dtype, const void* input, void* out, int B, int I)
{
    if (!input || !out || B < 0 || I <= 0) return -1;
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b)
        for (int i = 0; i < I; ++i) {
            const float x = ld(input, (size_t)b * 2 * I + i, dtype);
            const float y = ld(input, (size_t)b * 2 * I + I + i, dtype);
            st(out, (size_t)b * I + i, dtype, (x / (1.0f + expf(-x))) * y);
        }
    return 0;
}

/* ---------------------------------------------------------------- top-K sampling */

/*
 * Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11): counter-based,
 * so a CPU and a GPU produce the same stream from (key, counter) alone.  The reference draws its
 * uniform from cuRAND's XORWOW generator (src/kernels/topK_sampling.cu:28-30, `curand_init(step,
 * batch_id, 0)` + `curand_uniform`); cuRAND is a CUDA-toolkit library that is neither vendored in
 * the reference tree nor available here, so THAT stream is not reproduced: the random draw is
 * "parity unpinned" against the reference, and pinned only against this restatement (itself
 * checked on the published Philox known-answer vectors).
 */
void onellm_ref_philox4x32_10(const uint32_t ctr_in[4], const uint32_t key_in[2], uint32_t out[4])
{
    uint32_t c0 = ctr_in[0], c1 = ctr_in[1], c2 = ctr_in[2], c3 = ctr_in[3];
    uint32_t k0 = key_in[0], k1 = key_in[1];
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* uniform in (0, 1]: (x + 1) * 2^-32 evaluated as x * 2^-32 + 2^-32 in fp32 (one fma) */
float onellm_ref_uniform_from_u32(uint32_t x) { return fmaf((float)x, 0x1.0p-32f, 0x1.0p-32f); }

/* e^x for x <= 0 as a fixed fp32 sequence (same idea as the sin/cos above): n = rint(x*log2 e),
 * r = x - n*ln2 in two fma steps, degree-6 polynomial by Horner with fma, scale by 2^n through the
 * exponent field; below 2^-126 the result is 0. */
float onellm_ref_exp_fixed(float x)
{
    const float n = rintf(x * 0x1.715476p+0f);
    float r = fmaf(-n, 0x1.62e400p-1f, x);
    r = fmaf(-n, 0x1.7f7d1cp-20f, r);
    float p = fmaf(0x1.6c16c2p-10f, r, 0x1.111112p-7f);    /* 1/720, 1/120 */
    p = fmaf(p, r, 0x1.555556p-5f);                         /* 1/24 */
    p = fmaf(p, r, 0x1.555556p-3f);                         /* 1/6 */
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    const int e = (int)n;
    if (e < -126) return 0.0f;
    union { uint32_t u; float f; } s;
    s.u = (uint32_t)(e + 127) << 23;
    return p * s.f;
}

/*
 * Top-K sampling (src/kernels/topK_sampling.cu:6-41 kernel, :43-70 launcher).  Per batch row:
 *   w_i = exp(val_i - val_0)                      (:20-21; val_0 is the maximum, the row is sorted)
 *   sum = w_0 + ... + w_{K-1}, added in that order (:24-27)
 *   thr = u * sum, u uniform in (0, 1]            (:28-30)
 *   walk i = 0..K-1: thr -= w_i; first i with thr < 0 wins (:31-37).  The snapshot subtracts the
 *     same element every time (`topk_val[offset]` with thread 0's offset, :32); the walk over w_i is
 *     what the loop is for and is what is restated.  If rounding leaves thr >= 0 after the last
 *     element, the last element wins (the snapshot would leave the output unwritten).
 *   output_id = topk_id[i] % vocab_size           (:34)
 *   seqlen += 1 unless already finished (:38);  is_finished = (output_id == end_id) (:39)
 * The snapshot also overwrites topk_val with the w_i (:21); this restatement leaves the inputs alone.
 * RNG: Philox4x32-10, key = (seed low word, seed high word) with seed = the reference's `rand_num`
 * (the step), counter = (batch row, 0, 0, 0), first output word.
 */
int onellm_ref_topk_sample(const int* topk_id, const float* topk_val, int* output_id, int* seqlen,
                           unsigned char* is_finished, int B, int K, unsigned long long seed, int end_id, int vocab_size)
{
    if (!topk_id || !topk_val || !output_id || !seqlen || !is_finished || B < 0 || K <= 0 || vocab_size <= 0) return -1;
    for (int b = 0; b < B; ++b) {
        const float* v = topk_val + (size_t)b * K;
        float sum = 0.0f;
        for (int i = 0; i < K; ++i) sum += onellm_ref_exp_fixed(v[i] - v[0]);
        const uint32_t ctr[4] = {(uint32_t)b, 0, 0, 0}, key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
        uint32_t rnd[4];
        onellm_ref_philox4x32_10(ctr, key, rnd);
        float thr = onellm_ref_uniform_from_u32(rnd[0]) * sum;
        int pick = K - 1;
        for (int i = 0; i < K; ++i) {
            thr -= onellm_ref_exp_fixed(v[i] - v[0]);
            if (thr < 0) { pick = i; break; }
        }
        output_id[b] = topk_id[(size_t)b * K + pick] % vocab_size;
        seqlen[b] = is_finished[b] ? seqlen[b] : seqlen[b] + 1;
        is_finished[b] = output_id[b] == end_id ? 1 : 0;
    }
    return 0;
}
