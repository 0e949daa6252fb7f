"""Pins the CPU oracle's norm, KV-cache and beam top-K functions: the reference unit tests'
constant inputs with their closed-form answers, library routines (torch rms_norm, np.repeat,
np.lexsort) and exhaustive small cases.  No GPU needed."""
import itertools
import math

import numpy as np
import pytest
import torch


# ---------------------------------------------------------------- RMSNorm

def test_rmsnorm_reference_unit_vector(ref):
    # tests/unittests/test_rmsnorm.cu:65-98: 2 x 32, x = 1, gamma = 1, eps = 0.5 -> 1/sqrt(1.5)
    x = np.ones((2, 32), np.float32)
    ref.rmsnorm(x, np.ones(32, np.float32), 0.5)
    np.testing.assert_allclose(x, 1.0 / math.sqrt(1.5), rtol=1e-7)


@pytest.mark.parametrize("dtype,N,H", [(np.float32, 5, 4096), (np.float16, 7, 4096), (np.float32, 3, 100),
                                       (np.float16, 2, 8192)])
def test_rmsnorm_matches_torch(ref, dtype, N, H):
    rng = np.random.default_rng(N * H)
    x = rng.standard_normal((N, H)).astype(dtype)
    g = rng.uniform(0.5, 1.5, H).astype(dtype)
    want = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (H,), torch.from_numpy(g).double(), 1e-5).numpy()
    got = ref.rmsnorm(x.copy(), g, 1e-5)
    if dtype == np.float32:
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)
    else:
        # one rounding of the exact value to fp16
        np.testing.assert_allclose(got.astype(np.float64), want, rtol=2 ** -10, atol=1e-7)


def test_rmsnorm_scale_invariance_and_unit_mean_square(ref):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((4, 512)).astype(np.float32)
    g = np.ones(512, np.float32)
    a = ref.rmsnorm(x.copy(), g, 0.0)
    b = ref.rmsnorm((x * 8.0).copy(), g, 0.0)
    np.testing.assert_allclose(a, b, rtol=1e-6)
    np.testing.assert_allclose((a.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-6)
    # with eps: mean((y/gamma)^2) = 1 / (1 + eps/ms)
    eps = 0.3
    c = ref.rmsnorm(x.copy(), g, eps)
    ms = (x.astype(np.float64) ** 2).mean(axis=1)
    np.testing.assert_allclose((c.astype(np.float64) ** 2).mean(axis=1), 1.0 / (1.0 + eps / ms), rtol=1e-6)


# ---------------------------------------------------------------- fused add-bias-residual-RMSNorm

def test_fused_norm_reference_unit_vector(ref):
    # tests/unittests/test_fused_addres_rms.cu:65-98: out = 1, residual = 0, bias = 0, gamma = 1, eps 0.5
    out = np.ones((2, 32), np.float32)
    res = np.zeros((2, 32), np.float32)
    ref.fused_add_bias_residual_rmsnorm(res, out, np.zeros(32, np.float32), np.ones(32, np.float32), 0.5)
    np.testing.assert_allclose(out, 1.0 / math.sqrt(1.5), rtol=1e-7)
    np.testing.assert_array_equal(res, 1.0)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("with_bias", [True, False])
def test_fused_norm_matches_float64(ref, dtype, with_bias):
    rng = np.random.default_rng(11)
    N, H = 6, 1024
    out = rng.standard_normal((N, H)).astype(dtype)
    res = rng.standard_normal((N, H)).astype(dtype)
    bias = rng.standard_normal(H).astype(dtype) if with_bias else None
    g = rng.uniform(0.5, 1.5, H).astype(dtype)
    # fp32 sum in the order out + residual + bias, as the kernel's first loop adds them
    r32 = out.astype(np.float32) + res.astype(np.float32)
    if with_bias:
        r32 = r32 + bias.astype(np.float32)
    r = r32.astype(np.float64)
    want_out = torch.nn.functional.rms_norm(torch.from_numpy(r), (H,), torch.from_numpy(g).double(), 1e-5).numpy()
    got_res, got_out = ref.fused_add_bias_residual_rmsnorm(res.copy(), out.copy(), bias, g, 1e-5)
    np.testing.assert_array_equal(got_res, r32.astype(dtype))     # residual <- r, rounded once
    if dtype == np.float32:
        np.testing.assert_allclose(got_out, want_out, rtol=2e-6, atol=1e-7)
    else:
        np.testing.assert_allclose(got_out.astype(np.float64), want_out, rtol=2 ** -10, atol=1e-7)


def test_fused_norm_zero_residual_equals_rmsnorm(ref):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((3, 256)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 256).astype(np.float32)
    a = ref.rmsnorm(x.copy(), g, 1e-5)
    _, b = ref.fused_add_bias_residual_rmsnorm(np.zeros_like(x), x.copy(), None, g, 1e-5)
    np.testing.assert_array_equal(a, b)


def test_fused_norm_as_written_variant_leaves_residual(ref):
    rng = np.random.default_rng(13)
    out = rng.standard_normal((2, 64)).astype(np.float32)
    res = rng.standard_normal((2, 64)).astype(np.float32)
    g = np.ones(64, np.float32)
    r0 = res.copy()
    _, o = ref.fused_add_bias_residual_rmsnorm(res, out.copy(), np.zeros(64, np.float32), g, 1e-5, as_written=True)
    np.testing.assert_array_equal(res, r0)
    r = (out + r0).astype(np.float64)
    inv = 1.0 / np.sqrt((r ** 2).mean(axis=1, keepdims=True) + 1e-5)
    np.testing.assert_allclose(o, out * inv, rtol=2e-6)


# ---------------------------------------------------------------- KV concat

def test_append_reference_unit_vector(ref):
    # tests/unittests/test_append_kvcache.cu:12-60: B1 Hkv2 q_len16 S32 D8, src = 1, cur_len 16, history 1
    ks = np.ones((1, 2, 16, 8), np.float32)
    vs = np.ones((1, 2, 16, 8), np.float32)
    kc = np.full((1, 1, 2, 32, 8), -9.0, np.float32)
    vc = np.full((1, 1, 2, 32, 8), -9.0, np.float32)
    ref.kv_append(ks, vs, kc, vc, [16], [1])
    for c in (kc, vc):
        np.testing.assert_array_equal(c[0, 0, :, 1:17], 1.0)
        np.testing.assert_array_equal(c[0, 0, :, 0], -9.0)
        np.testing.assert_array_equal(c[0, 0, :, 17:], -9.0)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_append_matches_slice_assignment(ref, dtype):
    rng = np.random.default_rng(21)
    L, B, Hkv, Q, S, D = 3, 4, 2, 5, 20, 16
    ks = rng.standard_normal((B, Hkv, Q, D)).astype(dtype)
    vs = rng.standard_normal((B, Hkv, Q, D)).astype(dtype)
    kc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    vc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    cur = np.array([5, 0, 3, 1])
    hist = np.array([0, 7, 15, 19])
    wk, wv = kc.copy(), vc.copy()
    for b in range(B):
        wk[1, b, :, hist[b]:hist[b] + cur[b]] = ks[b, :, :cur[b]]
        wv[1, b, :, hist[b]:hist[b] + cur[b]] = vs[b, :, :cur[b]]
    ref.kv_append(ks, vs, kc, vc, cur, hist, layer=1)
    np.testing.assert_array_equal(kc.view(np.uint8), wk.view(np.uint8))
    np.testing.assert_array_equal(vc.view(np.uint8), wv.view(np.uint8))


def test_append_drops_rows_beyond_cache(ref):
    ks = np.ones((1, 1, 4, 8), np.float32)
    kc = np.zeros((1, 1, 1, 6, 8), np.float32)
    vc = np.zeros((1, 1, 1, 6, 8), np.float32)
    ref.kv_append(ks, ks.copy(), kc, vc, [4], [4])
    np.testing.assert_array_equal(kc[0, 0, 0, 4:6], 1.0)
    np.testing.assert_array_equal(kc[0, 0, 0, :4], 0.0)


# ---------------------------------------------------------------- KV repeat

def test_repeat_reference_unit_vector(ref):
    # tests/unittests/test_transpose.cu:13-57: two layers of [1,2,4,2] filled with i, ctx_len 2,
    # dst [1,2,2,2] -> k_dst = [0,1,2,3, 8,9,10,11]
    src = np.arange(2 * 1 * 2 * 4 * 2, dtype=np.float32).reshape(2, 1, 2, 4, 2)
    kd = np.full((1, 2, 2, 2), -1.0, np.float32)
    vd = np.full((1, 2, 2, 2), -1.0, np.float32)
    ref.kv_repeat(src, src.copy(), kd, vd, [2], layer=0)
    np.testing.assert_array_equal(kd.ravel(), [0, 1, 2, 3, 8, 9, 10, 11])
    np.testing.assert_array_equal(vd.ravel(), [0, 1, 2, 3, 8, 9, 10, 11])


@pytest.mark.parametrize("dtype,Hq,Hkv", [(np.float16, 8, 2), (np.float32, 4, 4), (np.float16, 6, 1)])
def test_repeat_matches_np_repeat(ref, dtype, Hq, Hkv):
    rng = np.random.default_rng(31)
    L, B, S, MK, D = 2, 3, 12, 10, 8
    kc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    vc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    lens = np.array([10, 1, 6])
    kd = np.full((B, Hq, MK, D), 5.0, dtype)
    vd = np.full((B, Hq, MK, D), 5.0, dtype)
    wk, wv = kd.copy(), vd.copy()
    rk = np.repeat(kc[1], Hq // Hkv, axis=1)
    rv = np.repeat(vc[1], Hq // Hkv, axis=1)
    for b in range(B):
        wk[b, :, :lens[b]] = rk[b, :, :lens[b]]
        wv[b, :, :lens[b]] = rv[b, :, :lens[b]]
    ref.kv_repeat(kc, vc, kd, vd, lens, layer=1)
    np.testing.assert_array_equal(kd.view(np.uint8), wk.view(np.uint8))
    np.testing.assert_array_equal(vd.view(np.uint8), wv.view(np.uint8))


def test_repeat_clips_length_to_destination(ref):
    kc = np.arange(1 * 1 * 1 * 8 * 2, dtype=np.float32).reshape(1, 1, 1, 8, 2)
    kd = np.zeros((1, 2, 4, 2), np.float32)
    vd = np.zeros((1, 2, 4, 2), np.float32)
    ref.kv_repeat(kc, kc.copy(), kd, vd, [7])
    np.testing.assert_array_equal(kd[0, 0], kc[0, 0, 0, :4])
    np.testing.assert_array_equal(kd[0, 1], kc[0, 0, 0, :4])


# ---------------------------------------------------------------- beam top-K

def lexsort_topk(vals, ids, K):
    """K best by (value desc, id asc) using numpy's lexsort — an independent statement of the order."""
    order = np.lexsort((ids, -vals.astype(np.float64)))[:K]
    return vals[order], ids[order]


def expected_topk(logits, B, beam, K):
    rows, V = logits.shape
    flat = logits.reshape(B, beam * V)
    fv = np.zeros((B, K), np.float32)
    fi = np.zeros((B, K), np.int32)
    for b in range(B):
        ids = np.arange(beam * V, dtype=np.int64) + b * beam * V
        v, i = lexsort_topk(flat[b], ids, K)
        fv[b], fi[b] = v, i
    return fv, fi


def test_topk_reference_unit_vector(ref):
    # tests/unittests/test_beamsearch_topK.cu:12-25: B1 beam2 V30000 probs[i] = i, K = 2 -> ids 59999, 59998
    logits = np.arange(60000, dtype=np.float32).reshape(2, 30000)
    _, _, fv, fi = ref.beam_topk(logits, 1, 2, 2)
    np.testing.assert_array_equal(fi, [[59999, 59998]])
    np.testing.assert_array_equal(fv, [[59999.0, 59998.0]])


def test_topk_round1_layout_and_ids(ref):
    # every (row, block) partial holds the K best of the tokens that block owns, ids are global
    rng = np.random.default_rng(41)
    B, beam, V, K, nblk = 2, 2, 5000, 3, 8
    logits = rng.standard_normal((B * beam, V)).astype(np.float32)
    vals, ids, _, _ = ref.beam_topk(logits, B, beam, K, nblk)
    tok = np.arange(V)
    for r in range(B * beam):
        for lane in range(nblk):
            own = tok[(tok // 256) % nblk == lane]
            v, i = lexsort_topk(logits[r, own], own + r * V, K)
            np.testing.assert_array_equal(vals[r, lane], v)
            np.testing.assert_array_equal(ids[r, lane], i)


def test_topk_planted_ties_match_lexsort(ref):
    # BASELINE config 5: B8 x beam4, V32000, K4, N(0,2) with duplicate maxima planted
    rng = np.random.default_rng(5)
    B, beam, V, K = 8, 4, 32000, 4
    logits = (rng.standard_normal((B * beam, V)) * 2.0).astype(np.float32)
    for b in range(B):
        top = logits[b * beam:(b + 1) * beam].max() + 1.0
        for r in (b * beam, b * beam + 3):
            logits[r, [17, 16000, 31999]] = top
    _, _, fv, fi = ref.beam_topk(logits, B, beam, K)
    wv, wi = expected_topk(logits, B, beam, K)
    np.testing.assert_array_equal(fi, wi)
    np.testing.assert_array_equal(fv, wv)
    # lower index wins: the first three winners are the planted copies of the first beam
    for b in range(B):
        r = b * beam
        np.testing.assert_array_equal(fi[b, :3], [r * V + 17, r * V + 16000, r * V + 31999])
        assert fi[b, 3] == (r + 3) * V + 17


def test_topk_exhaustive_tie_patterns(ref):
    # every assignment of 3 distinct values to 6 slots (2 rows x 3 tokens): all tie patterns
    K = 4
    for pattern in itertools.product([0.0, 1.0, -1.0], repeat=6):
        logits = np.array(pattern, np.float32).reshape(2, 3)
        _, _, fv, fi = ref.beam_topk(logits, 1, 2, K, nblk=2)
        wv, wi = expected_topk(logits, 1, 2, K)
        np.testing.assert_array_equal(fi, wi)
        np.testing.assert_array_equal(fv, wv)


def test_topk_fewer_candidates_than_k(ref):
    logits = np.array([[3.0, -np.inf]], np.float32)
    _, _, fv, fi = ref.beam_topk(logits, 1, 1, 4, nblk=1)
    np.testing.assert_array_equal(fi, [[0, 1, -1, -1]])
    assert fv[0, 0] == 3.0 and np.isneginf(fv[0, 1:]).all()


def test_topk_monotone_rows_and_sortedness(ref):
    rng = np.random.default_rng(43)
    logits = rng.standard_normal((6, 777)).astype(np.float32)
    _, _, fv, fi = ref.beam_topk(logits, 3, 2, 5)
    assert (np.diff(fv, axis=1) <= 0).all()
    flat = logits.ravel()
    np.testing.assert_array_equal(flat[fi], fv)
