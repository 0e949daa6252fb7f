"""Pins the oracle's prefill QKV-bias+RoPE+transpose and SwiGLU functions (the callers either side of
the decode path): the reference unit tests' constant inputs, independent float64 formulations, and the
prefill -> decode consistency of the RoPE convention.  No GPU needed."""
import numpy as np
import pytest
import torch

from test_oracle_attn import rope64


def _pack(B, seq_len, lens):
    """token -> padding_offset for sequences of the given lengths packed back to back."""
    po = []
    tok = 0
    for b, n in enumerate(lens):
        for s in range(n):
            po.append(b * seq_len + s - tok)
            tok += 1
    return np.array(po, np.int32)


def test_prefill_reference_unit_vector(ref):
    # tests/unittests/test_qkv_bias_and_rope.cu:111-145: B1, seq 32, Hq2, Hkv1, D8, rotary 128, base 10000,
    # QKV = 1, bias = 2, history 4, padding_offset 0
    B, S, Hq, Hkv, D = 1, 32, 2, 1, 8
    qkv = np.ones((32, Hq + 2 * Hkv, D), np.float32)
    bias = np.full((Hq + 2 * Hkv) * D, 2.0, np.float32)
    q = np.zeros((B, Hq, S, D), np.float32)
    k = np.zeros((B, Hkv, S, D), np.float32)
    v = np.zeros((B, Hkv, S, D), np.float32)
    ref.qkv_bias_rope_transpose(q, k, v, qkv, bias, np.zeros(32, np.int32), [4], 128, 10000.0)
    # the angle pos/freq is an fp32 number: at pos 35 half an ulp is 1.9e-6 rad, times |x| = 3*sqrt(2)
    for s in range(S):
        want = rope64(np.full(D, 3.0), 128, 10000.0, 4 + s)
        np.testing.assert_allclose(q[0, 0, s], want, rtol=0, atol=1.5e-5)
        np.testing.assert_allclose(q[0, 1, s], want, rtol=0, atol=1.5e-5)
        np.testing.assert_allclose(k[0, 0, s], want, rtol=0, atol=1.5e-5)
    np.testing.assert_array_equal(v, 3.0)                      # bias only, no rotation


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_prefill_ragged_against_float64(ref, dtype):
    rng = np.random.default_rng(8)
    B, S, Hq, Hkv, D = 3, 12, 4, 2, 16
    lens = [12, 5, 1]
    hist = np.array([0, 7, 30], np.int32)
    T = sum(lens)
    qkv = rng.standard_normal((T, Hq + 2 * Hkv, D)).astype(dtype)
    bias = rng.standard_normal((Hq + 2 * Hkv) * D).astype(dtype)
    po = _pack(B, S, lens)
    q = np.full((B, Hq, S, D), 9.0, dtype)
    k = np.full((B, Hkv, S, D), 9.0, dtype)
    v = np.full((B, Hkv, S, D), 9.0, dtype)
    ref.qkv_bias_rope_transpose(q, k, v, qkv, bias, po, hist, D, 10000.0)
    b3 = bias.astype(np.float32).reshape(Hq + 2 * Hkv, D)
    tok = 0
    tol = dict(rtol=0, atol=1.5e-5) if dtype == np.float32 else dict(rtol=2e-3, atol=2e-3)
    for b, n in enumerate(lens):
        for s in range(n):
            x = qkv[tok].astype(np.float32) + b3                 # fp32 add, as the kernel does
            np.testing.assert_allclose(q[b, :, s].astype(np.float64), rope64(x[:Hq], D, 10000.0, hist[b] + s), **tol)
            np.testing.assert_allclose(k[b, :, s].astype(np.float64), rope64(x[Hq:Hq + Hkv], D, 10000.0, hist[b] + s), **tol)
            np.testing.assert_array_equal(v[b, :, s], x[Hq + Hkv:].astype(dtype))
            tok += 1
        # padded positions untouched
        np.testing.assert_array_equal(q[b, :, n:], 9.0)
        np.testing.assert_array_equal(k[b, :, n:], 9.0)
        np.testing.assert_array_equal(v[b, :, n:], 9.0)


def test_prefill_then_decode_share_the_rope_convention(ref):
    # K rows written by the prefill function at 0-based positions 0..t-2, then one decode step at
    # rope_pos_offset = -1: the step's new K row must equal what prefill would have written for that
    # token, and the output must equal float64 attention over the un-rotated tokens with RoPE applied
    rng = np.random.default_rng(9)
    B, Hq, Hkv, D, S, t = 1, 2, 2, 16, 8, 6
    tokens = rng.standard_normal((t, Hq + 2 * Hkv, D)).astype(np.float32)
    q = np.zeros((B, Hq, S, D), np.float32)
    kc = np.zeros((1, B, Hkv, S, D), np.float32)
    vc = np.zeros((1, B, Hkv, S, D), np.float32)
    ref.qkv_bias_rope_transpose(q, kc[0], vc[0], tokens[:t - 1], None, np.zeros(t - 1, np.int32), [0], D, 10000.0)
    k_all = np.zeros((B, Hkv, S, D), np.float32)
    ref.qkv_bias_rope_transpose(np.zeros_like(q), k_all, np.zeros_like(k_all), tokens, None, np.zeros(t, np.int32), [0], D, 10000.0)
    out = ref.decode_attn(tokens[t - 1:t], None, kc, vc, Hq, t, D, 10000.0, rope_pos_offset=-1)
    np.testing.assert_array_equal(kc[0, 0, :, t - 1], k_all[0, :, t - 1])          # bit for bit
    K = np.stack([rope64(tokens[j, Hq:Hq + Hkv], D, 10000.0, j) for j in range(t)], 1)   # [Hkv, t, D]
    V = tokens[:, Hq + Hkv:].transpose(1, 0, 2).astype(np.float64)
    Q = rope64(tokens[t - 1, :Hq], D, 10000.0, t - 1)
    want = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(Q)[None, :, None], torch.from_numpy(K)[None], torch.from_numpy(V)[None]).reshape(1, -1).numpy()
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-6)


def test_prefill_rejects_tokens_outside_the_batch(ref):
    qkv = np.zeros((2, 3, 8), np.float32)
    q = np.zeros((1, 1, 1, 8), np.float32)
    with pytest.raises(RuntimeError):
        ref.qkv_bias_rope_transpose(q, q.copy(), q.copy(), qkv, None, [0, 0], [0], 8, 10000.0)   # token 1 -> batch 1


def test_swiglu_reference_unit_vector(ref):
    # tests/unittests/test_activation.cu:41-47: B16, I 11008, input[i] = i  ->  silu(x) = x for large x, out = x*y
    B, I = 16, 11008
    inp = np.arange(B * 2 * I, dtype=np.float32).reshape(B, 2, I)
    out = ref.silu_and_mul(inp, np.zeros((B, I), np.float32))
    x, y = inp[:, 0].astype(np.float64), inp[:, 1].astype(np.float64)
    np.testing.assert_allclose(out, x / (1 + np.exp(-x)) * y, rtol=2e-7)
    assert out[0, 0] == 0.0


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_swiglu_matches_torch_silu(ref, dtype):
    rng = np.random.default_rng(10)
    inp = (rng.standard_normal((7, 2, 300)) * 3).astype(dtype)
    out = ref.silu_and_mul(inp, np.zeros((7, 300), dtype))
    t = torch.from_numpy(inp).double()
    want = (torch.nn.functional.silu(t[:, 0]) * t[:, 1]).numpy()
    np.testing.assert_allclose(out.astype(np.float64), want, rtol=2e-6 if dtype == np.float32 else 2 ** -10, atol=1e-7)


# ---------------------------------------------------------------- top-K sampling

def test_philox_published_known_answers(ref):
    # Random123's kat_vectors for philox4x32-10
    assert [hex(x) for x in ref.philox4x32_10([0, 0, 0, 0], [0, 0])] == ['0x6627e8d5', '0xe169c58d', '0xbc57ac4c', '0x9b00dbd8']
    assert [hex(x) for x in ref.philox4x32_10([0xffffffff] * 4, [0xffffffff] * 2)] == \
        ['0x408f276d', '0x41c83b0e', '0xa20bc7c6', '0x6d5451fd']
    assert [hex(x) for x in ref.philox4x32_10([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0])] == \
        ['0xd16cfe09', '0x94fdcceb', '0x5001e420', '0x24126ea1']


def test_fixed_exp_and_uniform(ref):
    xs = np.linspace(-100, 0, 4001).astype(np.float32)
    got = np.array([ref.exp_fixed(x) for x in xs])
    want = np.exp(xs.astype(np.float64))
    ok = want > 1e-37
    assert (np.abs(got[ok] - want[ok]) / want[ok]).max() < 4e-7
    assert ref.exp_fixed(0.0) == 1.0 and ref.exp_fixed(-200.0) == 0.0
    assert ref.uniform_from_u32(0) == 2.0 ** -32 and ref.uniform_from_u32(0xffffffff) == 1.0      # (0, 1]


def _sample_model(ids, vals, seed, vocab):
    """Independent float64 statement: inverse-CDF sampling of softmax(vals) with the oracle's uniform."""
    from oracle import ref as r
    out = []
    for b in range(ids.shape[0]):
        u = r.uniform_from_u32(r.philox4x32_10([b, 0, 0, 0], [seed & 0xffffffff, seed >> 32])[0])
        p = np.exp(vals[b].astype(np.float64) - vals[b, 0])
        cdf = np.cumsum(p)
        i = int(np.searchsorted(cdf, u * cdf[-1], side="right"))
        out.append(ids[b, min(i, ids.shape[1] - 1)] % vocab)
    return np.array(out, np.int32)


def test_sampling_reference_unit_vector_shapes(ref):
    # tests/unittests/test_topK_sampling.cu:8-47: B3, K3, vocab 1000, step 5, end_id 10, ids 0..8, vals 2,1,0 per row
    B, K = 3, 3
    ids = np.arange(B * K, dtype=np.int32).reshape(B, K)
    vals = np.tile(np.array([2.0, 1.0, 0.0], np.float32), (B, 1))
    seqlen = np.full(B, 4, np.int32)
    fin = np.zeros(B, np.uint8)
    out = ref.topk_sample(ids, vals, seqlen, fin, 5, 10, 1000)
    np.testing.assert_array_equal(out, _sample_model(ids, vals, 5, 1000))
    assert all(out[b] in ids[b] for b in range(B))
    np.testing.assert_array_equal(seqlen, 5)
    np.testing.assert_array_equal(fin, 0)


def test_sampling_distribution_bookkeeping_and_determinism(ref):
    rng = np.random.default_rng(3)
    B, K, vocab = 4000, 4, 32000
    vals = np.sort(rng.standard_normal((B, K)).astype(np.float32) * 2, axis=1)[:, ::-1].copy()
    vals[:] = vals[0]                                       # same distribution in every row
    ids = np.tile(np.array([5, 32000 + 7, 9, 11], np.int32), (B, 1))     # a global flat id: % vocab -> 7
    seqlen = np.arange(B, dtype=np.int32)
    fin = (np.arange(B) % 2).astype(np.uint8)
    out = ref.topk_sample(ids, vals, seqlen, fin, 123456789012, 7, vocab)
    np.testing.assert_array_equal(out, _sample_model(ids, vals, 123456789012, vocab))
    # frequencies follow softmax(vals) (4000 draws: 4 sigma of a binomial)
    p = np.exp(vals[0].astype(np.float64) - vals[0, 0]); p /= p.sum()
    for k, tok in enumerate([5, 7, 9, 11]):
        f = (out == tok).mean()
        assert abs(f - p[k]) < 4 * np.sqrt(p[k] * (1 - p[k]) / B) + 1e-3
    np.testing.assert_array_equal(seqlen, np.arange(B) + (np.arange(B) % 2 == 0))      # finished rows do not grow
    np.testing.assert_array_equal(fin, (out == 7).astype(np.uint8))
    out2 = ref.topk_sample(ids, vals, np.zeros(B, np.int32), np.zeros(B, np.uint8), 123456789012, 7, vocab)
    np.testing.assert_array_equal(out, out2)
    out3 = ref.topk_sample(ids, vals, np.zeros(B, np.int32), np.zeros(B, np.uint8), 123456789013, 7, vocab)
    assert (out != out3).any()


def test_sampling_degenerate_rows(ref):
    ids = np.array([[3, 4, 5]], np.int32)
    vals = np.array([[0.0, -np.inf, -np.inf]], np.float32)              # all the mass on the first
    out = ref.topk_sample(ids, vals, np.zeros(1, np.int32), np.zeros(1, np.uint8), 1, -1, 100)
    assert out[0] == 3
    out = ref.topk_sample(ids[:, :1].copy(), vals[:, :1].copy(), np.zeros(1, np.int32), np.zeros(1, np.uint8), 9, -1, 100)
    assert out[0] == 3
