"""Pins the CPU oracle's decode attention: known answers taken from the reference's own unit
tests, closed forms, and independent float64 formulations (complex-number RoPE, torch SDPA,
explicit loops).  No GPU needed."""
import math

import numpy as np
import pytest
import torch


# ---------------------------------------------------------------- independent float64 model

def rope64(x, rotary_dim, base, pos):
    """RoPE as a complex multiplication: (x0 + i x1) * exp(i * pos * base**(-2i/rd))."""
    x = np.asarray(x, dtype=np.float64).copy()
    D = x.shape[-1]
    n = min(rotary_dim, D) // 2
    if n == 0:
        return x
    z = x[..., 0:2 * n:2] + 1j * x[..., 1:2 * n:2]
    theta = pos * np.power(float(base), -np.arange(n) * 2.0 / rotary_dim)
    z = z * np.exp(1j * theta)
    x[..., 0:2 * n:2] = z.real
    x[..., 1:2 * n:2] = z.imag
    return x


def attn64(qkv, bias, k_cache, v_cache, Hq, t, rotary_dim, base, layer=0, pos_offset=0, v_bias=True,
           store_dtype=np.float32):
    """Float64 model of one decode step.  Returns (out, new_k [B,Hkv,D], new_v)."""
    B, QKVH, D = qkv.shape
    Hkv = (QKVH - Hq) // 2
    G = Hq // Hkv
    qkv = qkv.astype(np.float64)
    bias = np.zeros(QKVH * D) if bias is None else bias.astype(np.float64)
    bq = bias[:Hq * D].reshape(Hq, D)
    bk = bias[Hq * D:(Hq + Hkv) * D].reshape(Hkv, D)
    bv = bias[(Hq + Hkv) * D:].reshape(Hkv, D)
    t = np.broadcast_to(np.asarray(t), (B,))
    out = np.zeros((B, Hq * D))
    nk = np.zeros((B, Hkv, D))
    nv = np.zeros((B, Hkv, D))
    for b in range(B):
        tb = int(t[b])
        pos = tb + pos_offset
        q = rope64(qkv[b, :Hq] + bq, rotary_dim, base, pos)
        k = rope64(qkv[b, Hq:Hq + Hkv] + bk, rotary_dim, base, pos)
        v = qkv[b, Hq + Hkv:] + (bv if v_bias else 0.0)
        k = k.astype(store_dtype).astype(np.float64)
        v = v.astype(store_dtype).astype(np.float64)
        nk[b], nv[b] = k, v
        for h in range(Hq):
            kvh = h // G
            K = np.concatenate([k_cache[layer, b, kvh, :tb - 1].astype(np.float64), k[kvh][None]], 0)
            V = np.concatenate([v_cache[layer, b, kvh, :tb - 1].astype(np.float64), v[kvh][None]], 0)
            s = K @ q[h] / math.sqrt(D)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[b, h * D:(h + 1) * D] = p @ V
    return out, nk, nv


# ---------------------------------------------------------------- sin/cos and RoPE

def test_sincos_against_float64(ref):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        np.linspace(0, 8192, 4001), rng.uniform(0, 20000, 4000), rng.uniform(-50, 50, 2000),
        np.arange(0, 64) * (math.pi / 4), [0.0, 1e-8, 1e-4, 0.5, math.pi / 2, math.pi, 4096.0, 8191.0],
    ]).astype(np.float32)
    s, c = ref.sincosf_array(x)
    es, ec = np.sin(x.astype(np.float64)), np.cos(x.astype(np.float64))
    # <= 2 ulp at magnitude 1 (absolute), which a wrong polynomial term or quadrant breaks
    assert np.abs(s - es).max() < 2.4e-7
    assert np.abs(c - ec).max() < 2.4e-7
    assert ref.sincosf(0.0) == (0.0, 1.0)


def test_sincos_quadrants(ref):
    # one point per quadrant with a known sign pattern
    for k in range(8):
        x = np.float32(0.3 + k * math.pi / 2)
        s, c = ref.sincosf(float(x))
        assert abs(s - math.sin(float(x))) < 2.4e-7 and abs(c - math.cos(float(x))) < 2.4e-7


def test_rope_freqs(ref):
    f = ref.rope_freqs(128, 10000.0)
    assert f.shape == (64,)
    assert f[0] == 1.0
    expect = 10000.0 ** (np.arange(64) * 2.0 / 128)
    np.testing.assert_allclose(f, expect, rtol=3e-7)


@pytest.mark.parametrize("D,rd,pos,tol", [(64, 64, 17, 2e-6), (128, 128, 5, 2e-6), (128, 64, 31, 4e-6),
                                           (16, 128, 4, 2e-6), (128, 128, 4096, 2e-3)])
def test_rope_row_matches_complex_rotation(ref, D, rd, pos, tol):
    # tol grows with pos only because the angle pos/freq is an fp32 number (ulp(4096) = 4.9e-4)
    rng = np.random.default_rng(D + pos)
    x = rng.standard_normal(D).astype(np.float32)
    got = ref.rope_row(x.copy(), rd, 10000.0, pos)
    want = rope64(x, rd, 10000.0, pos)
    np.testing.assert_allclose(got, want, atol=tol * 4, rtol=0)
    # untouched tail when rotary_dim < D
    if rd < D:
        np.testing.assert_array_equal(got[rd:], x[rd:])
    # a rotation keeps the length of every pair
    np.testing.assert_allclose(got[0::2] ** 2 + got[1::2] ** 2, x[0::2] ** 2 + x[1::2] ** 2, rtol=1e-5)


def test_rope_position_zero_is_identity(ref):
    x = np.random.default_rng(0).standard_normal(64).astype(np.float32)
    np.testing.assert_array_equal(ref.rope_row(x.copy(), 64, 10000.0, 0), x)


# ---------------------------------------------------------------- reference unit-test vectors

def _ref_unit_case():
    """Inputs of tests/unittests/test_decoder_masked_attn.cu:113-176 in the reference tree:
    B1, Hq2, Hkv1, D16, step 4, max_seq 32; qkv = 1, bias = 2, first `step` cache rows = 1."""
    B, Hq, Hkv, D, t, S = 1, 2, 1, 16, 4, 32
    qkv = np.ones((B, Hq + 2 * Hkv, D), np.float32)
    bias = np.full(((Hq + 2 * Hkv) * D,), 2.0, np.float32)
    kc = np.zeros((1, B, Hkv, S, D), np.float32)
    vc = np.zeros((1, B, Hkv, S, D), np.float32)
    kc[:, :, :, :t] = 1.0
    vc[:, :, :, :t] = 1.0
    return B, Hq, Hkv, D, t, S, qkv, bias, kc, vc


def test_reference_unit_vector_without_v_bias(ref):
    # all V rows (history and the raw new v) are 1 => output is exactly 1 whatever the weights are
    B, Hq, Hkv, D, t, S, qkv, bias, kc, vc = _ref_unit_case()
    out = ref.decode_attn(qkv, bias, kc, vc, Hq, t, 128, 10000.0, flags=ref.ATTN_NO_V_BIAS)
    np.testing.assert_allclose(out, 1.0, rtol=1e-6)
    np.testing.assert_array_equal(vc[0, 0, 0, t - 1], 1.0)


def test_reference_unit_vector_with_v_bias_closed_form(ref):
    # history V rows are 1, new row is 1+2 => out = 1 + 2*p_last; history K rows are all equal, so
    # p_last = 1 / (1 + (t-1) * exp(s_hist - s_last))
    B, Hq, Hkv, D, t, S, qkv, bias, kc, vc = _ref_unit_case()
    out = ref.decode_attn(qkv, bias, kc, vc, Hq, t, 128, 10000.0)
    q = rope64(np.full(D, 3.0), 128, 10000.0, t)
    k = rope64(np.full(D, 3.0), 128, 10000.0, t)
    s_hist = q.sum() / math.sqrt(D)
    s_last = (q * k).sum() / math.sqrt(D)
    p_last = 1.0 / (1.0 + (t - 1) * math.exp(s_hist - s_last))
    np.testing.assert_allclose(out, 1.0 + 2.0 * p_last, rtol=2e-6)
    np.testing.assert_array_equal(vc[0, 0, 0, t - 1], 3.0)
    np.testing.assert_allclose(kc[0, 0, 0, t - 1], k, rtol=2e-6, atol=1e-6)
    # rows beyond t-1 untouched
    assert not kc[0, 0, 0, t:].any() and not vc[0, 0, 0, t:].any()


def test_example_driver_shapes(ref):
    # examples/cpp/decoder/self_decoder_example.cpp:10-27: Hq4 Hkv2 D8 B2 step3 max_seq12,
    # rotary_dim 128 > D, two layers
    rng = np.random.default_rng(3)
    B, Hq, Hkv, D, t, S, L = 2, 4, 2, 8, 3, 12, 2
    qkv = rng.standard_normal((B, Hq + 2 * Hkv, D)).astype(np.float32)
    bias = rng.standard_normal((Hq + 2 * Hkv) * D).astype(np.float32)
    kc = rng.standard_normal((L, B, Hkv, S, D)).astype(np.float32)
    vc = rng.standard_normal((L, B, Hkv, S, D)).astype(np.float32)
    for layer in range(L):
        k0, v0 = kc.copy(), vc.copy()
        want, nk, nv = attn64(qkv, bias, k0, v0, Hq, t, 128, 10000.0, layer=layer)
        out = ref.decode_attn(qkv, bias, kc, vc, Hq, t, 128, 10000.0, layer=layer)
        np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(kc[layer, :, :, t - 1], nk, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(vc[layer, :, :, t - 1], nv, rtol=1e-6)
        # only row t-1 of this layer changed
        k0[layer, :, :, t - 1] = kc[layer, :, :, t - 1]
        v0[layer, :, :, t - 1] = vc[layer, :, :, t - 1]
        np.testing.assert_array_equal(k0, kc)
        np.testing.assert_array_equal(v0, vc)


# ---------------------------------------------------------------- closed forms / invariants

def test_empty_history_returns_v_plus_bias(ref):
    rng = np.random.default_rng(5)
    B, Hq, Hkv, D, S = 3, 4, 2, 32, 8
    qkv = rng.standard_normal((B, Hq + 2 * Hkv, D)).astype(np.float32)
    bias = rng.standard_normal((Hq + 2 * Hkv) * D).astype(np.float32)
    kc = np.full((1, B, Hkv, S, D), 7.0, np.float32)
    vc = np.full((1, B, Hkv, S, D), 7.0, np.float32)
    out = ref.decode_attn(qkv, bias, kc, vc, Hq, 1, D, 10000.0).reshape(B, Hq, D)
    v = qkv[:, Hq + Hkv:] + bias[(Hq + Hkv) * D:].reshape(Hkv, D)
    np.testing.assert_array_equal(out, np.repeat(v, Hq // Hkv, axis=1))


def test_no_rotary_equals_torch_sdpa(ref):
    rng = np.random.default_rng(6)
    B, H, D, t, S = 2, 4, 64, 33, 40
    qkv = rng.standard_normal((B, 3 * H, D)).astype(np.float32)
    kc = rng.standard_normal((1, B, H, S, D)).astype(np.float32)
    vc = rng.standard_normal((1, B, H, S, D)).astype(np.float32)
    K = torch.from_numpy(kc[0, :, :, :t].copy()).double()
    V = torch.from_numpy(vc[0, :, :, :t].copy()).double()
    K[:, :, t - 1] = torch.from_numpy(qkv[:, H:2 * H]).double()
    V[:, :, t - 1] = torch.from_numpy(qkv[:, 2 * H:]).double()
    Q = torch.from_numpy(qkv[:, :H]).double().unsqueeze(2)
    want = torch.nn.functional.scaled_dot_product_attention(Q, K, V).squeeze(2).reshape(B, H * D).numpy()
    out = ref.decode_attn(qkv, None, kc, vc, H, t, 0, 10000.0)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-6)


def test_constant_v_rows_give_that_constant(ref):
    rng = np.random.default_rng(7)
    B, H, D, t, S = 1, 2, 16, 9, 16
    qkv = rng.standard_normal((B, 3 * H, D)).astype(np.float32)
    qkv[:, 2 * H:] = 0.25
    kc = rng.standard_normal((1, B, H, S, D)).astype(np.float32)
    vc = np.full((1, B, H, S, D), 0.25, np.float32)
    out = ref.decode_attn(qkv, None, kc, vc, H, t, D, 10000.0)
    np.testing.assert_allclose(out, 0.25, rtol=1e-6)


@pytest.mark.parametrize("dtype,Hq,Hkv,D,ragged", [
    (np.float32, 8, 8, 64, False),   # BASELINE config 1 shape
    (np.float32, 4, 2, 16, True),
    (np.float16, 8, 2, 32, True),
    (np.float16, 4, 4, 128, False),
    (np.float16, 6, 1, 16, True),    # multi-query
])
def test_against_float64_model(ref, dtype, Hq, Hkv, D, ragged):
    rng = np.random.default_rng(hash((Hq, Hkv, D)) % 2**31)
    B, S = 3, 24
    t = rng.integers(1, S + 1, size=B) if ragged else 17
    qkv = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * 0.5).astype(dtype)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(dtype)
    kc = (rng.standard_normal((1, B, Hkv, S, D)) * 0.5).astype(dtype)
    vc = (rng.standard_normal((1, B, Hkv, S, D)) * 0.5).astype(dtype)
    want, nk, nv = attn64(qkv, bias, kc.copy(), vc.copy(), Hq, t, D, 10000.0, store_dtype=dtype)
    out = ref.decode_attn(qkv, bias, kc, vc, Hq, t, D, 10000.0)
    tb = np.broadcast_to(np.asarray(t), (B,))
    if dtype == np.float32:
        np.testing.assert_allclose(out, want, rtol=1e-5, atol=2e-6)
    else:
        np.testing.assert_allclose(out.astype(np.float64), want, rtol=1e-2, atol=1e-3)
    for b in range(B):
        got_v = vc[0, b, :, tb[b] - 1].astype(np.float64)
        np.testing.assert_array_equal(got_v, nv[b])          # one fp add, one rounding: exact
        got_k = kc[0, b, :, tb[b] - 1].astype(np.float64)
        np.testing.assert_allclose(got_k, nk[b], rtol=2e-3 if dtype == np.float16 else 1e-5, atol=2e-6)


def test_pos_offset_minus_one_is_zero_based_position(ref):
    rng = np.random.default_rng(9)
    B, H, D, t, S = 1, 2, 32, 6, 8
    qkv = rng.standard_normal((B, 3 * H, D)).astype(np.float32)
    kc = rng.standard_normal((1, B, H, S, D)).astype(np.float32)
    vc = rng.standard_normal((1, B, H, S, D)).astype(np.float32)
    want, _, _ = attn64(qkv, None, kc.copy(), vc.copy(), H, t, D, 10000.0, pos_offset=-1)
    out = ref.decode_attn(qkv, None, kc, vc, H, t, D, 10000.0, rope_pos_offset=-1)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-6)


def test_no_cache_write_flag(ref):
    rng = np.random.default_rng(10)
    B, H, D, t, S = 2, 2, 16, 5, 8
    qkv = rng.standard_normal((B, 3 * H, D)).astype(np.float32)
    kc = rng.standard_normal((1, B, H, S, D)).astype(np.float32)
    vc = rng.standard_normal((1, B, H, S, D)).astype(np.float32)
    k0, v0 = kc.copy(), vc.copy()
    a = ref.decode_attn(qkv, None, kc, vc, H, t, D, 10000.0, flags=ref.ATTN_NO_CACHE_WRITE)
    np.testing.assert_array_equal(kc, k0)
    np.testing.assert_array_equal(vc, v0)
    b = ref.decode_attn(qkv, None, kc, vc, H, t, D, 10000.0)
    np.testing.assert_array_equal(a, b)


def test_rejects_bad_arguments(ref):
    qkv = np.zeros((1, 3, 8), np.float32)
    kc = np.zeros((1, 1, 1, 4, 8), np.float32)
    with pytest.raises(RuntimeError):
        ref.decode_attn(qkv, None, kc, kc.copy(), 1, 5, 8, 10000.0)   # t > S
    with pytest.raises(RuntimeError):
        ref.decode_attn(qkv, None, kc, kc.copy(), 1, 0, 8, 10000.0)   # t < 1
