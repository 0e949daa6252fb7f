"""GPU parity of the prefill QKV-bias+RoPE+transpose and SwiGLU kernels against the CPU oracle, through
the C ABI.  The prefill outputs are bit-exact (same fixed fp32 operation sequence on both sides);
SwiGLU: fp32 1e-5 relative, fp16 2e-3 absolute / 1e-2 relative (exp differs by an ulp between libm and
the GPU)."""
import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


def _bits(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def _pack(B, seq_len, lens):
    po, tok = [], 0
    for b, n in enumerate(lens):
        for s in range(n):
            po.append(b * seq_len + s - tok)
            tok += 1
    return np.array(po, np.int32)


@pytest.mark.parametrize("dtype,Hq,Hkv,D,rd", [(np.float32, 2, 1, 8, 128), (np.float16, 32, 32, 128, 128),
                                               (np.float16, 32, 8, 128, 64), (np.float32, 4, 2, 64, 64),
                                               (np.float16, 4, 4, 12, 12), (np.float32, 3, 1, 6, 6),
                                               (np.float16, 5, 1, 8, 8), (np.float16, 6, 2, 16, 6), (np.float16, 3, 3, 32, 32),
                                               (np.float16, 40, 8, 64, 32), (np.float16, 9, 3, 256, 256), (np.float16, 2, 1, 512, 100),
                                               (np.float32, 7, 7, 4, 4), (np.float32, 3, 1, 128, 128), (np.float32, 2, 2, 256, 254)])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("kernel", ["rows", "index"])
def test_prefill_matches_oracle(capi, ref, dev, dtype, Hq, Hkv, D, rd, with_bias, kernel):
    # "rows": the kernel whose threads keep one (token, piece) and walk the heads (rows of a power-of-two number of
    # 16-byte pieces); "index": the general kernel, forced for every shape
    announce("prefill rope", dtype.__name__, Hq, Hkv, D, rd, with_bias, kernel)
    capi.tune_set("prefill_generic", 1 if kernel == "index" else -1)
    rng = np.random.default_rng(Hq * 100 + D)
    B, S = 4, 40
    lens = [40, 17, 1, 0]
    hist = np.array([0, 23, 4000, 5], np.int32)
    T = sum(lens)
    qkv = (rng.standard_normal((T, Hq + 2 * Hkv, D)) * 0.5).astype(dtype)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(dtype) if with_bias else None
    po = _pack(B, S, lens)
    q = np.full((B, Hq, S, D), 9.0, dtype)
    k = np.full((B, Hkv, S, D), 9.0, dtype)
    v = np.full((B, Hkv, S, D), 9.0, dtype)
    d = [torch.from_numpy(x).to(dev) for x in (q, k, v, qkv)]
    d_bias = torch.from_numpy(bias).to(dev) if with_bias else None
    capi.qkv_bias_rope_transpose(d[0], d[1], d[2], d[3], d_bias, torch.from_numpy(po).to(dev), torch.from_numpy(hist).to(dev),
                                 rd, 10000.0)
    capi.tune_set("prefill_generic", -1)
    ref.qkv_bias_rope_transpose(q, k, v, qkv, bias, po, hist, rd, 10000.0)
    for got, want in zip(d[:3], (q, k, v)):
        np.testing.assert_array_equal(_bits(got.cpu().numpy()), _bits(want))


def test_prefill_reference_unit_vector(capi, ref, dev):
    announce("prefill rope unit vector")
    qkv = torch.ones(32, 4, 8, device=dev)
    bias = torch.full((32,), 2.0, device=dev)
    q = torch.zeros(1, 2, 32, 8, device=dev)
    k = torch.zeros(1, 1, 32, 8, device=dev)
    v = torch.zeros(1, 1, 32, 8, device=dev)
    capi.qkv_bias_rope_transpose(q, k, v, qkv, bias, torch.zeros(32, dtype=torch.int32, device=dev),
                                 torch.tensor([4], dtype=torch.int32, device=dev), 128, 10000.0)
    assert torch.equal(v, torch.full_like(v, 3.0))
    # a rotation keeps each pair's length: (3, 3) -> 18
    qq = q.cpu().numpy()
    np.testing.assert_allclose(qq[..., 0::2] ** 2 + qq[..., 1::2] ** 2, 18.0, rtol=1e-6)
    assert torch.equal(q[0, 0], k[0, 0]) and torch.equal(q[0, 0], q[0, 1])


def test_prefill_feeds_decode(capi, ref, dev):
    # prefill 300 tokens with the kernel, append its K/V to the cache, run one decode step with
    # rope_pos_offset = -1, compare with the oracle doing the same three steps
    announce("prefill -> append -> decode")
    rng = np.random.default_rng(12)
    B, Hq, Hkv, D, S, n = 2, 8, 2, 128, 512, 300
    qkv = (rng.standard_normal((B * n, Hq + 2 * Hkv, D)) * 0.5).astype(np.float16)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(np.float16)
    po = np.zeros(B * n, np.int32)
    hist0 = np.zeros(B, np.int32)
    nxt = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * 0.5).astype(np.float16)
    # oracle
    rq = np.zeros((B, Hq, n, D), np.float16); rk = np.zeros((B, Hkv, n, D), np.float16); rv = np.zeros_like(rk)
    ref.qkv_bias_rope_transpose(rq, rk, rv, qkv, bias, po, hist0, D, 10000.0)
    rkc = np.zeros((1, B, Hkv, S, D), np.float16); rvc = np.zeros_like(rkc)
    ref.kv_append(rk, rv, rkc, rvc, np.full(B, n, np.int32), hist0)
    want = ref.decode_attn(nxt, bias, rkc, rvc, Hq, n + 1, D, 10000.0, rope_pos_offset=-1)
    # GPU
    t = lambda a: torch.from_numpy(a).to(dev)
    gq = torch.zeros(B, Hq, n, D, dtype=torch.float16, device=dev); gk = torch.zeros(B, Hkv, n, D, dtype=torch.float16, device=dev)
    gv = torch.zeros_like(gk)
    capi.qkv_bias_rope_transpose(gq, gk, gv, t(qkv), t(bias), t(po), t(hist0), D, 10000.0)
    gkc = torch.zeros(1, B, Hkv, S, D, dtype=torch.float16, device=dev); gvc = torch.zeros_like(gkc)
    capi.kv_append(gk, gv, gkc, gvc, t(np.full(B, n, np.int32)), t(hist0))
    out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    capi.decode_attn(t(nxt), t(bias), gkc, gvc, out, Hq, n + 1, D, 10000.0, rope_pos_offset=-1)
    np.testing.assert_array_equal(_bits(gkc.cpu().numpy()), _bits(rkc))
    np.testing.assert_array_equal(_bits(gvc.cpu().numpy()), _bits(rvc))
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), rtol=1e-2, atol=2e-3)


@pytest.mark.parametrize("dtype,B,I", [(np.float32, 16, 11008), (np.float16, 16, 11008), (np.float16, 3, 100),
                                       (np.float32, 2, 7), (np.float16, 512, 11008)])
def test_swiglu_matches_oracle(capi, ref, dev, dtype, B, I):
    announce("swiglu", dtype.__name__, B, I)
    rng = np.random.default_rng(B + I)
    inp = (rng.standard_normal((B, 2, I)) * 3).astype(dtype)
    out = torch.zeros(B, I, dtype=torch.float16 if dtype == np.float16 else torch.float32, device=dev)
    capi.silu_and_mul(torch.from_numpy(inp).to(dev), out)
    want = ref.silu_and_mul(inp, np.zeros((B, I), dtype))
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == np.float32 else dict(rtol=1e-2, atol=2e-3)
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), **tol)


def test_swiglu_reference_unit_vector(capi, dev):
    # tests/unittests/test_activation.cu:41-47 of the reference: input[i] = i; silu(x) = x for large x
    announce("swiglu unit vector")
    B, I = 16, 11008
    inp = torch.arange(B * 2 * I, dtype=torch.float32, device=dev).view(B, 2, I)
    out = torch.zeros(B, I, device=dev)
    capi.silu_and_mul(inp, out)
    x, y = inp[:, 0].double(), inp[:, 1].double()
    want = x / (1 + torch.exp(-x)) * y
    assert ((out.double() - want).abs() <= 1e-6 * want.abs() + 1e-6).all()


def test_sampling_matches_oracle_bit_for_bit(capi, ref, dev):
    announce("topk sampling")
    rng = np.random.default_rng(13)
    for (B, K, vocab, seed) in ((3, 3, 1000, 5), (1000, 4, 32000, 987654321098), (65, 8, 50, 0), (1, 1, 7, 42)):
        vals = np.sort(rng.standard_normal((B, K)).astype(np.float32) * 3, axis=1)[:, ::-1].copy()
        ids = rng.integers(0, 4 * vocab, size=(B, K)).astype(np.int32)
        seqlen = rng.integers(0, 100, B).astype(np.int32)
        fin = rng.integers(0, 2, B).astype(np.uint8)
        end_id = int(ids[0, 0] % vocab)
        d_out = torch.zeros(B, dtype=torch.int32, device=dev)
        d_seq, d_fin = torch.from_numpy(seqlen).to(dev), torch.from_numpy(fin).to(dev)
        capi.topk_sample(torch.from_numpy(ids).to(dev), torch.from_numpy(vals).to(dev), d_out, d_seq, d_fin, seed, end_id, vocab)
        want = ref.topk_sample(ids, vals, seqlen, fin, seed, end_id, vocab)
        np.testing.assert_array_equal(d_out.cpu().numpy(), want)
        np.testing.assert_array_equal(d_seq.cpu().numpy(), seqlen)
        np.testing.assert_array_equal(d_fin.cpu().numpy(), fin)


def test_topk_then_sampling_pipeline(capi, ref, dev):
    # beam top-K feeds sampling: final (val, id) pairs of each batch entry -> one token per entry
    announce("topk -> sampling")
    rng = np.random.default_rng(14)
    B, beam, V, K = 8, 4, 32000, 4
    logits = (rng.standard_normal((B * beam, V)) * 2).astype(np.float32)
    _, _, _, fv, fi = capi.beam_topk(torch.from_numpy(logits).to(dev), B, beam, K)
    out = torch.zeros(B, dtype=torch.int32, device=dev)
    seq = torch.zeros(B, dtype=torch.int32, device=dev)
    fin = torch.zeros(B, dtype=torch.uint8, device=dev)
    capi.topk_sample(fi.contiguous(), fv.contiguous(), out, seq, fin, 77, 2, V)
    _, _, wfv, wfi = ref.beam_topk(logits, B, beam, K)
    want = ref.topk_sample(wfi, wfv, np.zeros(B, np.int32), np.zeros(B, np.uint8), 77, 2, V)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    assert (out.cpu().numpy() < V).all() and (seq.cpu().numpy() == 1).all()
