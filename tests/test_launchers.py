"""The six launch* shims with oneLLM's own signatures, driven through a small C harness that builds
Tensor / BaseWeight / LayerNormWeight objects the way the oneLLM layers and unit tests do.
Host-side behaviour (carrier types, argument errors -> exceptions) runs without a GPU; the parity
checks against the CPU oracle are marked gpu."""
import ctypes
import math
import os

import numpy as np
import pytest

from conftest import announce

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "tests", "cpp", "liblauncher_harness.so")


@pytest.fixture(scope="module")
def H():
    assert os.path.exists(HARNESS), "build it with `python -m onellm_amd.build`"
    import torch  # noqa: F401  first, so that the HIP runtime torch ships is the one this process uses
    L = ctypes.CDLL(HARNESS)
    vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    L.h_last_error.restype = ctypes.c_char_p
    L.h_decode_mha.argtypes = [ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, ci, cf]
    L.h_rmsnorm.argtypes = [ci, vp, vp, ci, ci, cf]
    L.h_fused_norm.argtypes = [ci, vp, vp, vp, vp, ci, ci, cf]
    L.h_append.argtypes = [ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci]
    L.h_repeat.argtypes = [ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci]
    L.h_topk.argtypes = [vp, ci, ci, vp]
    L.h_prefill_rope.argtypes = [ci, vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, cf]
    L.h_act.argtypes = [ci, vp, vp, ci, ci]
    L.h_sampling.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci]
    L.h_set_launch_stream.argtypes = [vp]
    L.h_set_launch_stream.restype = None
    return L


# ---------------------------------------------------------------- host only

def test_carrier_types(H):
    assert H.h_type_tags() == 63
    assert H.h_tensor_size(2, 3, 4) == 24
    assert H.h_getval_requires_cpu_tensor() == 1          # getVal on a GPU tensor throws
    assert b"[oneLLM][ERROR]" in H.h_last_error()
    assert H.h_equality_and_status_checks() == 31         # Tensor == Tensor and CHECK_CUBLAS as the reference's


def test_tensor_map_and_layer_weight_views(H):
    assert H.h_tensor_map_checks() == 63
    assert b"missing" in H.h_last_error()
    assert H.h_layer_weight_checks(4, 2, 8, 12, 1) == 127
    assert H.h_layer_weight_checks(32, 8, 128, 11008, 0) == 127


def test_precondition_failures_throw_without_touching_the_gpu(H):
    fake = ctypes.c_void_p(0x1000)
    # step tensor on the GPU: the launcher must refuse to dereference it on the host
    assert H.h_decode_mha(0, fake, None, fake, fake, fake, 1, 2, 1, 16, 32, 1, 4, 1, 128, 10000.0) == 1
    assert b"step must be a host tensor" in H.h_last_error()
    # unsupported element type
    assert H.h_rmsnorm(5, fake, fake, 2, 32, 1e-5) == 1
    assert b"only FP32 and FP16" in H.h_last_error()
    # step beyond the cache
    assert H.h_decode_mha(0, fake, None, fake, fake, fake, 1, 2, 1, 16, 32, 1, 33, 0, 128, 10000.0) == 1
    assert b"step outside" in H.h_last_error()
    # a head size the kernels are not built for: rejected by the C ABI before any launch, surfaces as [TM][ERROR]
    assert H.h_decode_mha(0, fake, None, fake, fake, fake, 1, 2, 1, 600, 32, 1, 4, 0, 128, 10000.0) == 1
    assert b"[TM][ERROR] launchDecoderMaskedMHA" in H.h_last_error()
    assert H.h_topk(None, 1, 100, fake) == 1
    assert b"launchTopKforBeamSearch" in H.h_last_error()


# ---------------------------------------------------------------- GPU parity through the launchers

def _dev(a, dev):
    import torch
    return torch.from_numpy(a).to(dev)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,five_d", [(np.float32, True), (np.float32, False), (np.float16, True)])
def test_launchDecoderMaskedMHA(H, ref, dev, dtype, five_d):
    announce("launchDecoderMaskedMHA", dtype.__name__, five_d)
    rng = np.random.default_rng(1)
    B, Hq, Hkv, D, S, t = 2, 4, 2, 64, 48, 37
    L = 2 if five_d else 1
    qkv = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * 0.5).astype(dtype)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(dtype)
    kc = (rng.standard_normal((L, B, Hkv, S, D)) * 0.5).astype(dtype)
    vc = (rng.standard_normal((L, B, Hkv, S, D)) * 0.5).astype(dtype)
    import torch
    d = [_dev(a, dev) for a in (qkv, bias, kc, vc)]
    out = torch.zeros(B, Hq * D, dtype=d[0].dtype, device=dev)
    code = 1 if dtype == np.float16 else 0
    rc = H.h_decode_mha(code, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), out.data_ptr(),
                        B, Hq, Hkv, D, S, L if five_d else 0, t, 0, D, 10000.0)
    assert rc == 0, H.h_last_error()
    assert H.h_sync_and_check() == 0, H.h_last_error()
    want = ref.decode_attn(qkv, bias, kc, vc, Hq, t, D, 10000.0, layer=0)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == np.float32 else dict(rtol=1e-2, atol=2e-3)
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), **tol)
    it = np.uint32 if dtype == np.float32 else np.uint16
    np.testing.assert_array_equal(d[2].cpu().numpy().view(it), kc.view(it))
    np.testing.assert_array_equal(d[3].cpu().numpy().view(it), vc.view(it))


@pytest.mark.gpu
def test_launchDecoderMaskedMHA_with_a_sequence_split(H, ref, dev):
    """One or two sequences with a long history: the entry point splits the sequence, the launcher creates its
    zero-filled workspace and the pieces are merged inside the attention kernel.  Several steps of different lengths
    reuse that workspace."""
    import torch
    rng = np.random.default_rng(7)
    B, Hq, Hkv, D, S = 2, 8, 2, 128, 1100
    qkv = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * 0.5).astype(np.float16)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(np.float16)
    kc = (rng.standard_normal((1, B, Hkv, S, D)) * 0.5).astype(np.float16)
    vc = (rng.standard_normal((1, B, Hkv, S, D)) * 0.5).astype(np.float16)
    d_qkv, d_bias = _dev(qkv, dev), _dev(bias, dev)
    for t in (1000, 300, 1100, 129, 1000):
        announce("launchDecoderMaskedMHA split, step", t)
        d_kc, d_vc = _dev(kc, dev), _dev(vc, dev)
        out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
        rc = H.h_decode_mha(1, d_qkv.data_ptr(), d_bias.data_ptr(), d_kc.data_ptr(), d_vc.data_ptr(), out.data_ptr(),
                            B, Hq, Hkv, D, S, 1, t, 0, D, 10000.0)
        assert rc == 0, H.h_last_error()
        assert H.h_sync_and_check() == 0, H.h_last_error()
        r_kc, r_vc = kc.copy(), vc.copy()
        want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, t, D, 10000.0)
        np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), rtol=1e-2, atol=2e-3)
        np.testing.assert_array_equal(d_kc.cpu().numpy().view(np.uint16), r_kc.view(np.uint16))
        np.testing.assert_array_equal(d_vc.cpu().numpy().view(np.uint16), r_vc.view(np.uint16))


@pytest.mark.gpu
def test_launchRMSNorm_and_fused_norm(H, ref, dev):
    import torch
    announce("launchRMSNorm / launchFusedAddBiasResidualRMSNorm")
    # the reference unit-test vectors: 2 x 32 ones, eps 0.5
    x = torch.ones(2, 32, device=dev)
    g = torch.ones(32, device=dev)
    assert H.h_rmsnorm(0, x.data_ptr(), g.data_ptr(), 2, 32, 0.5) == 0, H.h_last_error()
    np.testing.assert_allclose(x.cpu().numpy(), 1 / math.sqrt(1.5), rtol=1e-6)
    rng = np.random.default_rng(2)
    for dtype, code in ((np.float32, 0), (np.float16, 1)):
        out = rng.standard_normal((9, 4096)).astype(dtype)
        res = rng.standard_normal((9, 4096)).astype(dtype)
        bias = rng.standard_normal(4096).astype(dtype)
        gam = rng.uniform(0.5, 1.5, 4096).astype(dtype)
        d = [_dev(a, dev) for a in (res, out, bias, gam)]
        assert H.h_fused_norm(code, d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), 9, 4096, 1e-5) == 0
        w_res, w_out = ref.fused_add_bias_residual_rmsnorm(res, out, bias, gam, 1e-5)
        it = np.uint32 if dtype == np.float32 else np.uint16
        np.testing.assert_array_equal(d[0].cpu().numpy().view(it), w_res.view(it))
        tol = dict(rtol=1e-5, atol=1e-6) if dtype == np.float32 else dict(rtol=1e-2, atol=2e-3)
        np.testing.assert_allclose(d[1].cpu().numpy().astype(np.float64), w_out.astype(np.float64), **tol)
    assert H.h_sync_and_check() == 0


@pytest.mark.gpu
def test_launchAppendKVCache_and_launchTransposeKVCache(H, ref, dev):
    import torch
    announce("launchAppendKVCache / launchTransposeKVCache")
    rng = np.random.default_rng(3)
    L, B, Hq, Hkv, Q, S, D, MK = 2, 3, 8, 2, 5, 24, 16, 20
    ks = rng.standard_normal((B, Hkv, Q, D)).astype(np.float32)
    vs = rng.standard_normal((B, Hkv, Q, D)).astype(np.float32)
    kc = rng.standard_normal((L, B, Hkv, S, D)).astype(np.float32)
    vc = rng.standard_normal((L, B, Hkv, S, D)).astype(np.float32)
    cur = np.array([5, 2, 0], np.int32)
    hist = np.array([3, 19, 7], np.int32)
    d = [_dev(a, dev) for a in (ks, vs, kc, vc, cur, hist)]
    assert H.h_append(0, *[t.data_ptr() for t in d], B, Hkv, Q, S, D, L, 1) == 0, H.h_last_error()
    ref.kv_append(ks, vs, kc, vc, cur, hist, layer=1)
    np.testing.assert_array_equal(d[2].cpu().numpy().view(np.uint32), kc.view(np.uint32))
    np.testing.assert_array_equal(d[3].cpu().numpy().view(np.uint32), vc.view(np.uint32))
    ctx = (hist + cur).astype(np.int32)
    kd = np.full((B, Hq, MK, D), 9.0, np.float32)
    vd = np.full((B, Hq, MK, D), 9.0, np.float32)
    e = [_dev(a, dev) for a in (kd, vd, ctx)]
    assert H.h_repeat(0, d[2].data_ptr(), d[3].data_ptr(), e[0].data_ptr(), e[1].data_ptr(), e[2].data_ptr(),
                      B, Hq, Hkv, S, MK, D, L, 1) == 0, H.h_last_error()
    ref.kv_repeat(kc, vc, kd, vd, ctx, layer=1)
    np.testing.assert_array_equal(e[0].cpu().numpy().view(np.uint32), kd.view(np.uint32))
    np.testing.assert_array_equal(e[1].cpu().numpy().view(np.uint32), vd.view(np.uint32))
    assert H.h_sync_and_check() == 0


@pytest.mark.gpu
def test_launchTopKforBeamSearch_reference_layout(H, ref, dev):
    import torch
    announce("launchTopKforBeamSearch")
    B, V = 3, 30000
    rng = np.random.default_rng(4)
    logits = rng.integers(-50, 50, size=(B * 2, V)).astype(np.float32)
    ws = torch.zeros(2 * B * 2 + 2 * B * 2 * 8 * 2, dtype=torch.float32, device=dev)     # the reference test's size
    assert H.h_topk(_dev(logits, dev).data_ptr(), B, V, ws.data_ptr()) == 0, H.h_last_error()
    assert H.h_sync_and_check() == 0
    w = ws.cpu().numpy()
    off = 2 * B * 2 * 8 * 2                                                              # where the reference test reads
    _, _, wfv, wfi = ref.beam_topk(logits, B, 2, 2)
    np.testing.assert_array_equal(w[off:off + B * 2].reshape(B, 2), wfv)
    np.testing.assert_array_equal(w.view(np.int32)[off + B * 2:off + 2 * B * 2].reshape(B, 2), wfi)


@pytest.mark.gpu
def test_launchAddFusedQKVBiasTransposeAndRoPE_and_launchAct(H, ref, dev):
    import torch
    announce("launchAddFusedQKVBiasTransposeAndRoPE / launchAct")
    rng = np.random.default_rng(6)
    B, S, Hq, Hkv, D = 2, 16, 4, 2, 64
    lens = [16, 9]
    T = sum(lens)
    po = np.array([0] * 16 + [16 + s - (16 + s) + 0 for s in range(9)], np.int32)    # packed: second sequence starts at token 16 = slot 16
    hist = np.array([3, 100], np.int32)
    qkv = rng.standard_normal((T, Hq + 2 * Hkv, D)).astype(np.float32)
    bias = rng.standard_normal((Hq + 2 * Hkv) * D).astype(np.float32)
    q = np.zeros((B, Hq, S, D), np.float32); k = np.zeros((B, Hkv, S, D), np.float32); v = np.zeros_like(k)
    d = [_dev(a, dev) for a in (q, k, v, qkv, bias, po, hist, np.array(lens, np.int32))]
    assert H.h_prefill_rope(0, *[t.data_ptr() for t in d], B, S, T, Hq, Hkv, D, D, 10000.0) == 0, H.h_last_error()
    ref.qkv_bias_rope_transpose(q, k, v, qkv, bias, po, hist, D, 10000.0)
    for got, want in zip(d[:3], (q, k, v)):
        np.testing.assert_array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    for dtype, code in ((np.float32, 0), (np.float16, 1)):
        inp = (rng.standard_normal((5, 2, 11008)) * 2).astype(dtype)
        out = torch.zeros(5, 11008, dtype=torch.float32 if code == 0 else torch.float16, device=dev)
        assert H.h_act(code, _dev(inp, dev).data_ptr(), out.data_ptr(), 5, 11008) == 0, H.h_last_error()
        want = ref.silu_and_mul(inp, np.zeros((5, 11008), dtype))
        tol = dict(rtol=1e-5, atol=1e-6) if code == 0 else dict(rtol=1e-2, atol=2e-3)
        np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), **tol)
    assert H.h_sync_and_check() == 0


@pytest.mark.gpu
def test_launchSampling(H, ref, dev):
    import torch
    announce("launchSampling")
    # the reference unit test's inputs: B3, K3, ids 0..8, vals 2,1,0, seqlen 4, step 5, end_id 10, vocab 1000
    B, K = 3, 3
    ids = np.arange(B * K, dtype=np.int32).reshape(B, K)
    vals = np.tile(np.array([2.0, 1.0, 0.0], np.float32), (B, 1))
    seqlen = np.full(B, 4, np.int32)
    fin = np.zeros(B, np.uint8)
    d = [_dev(a, dev) for a in (ids, vals, seqlen, fin)]
    out = torch.zeros(B, dtype=torch.int32, device=dev)
    assert H.h_sampling(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), out.data_ptr(), B, K, 5, 10, 1000) == 0, H.h_last_error()
    assert H.h_sync_and_check() == 0
    want = ref.topk_sample(ids, vals, seqlen, fin, 5, 10, 1000)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    np.testing.assert_array_equal(d[2].cpu().numpy(), seqlen)
    np.testing.assert_array_equal(d[3].cpu().numpy(), fin)


@pytest.mark.gpu
def test_every_launcher_queues_on_the_launch_stream(H, dev):
    """onellmSetLaunchStream names the stream of the calling thread's launches.  All nine launchers are captured into
    one HIP graph on a side stream (a launch that went to the null stream instead would be refused during capture or be
    missing from the graph); the replay must reproduce what the same calls produce eagerly, bit for bit."""
    import torch
    announce("launchers under graph capture on a side stream")
    torch.manual_seed(3)
    B, Hq, Hkv, D, S, t, H_, I, V, K = 2, 8, 2, 128, 96, 70, 1024, 512, 4000, 4
    G = Hq // Hkv
    h = lambda *s: torch.randn(*s, device=dev).mul(0.5).half()
    qkv, bias = h(B, Hq + 2 * Hkv, D), h((Hq + 2 * Hkv) * D)
    kc0, vc0 = h(1, B, Hkv, S, D), h(1, B, Hkv, S, D)
    x0, res0, gam, nb = h(B, H_), h(B, H_), torch.rand(H_, device=dev).add(0.5).half(), h(H_)
    ks, vs = h(B, Hkv, 1, D), h(B, Hkv, 1, D)
    cur = torch.ones(B, dtype=torch.int32, device=dev)
    hist = torch.full((B,), t, dtype=torch.int32, device=dev)
    ctx = torch.full((B,), t + 1, dtype=torch.int32, device=dev)
    pair = h(B, 2, I)
    logits = torch.randn(B * 2, V, device=dev)
    pq, pk, pv = (torch.zeros(B, n, 4, D, dtype=torch.float16, device=dev) for n in (Hq, Hkv, Hkv))
    pqkv = h(B * 4, Hq + 2 * Hkv, D)
    pad = torch.zeros(B * 4, dtype=torch.int32, device=dev)
    zeros_b = torch.zeros(B, dtype=torch.int32, device=dev)
    four_b = torch.full((B,), 4, dtype=torch.int32, device=dev)
    tid = torch.randint(0, V, (B, K), dtype=torch.int32, device=dev)
    tval = torch.rand(B, K, device=dev)

    kc, vc, x, res = kc0.clone(), vc0.clone(), x0.clone(), res0.clone()
    out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    rk, rv = (torch.zeros(B, Hq, S, D, dtype=torch.float16, device=dev) for _ in range(2))
    act = torch.zeros(B, I, dtype=torch.float16, device=dev)
    tws = torch.zeros((2 * B * 2 * 8 * 2 + 2 * B * 2), dtype=torch.float32, device=dev)
    seqlen, fin, sampled = zeros_b.clone(), torch.zeros(B, dtype=torch.uint8, device=dev), zeros_b.clone()
    state = (kc, vc, x, res, out, rk, rv, act, tws, pq, pk, pv, seqlen, fin, sampled)

    def restore():
        kc.copy_(kc0); vc.copy_(vc0); x.copy_(x0); res.copy_(res0)
        for a in (out, rk, rv, act, tws, pq, pk, pv, seqlen, fin, sampled):
            a.zero_()

    def calls():
        p = lambda a: a.data_ptr()
        ok = [H.h_rmsnorm(1, p(x), p(gam), B, H_, 1e-5),
              H.h_decode_mha(1, p(qkv), p(bias), p(kc), p(vc), p(out), B, Hq, Hkv, D, S, 1, t, 0, D, 10000.0),
              H.h_fused_norm(1, p(res), p(x), p(nb), p(gam), B, H_, 1e-5),
              H.h_append(1, p(ks), p(vs), p(kc), p(vc), p(cur), p(hist), B, Hkv, 1, S, D, 1, 0),
              H.h_repeat(1, p(kc), p(vc), p(rk), p(rv), p(ctx), B, Hq, Hkv, S, S, D, 1, 0),
              H.h_act(1, p(pair), p(act), B, I),
              H.h_topk(p(logits), B, V, p(tws)),
              H.h_prefill_rope(1, p(pq), p(pk), p(pv), p(pqkv), p(bias), p(pad), p(zeros_b), p(four_b), B, 4, B * 4, Hq, Hkv, D, D, 10000.0),
              H.h_sampling(p(tid), p(tval), p(seqlen), p(fin), p(sampled), B, K, 5, 10, V)]
        assert ok == [0] * 9, ok

    restore()
    calls()                                      # eager, null stream
    torch.cuda.synchronize()
    want = [a.clone() for a in state]

    side = torch.cuda.Stream()
    H.h_set_launch_stream(side.cuda_stream)
    try:
        restore()
        torch.cuda.synchronize()
        calls()                                  # eager on the side stream (also creates the attention workspace if needed)
        torch.cuda.synchronize()
        for a, b in zip(state, want):
            assert torch.equal(a, b)
        restore()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            calls()
        for replay in range(3):
            restore()
            x0.float().sum().item()
            g.replay()
            torch.cuda.synchronize()
            for i, (a, b) in enumerate(zip(state, want)):
                assert torch.equal(a, b), f"replay {replay}: buffer {i} differs from the eager result"
    finally:
        H.h_set_launch_stream(None)


@pytest.mark.gpu
def test_first_split_step_on_a_capturing_stream_is_refused(H, dev):
    """The attention launcher owns a workspace per launch stream and creates it (allocation, clear) when a step first
    needs one.  That must not happen while the stream is being captured: the launcher throws, nothing is recorded or
    launched, and the same step runs normally once the capture is over."""
    import torch
    announce("launchDecoderMaskedMHA first split step under capture")
    torch.manual_seed(8)
    B, Hq, Hkv, D, S, t = 1, 8, 2, 128, 2048, 2000            # one sequence, two kv heads: split into pieces
    h = lambda *s: torch.randn(*s, device=dev).mul(0.5).half()
    qkv, bias, kc, vc = h(B, Hq + 2 * Hkv, D), h((Hq + 2 * Hkv) * D), h(1, B, Hkv, S, D), h(1, B, Hkv, S, D)
    out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    p = lambda a: a.data_ptr()
    call = lambda: H.h_decode_mha(1, p(qkv), p(bias), p(kc), p(vc), p(out), B, Hq, Hkv, D, S, 1, t, 0, D, 10000.0)
    side = torch.cuda.Stream()                                 # a stream no launcher has seen
    H.h_set_launch_stream(side.cuda_stream)
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            qkv.add_(0)                                        # (something for the graph to hold)
            rc = call()
            msg = H.h_last_error()
        assert rc == 1 and b"captured" in msg, msg
        torch.cuda.synchronize()
        assert not out.any()
        assert call() == 0, H.h_last_error()                   # outside a capture the workspace is created
        torch.cuda.synchronize()
        assert out.any()
    finally:
        H.h_set_launch_stream(None)
