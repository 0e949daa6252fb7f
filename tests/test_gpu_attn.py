"""GPU parity of the fused decode attention against the CPU oracle, through the C ABI.

Tolerances (written once, used everywhere): fp32 outputs 1e-5 relative (plus 1e-6 absolute for
values that cancel to near zero); fp16 outputs 2e-3 absolute / 1e-2 relative.  The cache row the
step writes is compared bit for bit: v is one fp32 add rounded once, k goes through the same fixed
sequence of fp32 operations on both sides."""
import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

TOL = {np.float32: dict(rtol=1e-5, atol=1e-6), np.float16: dict(rtol=1e-2, atol=2e-3)}


def _bits(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def _case(dtype, B, Hq, Hkv, D, S, L, seed, std=1.0):
    rng = np.random.default_rng(seed)
    qkv = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * std).astype(dtype)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * std).astype(dtype)
    kc = (rng.standard_normal((L, B, Hkv, S, D)) * std).astype(dtype)
    vc = (rng.standard_normal((L, B, Hkv, S, D)) * std).astype(dtype)
    return qkv, bias, kc, vc


def _run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, rotary_dim, base=10000.0, layer=0, pos_offset=0, flags=0):
    """Runs GPU and oracle on the same inputs; returns (gpu_out, ref_out, gpu_kc, gpu_vc, ref_kc, ref_vc)."""
    d_qkv = torch.from_numpy(qkv).to(dev)
    d_bias = torch.from_numpy(bias).to(dev) if bias is not None else None
    d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
    B, _, D = qkv.shape
    d_out = torch.zeros(B, Hq * D, dtype=d_qkv.dtype, device=dev)
    if isinstance(t, np.ndarray):
        t_dev = torch.from_numpy(t.astype(np.int32)).to(dev)
        capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, d_out, Hq, int(t.max()), rotary_dim, base, layer=layer,
                         t_dev=t_dev, max_t=int(t.max()), rope_pos_offset=pos_offset, flags=flags)
    else:
        capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, d_out, Hq, t, rotary_dim, base, layer=layer,
                         rope_pos_offset=pos_offset, flags=flags)
    r_kc, r_vc = kc.copy(), vc.copy()
    r_out = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, t, rotary_dim, base, layer=layer, rope_pos_offset=pos_offset,
                            flags=flags)
    return d_out.cpu().numpy(), r_out, d_kc.cpu().numpy(), d_vc.cpu().numpy(), r_kc, r_vc


def _assert_parity(res, dtype):
    g_out, r_out, g_kc, g_vc, r_kc, r_vc = res
    np.testing.assert_allclose(g_out.astype(np.float64), r_out.astype(np.float64), **TOL[dtype])
    np.testing.assert_array_equal(_bits(g_kc), _bits(r_kc))      # whole cache, including the new row
    np.testing.assert_array_equal(_bits(g_vc), _bits(r_vc))


def test_config1_fp32_small(capi, ref, dev):
    # BASELINE config 1: fp32, B1, 8 heads x 64, 16 cached steps + the current token, rotary 64, seed 0
    announce("attn config1")
    qkv, bias, kc, vc = _case(np.float32, 1, 8, 8, 64, 32, 1, seed=0)
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 8, 17, 64), np.float32)


def test_reference_unit_test_shape(capi, ref, dev):
    # tests/unittests/test_decoder_masked_attn.cu:113-176 of the reference: B1 Hq2 Hkv1 D16 step4
    announce("attn unit-test shape")
    B, Hq, Hkv, D, t, S = 1, 2, 1, 16, 4, 32
    qkv = np.ones((B, Hq + 2 * Hkv, D), np.float32)
    bias = np.full(((Hq + 2 * Hkv) * D,), 2.0, np.float32)
    kc = np.zeros((1, B, Hkv, S, D), np.float32)
    vc = np.zeros((1, B, Hkv, S, D), np.float32)
    kc[:, :, :, :t] = 1.0
    vc[:, :, :, :t] = 1.0
    res = _run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, 128, flags=capi.ATTN_NO_V_BIAS)
    _assert_parity(res, np.float32)
    np.testing.assert_allclose(res[0], 1.0, rtol=1e-6)            # all V rows are 1
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, 128), np.float32)


def test_example_driver_shape_two_layers(capi, ref, dev):
    # examples/cpp/decoder/self_decoder_example.cpp:10-27: Hq4 Hkv2 D8 B2 step3 max_seq12 rotary 128
    announce("attn example driver shape")
    qkv, bias, kc, vc = _case(np.float32, 2, 4, 2, 8, 12, 2, seed=3)
    for layer in (0, 1):
        _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 3, 128, layer=layer), np.float32)


@pytest.mark.parametrize("dtype,Hq,Hkv,D", [
    (np.float16, 4, 4, 128), (np.float16, 8, 2, 128), (np.float16, 8, 1, 64), (np.float16, 6, 3, 32),
    (np.float16, 16, 2, 128), (np.float16, 14, 2, 128), (np.float16, 16, 1, 128), (np.float16, 40, 2, 128),
    (np.float16, 3, 1, 128), (np.float16, 12, 2, 256), (np.float16, 2, 2, 8), (np.float16, 4, 2, 16), (np.float16, 2, 1, 512),
    (np.float32, 4, 4, 128), (np.float32, 8, 2, 64), (np.float32, 3, 1, 32), (np.float32, 2, 2, 256),
    (np.float32, 4, 1, 4), (np.float32, 10, 2, 16), (np.float32, 16, 2, 128), (np.float32, 12, 1, 128), (np.float32, 40, 2, 128),
    # rows of 10, 12, 20, 24, 40 or 48 16-byte pieces: the tiled kernel with idle lanes in every row group
    (np.float16, 4, 2, 96), (np.float16, 8, 8, 80), (np.float16, 6, 2, 160), (np.float16, 4, 1, 192), (np.float16, 2, 2, 320),
    (np.float16, 3, 1, 384), (np.float32, 4, 2, 40), (np.float32, 5, 5, 48), (np.float32, 8, 2, 80), (np.float32, 2, 1, 96),
    (np.float32, 2, 2, 160), (np.float32, 6, 1, 192),
])
@pytest.mark.parametrize("t", [1, 2, 63, 64, 65, 300])
def test_shapes_and_lengths(capi, ref, dev, dtype, Hq, Hkv, D, t):
    announce("attn", dtype.__name__, Hq, Hkv, D, "t", t)
    qkv, bias, kc, vc = _case(dtype, 3, Hq, Hkv, D, 304, 1, seed=Hq * 1000 + D + t, std=0.5)
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, D), dtype)


@pytest.mark.parametrize("dtype,Hq,Hkv,D", [(np.float16, 4, 2, 72), (np.float16, 8, 8, 100), (np.float32, 2, 1, 7),
                                            (np.float32, 3, 3, 100), (np.float16, 2, 1, 2), (np.float32, 2, 2, 1),
                                            (np.float16, 2, 1, 500), (np.float16, 2, 2, 112)])
@pytest.mark.parametrize("t", [1, 2, 70])
def test_head_sizes_outside_the_tiled_kernels(capi, ref, dev, dtype, Hq, Hkv, D, t):
    # rows the tiled kernels are not built for (not a whole number of 16-byte pieces, or a piece count outside
    # their list) run the scalar kernel: same parity bars
    announce("attn generic", dtype.__name__, Hq, Hkv, D, "t", t)
    qkv, bias, kc, vc = _case(dtype, 2, Hq, Hkv, D, 72, 2, seed=D * 7 + t, std=0.5)
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, D, layer=1), dtype)
    lens = np.array([t, max(1, t // 2)])
    _assert_parity(_run_both(capi, ref, dev, qkv, None, kc, vc, Hq, lens, D - D % 2), dtype)


def test_unaligned_cache_takes_the_scalar_kernel(capi, ref, dev):
    announce("attn unaligned cache")
    qkv, bias, kc, vc = _case(np.float16, 2, 4, 2, 64, 40, 1, seed=77, std=0.5)
    d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
    n = kc.size
    kbuf = torch.zeros(n + 8, dtype=torch.float16, device=dev)
    vbuf = torch.zeros(n + 8, dtype=torch.float16, device=dev)
    d_kc, d_vc = kbuf[1:1 + n].view(kc.shape), vbuf[1:1 + n].view(vc.shape)      # 2 bytes off a 16-byte boundary
    d_kc.copy_(torch.from_numpy(kc)); d_vc.copy_(torch.from_numpy(vc))
    out = torch.zeros(2, 4 * 64, dtype=torch.float16, device=dev)
    rc = capi.lib().onellm_decode_attn(capi.FP16, d_qkv.data_ptr(), d_bias.data_ptr(), d_kc.data_ptr(), d_vc.data_ptr(),
                                       out.data_ptr(), 2, 4, 2, 64, 40, 0, 1, 33, None, 33, 64, 10000.0, 0, 0, None, 0,
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    want = ref.decode_attn(qkv, bias, kc, vc, 4, 33, 64, 10000.0)
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL[np.float16])
    np.testing.assert_array_equal(_bits(d_kc.cpu().numpy()), _bits(kc))
    np.testing.assert_array_equal(_bits(d_vc.cpu().numpy()), _bits(vc))
    assert kbuf[0].item() == 0 and kbuf[n + 1].item() == 0


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("nsplit", [1, 2, 5, 64])
def test_sequence_split_counts_and_ragged_lengths(capi, ref, dev, dtype, nsplit):
    announce("attn ragged", dtype.__name__, "nsplit", nsplit)
    B, Hq, Hkv, D, S = 6, 8, 2, 128 if dtype == np.float16 else 64, 1100
    qkv, bias, kc, vc = _case(dtype, B, Hq, Hkv, D, S, 1, seed=11 + nsplit, std=0.5)
    t = np.array([1, 1100, 64, 513, 2, 777])
    capi.tune_set("attn_nsplit", nsplit)
    try:
        _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, D), dtype)
        if dtype == np.float16:
            # 7 query heads per kv head: the 8-head matrix-core tile with one head of padding
            qkv7, bias7, kc7, vc7 = _case(dtype, B, 14, 2, D, S, 1, seed=31 + nsplit, std=0.5)
            _assert_parity(_run_both(capi, ref, dev, qkv7, bias7, kc7, vc7, 14, t, D), dtype)
    finally:
        capi.tune_set("attn_nsplit", -1)


def test_options(capi, ref, dev):
    announce("attn options")
    qkv, bias, kc, vc = _case(np.float16, 2, 4, 2, 64, 40, 1, seed=21, std=0.5)
    _assert_parity(_run_both(capi, ref, dev, qkv, None, kc, vc, 4, 33, 64), np.float16)               # no bias
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 33, 0), np.float16)                # no rotation
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 33, 32), np.float16)               # partial rotation
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 33, 64, pos_offset=-1), np.float16)
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 33, 64, base=500000.0), np.float16)
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 33, 64, flags=capi.ATTN_NO_V_BIAS), np.float16)
    res = _run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 33, 64, flags=capi.ATTN_NO_CACHE_WRITE)
    _assert_parity(res, np.float16)
    np.testing.assert_array_equal(_bits(res[2]), _bits(kc))                                          # untouched
    _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, 4, 40, 64), np.float16)               # t == S


def test_config2_llama7b_full_size(capi, ref, dev):
    # BASELINE config 2: fp16, B16, 32 x 128, cache [1,16,32,4096,128] ~ N(0,0.5); contexts 512..4096
    torch.manual_seed(2)
    B, H, D, S = 16, 32, 128, 4096
    d_kc = torch.randn(1, B, H, S, D, device=dev).mul_(0.5).half()
    d_vc = torch.randn(1, B, H, S, D, device=dev).mul_(0.5).half()
    d_qkv = torch.randn(B, 3 * H, D, device=dev).mul_(0.5).half()
    d_bias = torch.randn(3 * H * D, device=dev).mul_(0.5).half()
    kc, vc = d_kc.cpu().numpy(), d_vc.cpu().numpy()
    qkv, bias = d_qkv.cpu().numpy(), d_bias.cpu().numpy()
    ws = torch.empty(capi.decode_attn_workspace_bytes(B, H, H, D, S), dtype=torch.uint8, device=dev)
    for t in (512, 1024, 2048, 4096):
        announce("attn config2 t", t)
        g_kc, g_vc = d_kc.clone(), d_vc.clone()
        out = torch.zeros(B, H * D, dtype=torch.float16, device=dev)
        capi.decode_attn(d_qkv, d_bias, g_kc, g_vc, out, H, t, D, 10000.0, workspace=ws)
        r_kc, r_vc = kc.copy(), vc.copy()
        want = ref.decode_attn(qkv, bias, r_kc, r_vc, H, t, D, 10000.0)
        np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL[np.float16])
        np.testing.assert_array_equal(_bits(g_kc[0, :, :, t - 1].cpu().numpy()), _bits(r_kc[0, :, :, t - 1]))
        np.testing.assert_array_equal(_bits(g_vc[0, :, :, t - 1].cpu().numpy()), _bits(r_vc[0, :, :, t - 1]))
        g_kc[0, :, :, t - 1] = d_kc[0, :, :, t - 1]
        g_vc[0, :, :, t - 1] = d_vc[0, :, :, t - 1]
        assert torch.equal(g_kc, d_kc) and torch.equal(g_vc, d_vc)              # nothing else was written
        # run-to-run: bit-identical output
        out2 = torch.zeros_like(out)
        capi.decode_attn(d_qkv, d_bias, d_kc.clone(), d_vc.clone(), out2, H, t, D, 10000.0, workspace=ws)
        assert torch.equal(out, out2)


@pytest.mark.parametrize("finish", ["merge_launch", "fused_finish"])
def test_config3_gqa_fused_equals_repeat_path(capi, ref, dev, finish):
    # BASELINE config 3: fp16, B32, 32 q heads over 8 kv heads x 128, S 8192, lengths U[1024, 8192].
    # (i) reference-style: concat the new row, repeat KV to 32 heads, attend with Hkv == Hq;
    # (ii) fused: attend straight from the [B, 8, S, 128] cache.  Both against the oracle.
    # `fused_finish` hands the library a zero-filled workspace with ONELLM_ATTN_ZEROED_WORKSPACE: the form the
    # launcher shim always uses and bench.py times (balanced schedule, one workgroup per compute unit, the piece that
    # arrives last merges its unit inside the attention kernel); `merge_launch` is the plain call (a second launch).
    announce("attn config3 setup", finish)
    flags = capi.ATTN_ZEROED_WORKSPACE if finish == "fused_finish" else 0
    torch.manual_seed(3)
    B, Hq, Hkv, D, S = 32, 32, 8, 128, 8192
    G = Hq // Hkv
    d_kc = torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half()
    d_vc = torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half()
    d_qkv = torch.randn(B, Hq + 2 * Hkv, D, device=dev).mul_(0.5).half()
    d_bias = torch.randn((Hq + 2 * Hkv) * D, device=dev).mul_(0.5).half()
    t = np.random.default_rng(3).integers(1024, 8193, size=B).astype(np.int32)
    t[0], t[1] = 8192, 1024
    d_t = torch.from_numpy(t).to(dev)
    # oracle
    r_kc, r_vc = d_kc.cpu().numpy(), d_vc.cpu().numpy()
    want = ref.decode_attn(d_qkv.cpu().numpy(), d_bias.cpu().numpy(), r_kc, r_vc, Hq, t, D, 10000.0)
    # (ii) fused
    announce("attn config3 fused")
    f_kc, f_vc = d_kc.clone(), d_vc.clone()
    out_f = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    capi.decode_attn(d_qkv, d_bias, f_kc, f_vc, out_f, Hq, int(t.max()), D, 10000.0, t_dev=d_t, max_t=int(t.max()),
                     flags=flags, workspace=ws)
    np.testing.assert_allclose(out_f.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL[np.float16])
    assert np.array_equal(_bits(f_kc.cpu().numpy()), _bits(r_kc)) and np.array_equal(_bits(f_vc.cpu().numpy()), _bits(r_vc))
    if flags:
        # the fused finish leaves its arrival counters (the first 64 KiB of the workspace) at zero, and a second
        # step on the same workspace gives the same bits
        assert int(ws[:64 * 1024].view(torch.int32).abs().max().item()) == 0
        out_f2 = torch.zeros_like(out_f)
        capi.decode_attn(d_qkv, d_bias, f_kc, f_vc, out_f2, Hq, int(t.max()), D, 10000.0, t_dev=d_t, max_t=int(t.max()),
                         flags=flags, workspace=ws)
        assert torch.equal(out_f, out_f2)
    # (i) repeat path on the cache that already holds the new rows: broadcast to 32 heads, then a
    # 32-head attention that re-derives the same new row (written again, same bits)
    announce("attn config3 repeat path")
    rk = torch.zeros(1, B, Hq, S, D, dtype=torch.float16, device=dev)
    rv = torch.zeros(1, B, Hq, S, D, dtype=torch.float16, device=dev)
    capi.kv_repeat(f_kc, f_vc, rk[0], rv[0], d_t)
    # MHA over the repeated cache: q heads as they are, k/v heads repeated in the fused buffer too
    qkv_r = torch.cat([d_qkv[:, :Hq], d_qkv[:, Hq:Hq + Hkv].repeat_interleave(G, 1),
                       d_qkv[:, Hq + Hkv:].repeat_interleave(G, 1)], 1).contiguous()
    b3 = d_bias.view(Hq + 2 * Hkv, D)
    bias_r = torch.cat([b3[:Hq], b3[Hq:Hq + Hkv].repeat_interleave(G, 0), b3[Hq + Hkv:].repeat_interleave(G, 0)], 0).contiguous().view(-1)
    out_r = torch.zeros_like(out_f)
    ws_r = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hq, D, S), dtype=torch.uint8, device=dev)
    capi.decode_attn(qkv_r, bias_r, rk, rv, out_r, Hq, int(t.max()), D, 10000.0, t_dev=d_t, max_t=int(t.max()),
                     flags=flags, workspace=ws_r)
    np.testing.assert_allclose(out_r.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL[np.float16])
    # same rows, same arithmetic per row group => the two paths agree far inside the tolerance
    assert (out_r.float() - out_f.float()).abs().max().item() <= 2e-3


def test_constant_value_rows_at_full_size(capi, dev):
    # size-independent property at config-2 size: if every V row (cache and new) equals c, out == c
    announce("attn constant V")
    torch.manual_seed(7)
    B, H, D, S, t = 16, 32, 128, 4096, 4096
    kc = torch.randn(1, B, H, S, D, device=dev).mul_(0.5).half()
    vc = torch.full((1, B, H, S, D), 0.375, dtype=torch.float16, device=dev)
    qkv = torch.randn(B, 3 * H, D, device=dev).mul_(0.5).half()
    qkv[:, 2 * H:] = 0.375
    out = torch.zeros(B, H * D, dtype=torch.float16, device=dev)
    capi.decode_attn(qkv, None, kc, vc, out, H, t, D, 10000.0)
    assert (out.float() - 0.375).abs().max().item() <= 1e-3


@pytest.mark.parametrize("D,Hq,dtype", [(128, 8, np.float16), (64, 8, np.float16), (256, 8, np.float16), (64, 32, np.float16),
                                        (256, 12, np.float16), (128, 16, np.float32), (128, 24, np.float32), (128, 40, np.float32), (64, 16, np.float32), (64, 34, np.float32)])
def test_options_on_the_matrix_core_kernel(capi, ref, dev, D, Hq, dtype):
    """The same option matrix as test_options on shapes that take the MFMA grouped-query kernels (fp16: head size 64,
    128 or 256, 4 / 6 / 16 query heads per kv head; fp32: head size 128, 8 / 12 / 20 heads per kv head), with one and
    with several sequence splits."""
    announce("attn options, mfma kernel", D, Hq, dtype.__name__)
    qkv, bias, kc, vc = _case(dtype, 2, Hq, 2, D, 200, 2, seed=23 + D, std=0.5)
    for nsplit in (-1, 3):
        capi.tune_set("attn_nsplit", nsplit)
        try:
            _assert_parity(_run_both(capi, ref, dev, qkv, None, kc, vc, Hq, 177, D, layer=1), dtype)
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, 177, 0), dtype)
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, 177, D // 2), dtype)
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, 177, D, pos_offset=-1, layer=1), dtype)
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, 177, D, base=500000.0), dtype)
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, 177, D, flags=capi.ATTN_NO_V_BIAS), dtype)
            res = _run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, 177, D, flags=capi.ATTN_NO_CACHE_WRITE)
            _assert_parity(res, dtype)
            np.testing.assert_array_equal(_bits(res[2]), _bits(kc))
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, 200, D), dtype)       # t == S
            for t in (1, 2, 16, 17, 63, 65):                                                           # short and partial batches
                _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, D), dtype)
        finally:
            capi.tune_set("attn_nsplit", -1)


@pytest.mark.parametrize("dtype,Hq,Hkv,D", [(np.float16, 8, 2, 128), (np.float16, 4, 4, 128), (np.float16, 14, 2, 128),
                                            (np.float16, 40, 2, 128), (np.float16, 8, 1, 64), (np.float16, 12, 2, 256),
                                            (np.float16, 6, 3, 32), (np.float32, 8, 2, 64), (np.float32, 3, 3, 128)])
@pytest.mark.parametrize("nwg", [1, 3, 50, 512, 1024])
def test_balanced_schedule(capi, ref, dev, dtype, Hq, Hkv, D, nwg):
    """The balanced workgroup schedule (equal shares of rows per workgroup, units split wherever a share ends) on
    ragged and equal lengths: lengths of 1 and 2, one long sequence among short ones (a unit with many partial
    states), more workgroups than work items."""
    announce("attn balanced", dtype.__name__, Hq, Hkv, D, "nwg", nwg)
    B, S = 7, 1500
    qkv, bias, kc, vc = _case(dtype, B, Hq, Hkv, D, S, 2, seed=nwg * 31 + Hq + D, std=0.5)
    capi.tune_set("attn_balanced", 1)
    capi.tune_set("attn_balanced_wgs", nwg)
    try:
        _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, np.array([1, 1500, 64, 65, 2, 777, 130]), D, layer=1), dtype)
        _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, np.array([1, 1, 1, 1, 1, 1, 1]), D), dtype)
        _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, np.array([3, 2, 1400, 2, 1, 1, 9]), D), dtype)
        for t in (1, 2, 129, 640, 1500):
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, D), dtype)
    finally:
        capi.tune_set("attn_balanced", -1)
        capi.tune_set("attn_balanced_wgs", -1)


def test_balanced_schedule_many_sequences(capi, ref, dev):
    """More sequences than a wave has lanes: the length scan of the balanced schedule runs over several blocks."""
    announce("attn balanced, 150 sequences")
    B, Hq, Hkv, D, S = 150, 4, 2, 128, 96
    qkv, bias, kc, vc = _case(np.float16, B, Hq, Hkv, D, S, 1, seed=151, std=0.5)
    t = np.random.default_rng(9).integers(1, S + 1, size=B)
    capi.tune_set("attn_balanced", 1)
    try:
        for nwg in (5, 512):
            capi.tune_set("attn_balanced_wgs", nwg)
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, D), np.float16)
    finally:
        capi.tune_set("attn_balanced", -1)
        capi.tune_set("attn_balanced_wgs", -1)


@pytest.mark.parametrize("dtype,Hq,Hkv,D", [(np.float16, 8, 2, 128), (np.float16, 4, 4, 128), (np.float16, 40, 2, 128),
                                            (np.float16, 8, 1, 64), (np.float16, 12, 2, 256), (np.float32, 8, 2, 64),
                                            (np.float32, 3, 3, 128)])
@pytest.mark.parametrize("schedule", ["default", "grid2", "grid5", "grid64", "balanced3", "balanced50", "balanced512"])
def test_fused_finish_with_a_zeroed_workspace(capi, ref, dev, dtype, Hq, Hkv, D, schedule):
    """ONELLM_ATTN_ZEROED_WORKSPACE: the piece of a split sequence that arrives last merges the sequence inside the
    attention kernel (no merge launch).  One workspace, zero-filled once, serves a series of calls with different
    lengths and splits: every call must leave its arrival counters at zero for the next."""
    announce("attn fused finish", dtype.__name__, Hq, Hkv, D, schedule)
    B, S = 7, 1500
    qkv, bias, kc, vc = _case(dtype, B, Hq, Hkv, D, S, 2, seed=len(schedule) * 17 + Hq + D, std=0.5)
    d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    if schedule.startswith("grid"):
        capi.tune_set("attn_nsplit", int(schedule[4:]))
    elif schedule.startswith("balanced"):
        capi.tune_set("attn_balanced", 1)
        capi.tune_set("attn_balanced_wgs", int(schedule[8:]))
    try:
        for rep, t in enumerate([np.array([1, 1500, 64, 65, 2, 777, 130]), 1500, np.array([3, 2, 1400, 2, 1, 1, 9]), 640,
                                 np.array([1, 1, 1, 1, 1, 1, 1]), np.array([1500, 1499, 1498, 700, 701, 702, 64]), 129]):
            d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
            out = torch.zeros(B, Hq * D, dtype=d_qkv.dtype, device=dev)
            ragged = isinstance(t, np.ndarray)
            t_dev = torch.from_numpy(t.astype(np.int32)).to(dev) if ragged else None
            max_t = int(t.max()) if ragged else t
            capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, out, Hq, max_t, D, 10000.0, layer=1, t_dev=t_dev, max_t=max_t,
                             flags=capi.ATTN_ZEROED_WORKSPACE, workspace=ws)
            r_kc, r_vc = kc.copy(), vc.copy()
            want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, t, D, 10000.0, layer=1)
            _assert_parity((out.cpu().numpy(), want, d_kc.cpu().numpy(), d_vc.cpu().numpy(), r_kc, r_vc), dtype)
            # (there is one counter per unit and at least one unit per kv head)
            assert int(ws[:B * Hkv * 4].view(torch.int32).abs().max().item()) == 0, "arrival counters not back at zero (call %d)" % rep
    finally:
        capi.tune_set("attn_nsplit", -1)
        capi.tune_set("attn_balanced", -1)
        capi.tune_set("attn_balanced_wgs", -1)


def test_fused_finish_at_full_size_matches_the_merge_launch(capi, dev):
    """Config-3 size (batch 32, 32 query heads over 8 kv heads, 8192-row caches) and a small-batch split shape: the
    in-kernel finish gives the merge launch's result (same pieces, merged in piece order either way) and is
    bit-identical from run to run, over a series of length vectors on one workspace."""
    torch.manual_seed(33)
    B, Hq, Hkv, D, S = 32, 32, 8, 128, 8192
    kc = torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half()
    vc = torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half()
    qkv = torch.randn(B, Hq + 2 * Hkv, D, device=dev).mul_(0.5).half()
    bias = torch.randn((Hq + 2 * Hkv) * D, device=dev).mul_(0.5).half()
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    rng = np.random.default_rng(33)
    outs = [torch.zeros(B, Hq * D, dtype=torch.float16, device=dev) for _ in range(3)]
    for rep in range(12):
        nb = [32, 32, 4, 1][rep % 4]
        if rep % 3 == 2:
            t, t_dev = int(rng.integers(2000, S + 1)), None
        else:
            lens = rng.integers(1, S + 1, size=nb).astype(np.int32)
            t, t_dev = int(lens.max()), torch.from_numpy(lens).to(dev)
        announce("attn fused finish full size, rep", rep, "batch", nb, "t", t, "ragged", t_dev is not None)
        for o, fl in zip(outs, (0, capi.ATTN_ZEROED_WORKSPACE, capi.ATTN_ZEROED_WORKSPACE)):
            capi.decode_attn(qkv[:nb], bias, kc[:, :nb].contiguous() if nb != B else kc, vc[:, :nb].contiguous() if nb != B else vc,
                             o[:nb], Hq, t, D, 10000.0, t_dev=t_dev, max_t=t, workspace=ws, flags=fl | capi.ATTN_NO_CACHE_WRITE)
        assert torch.equal(outs[1][:nb], outs[2][:nb])
        assert (outs[0][:nb].float() - outs[1][:nb].float()).abs().max().item() <= 1e-3


def test_fused_finish_soak_on_one_workspace(capi, dev):
    """200 calls of mixed shapes, schedules and lengths on ONE zero-filled workspace, each compared with the same call
    finished by the merge launch (same pieces, merged in piece order either way) and stopped at the first mismatch.
    The fused finish hands partial states between workgroups through agent-scope accesses and an arrival counter; a
    piece that read a stale state, or a counter that was not back at zero, shows up here as a wrong output."""
    torch.manual_seed(5)
    B, Hq, Hkv, D, S = 32, 32, 8, 128, 4096
    kc = torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half()
    vc = torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half()
    qkv = torch.randn(B, Hq + 2 * Hkv, D, device=dev).mul_(0.5).half()
    bias = torch.randn((Hq + 2 * Hkv) * D, device=dev).mul_(0.5).half()
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    ws_merge = torch.empty_like(ws)
    small = {nb: (kc[:, :nb].contiguous(), vc[:, :nb].contiguous()) for nb in (1, 2, 4, 8, 16)}
    small[32] = (kc, vc)
    rng = np.random.default_rng(5)
    o_merge = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    o_fused = torch.zeros_like(o_merge)
    try:
        for rep in range(200):
            mode = rep % 5
            nb = int(rng.choice([1, 2, 4, 8, 16, 32]))
            if mode == 0:
                t, t_dev = int(rng.integers(1, S + 1)), None
            else:
                lens = rng.integers(1, S + 1, size=nb).astype(np.int32)
                if mode == 2:
                    lens[:] = np.minimum(lens, 300)
                t, t_dev = int(lens.max()), torch.from_numpy(lens).to(dev)
            if mode == 3:
                capi.tune_set("attn_balanced", 1)
                capi.tune_set("attn_balanced_wgs", int(rng.choice([7, 100, 512, 1024])))
            if mode == 4:
                capi.tune_set("attn_ordered_finish", 1)      # the formally ordered hand-over (release / acquire fence)
            # the register-held merge by a piece that finds the others arrived: forced on, forced off, or the default
            capi.tune_set("attn_early_look", [1, 0, -1][rep % 3])
            if rep % 20 == 0:
                announce("attn fused soak, rep", rep)
            k, v = small[nb]
            capi.decode_attn(qkv[:nb], bias, k, v, o_merge[:nb], Hq, t, D, 10000.0, t_dev=t_dev, max_t=t, workspace=ws_merge,
                             flags=capi.ATTN_NO_CACHE_WRITE)
            capi.decode_attn(qkv[:nb], bias, k, v, o_fused[:nb], Hq, t, D, 10000.0, t_dev=t_dev, max_t=t, workspace=ws,
                             flags=capi.ATTN_NO_CACHE_WRITE | capi.ATTN_ZEROED_WORKSPACE)
            capi.tune_set("attn_balanced", -1)
            capi.tune_set("attn_balanced_wgs", -1)
            capi.tune_set("attn_ordered_finish", -1)
            capi.tune_set("attn_early_look", -1)
            diff = (o_merge[:nb].float() - o_fused[:nb].float()).abs().max().item()
            assert diff <= 1e-3, "call %d (mode %d, batch %d, t %d): fused finish differs from the merge launch by %g" % (rep, mode, nb, t, diff)
        assert int(ws[:65536].view(torch.int32).abs().max().item()) == 0, "arrival counters not back at zero"
    finally:
        capi.tune_set("attn_balanced", -1)
        capi.tune_set("attn_balanced_wgs", -1)
        capi.tune_set("attn_ordered_finish", -1)
        capi.tune_set("attn_early_look", -1)


@pytest.mark.parametrize("B,Hq,Hkv,t", [(9, 32, 32, 600), (36, 32, 8, 600), (5, 64, 64, 1100), (20, 16, 8, 1300), (72, 32, 8, 330),
                                        (81, 16, 8, 290)])
@pytest.mark.parametrize("zeroed", [False, True])
def test_equal_lengths_on_an_uneven_grid(capi, ref, dev, B, Hq, Hkv, t, zeroed):
    """Equal lengths with a grid that does not fill the chip evenly (288, 320 units; 160 units cut in two; 576 and 648
    grouped-query units on the matrix-core kernel, which holds two workgroups per compute unit): the launcher hands
    the compute units equal shares of the rows instead (balanced schedule, 256 or 512 workgroups), with the merge
    launch or - on a zeroed workspace - the fused finish."""
    announce("attn uneven grid", B, Hq, Hkv, t, zeroed)
    D, S = 128, t + 20
    qkv, bias, kc, vc = _case(np.float16, B, Hq, Hkv, D, S, 1, seed=B * 7 + t, std=0.5)
    d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
    d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    for rep in range(2):
        out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
        g_kc, g_vc = d_kc.clone(), d_vc.clone()
        capi.decode_attn(d_qkv, d_bias, g_kc, g_vc, out, Hq, t, D, 10000.0, workspace=ws,
                         flags=capi.ATTN_ZEROED_WORKSPACE if zeroed else 0)
        r_kc, r_vc = kc.copy(), vc.copy()
        want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, t, D, 10000.0)
        _assert_parity((out.cpu().numpy(), want, g_kc.cpu().numpy(), g_vc.cpu().numpy(), r_kc, r_vc), np.float16)
        assert int(ws[:65536].view(torch.int32).abs().max().item()) == 0, "the counter region must stay zero either way"


@pytest.mark.parametrize("B,Hq,Hkv,D,t", [(1, 32, 8, 128, 8192), (2, 32, 8, 128, 8192), (1, 64, 8, 128, 8192), (1, 32, 32, 128, 4096),
                                          (1, 16, 2, 256, 6000), (1, 16, 16, 64, 8192)])
def test_long_sequences_of_a_small_batch(capi, ref, dev, B, Hq, Hkv, D, t):
    """One or two long sequences: every unit is cut into up to 64 pieces and finished inside the kernel by the piece
    that arrives last (on a zeroed workspace) - with many pieces through the LDS-staged form of that merge - or by
    the merge launch; both against the oracle."""
    announce("attn long sequence, small batch", B, Hq, Hkv, D, t)
    S = t
    qkv, bias, kc, vc = _case(np.float16, B, Hq, Hkv, D, S, 1, seed=t + Hq, std=0.5)
    d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    r_kc, r_vc = kc.copy(), vc.copy()
    want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, t, D, 10000.0)
    for flags in (capi.ATTN_ZEROED_WORKSPACE, capi.ATTN_ZEROED_WORKSPACE, 0):
        d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
        out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
        capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, out, Hq, t, D, 10000.0, workspace=ws, flags=flags)
        _assert_parity((out.cpu().numpy(), want, d_kc.cpu().numpy(), d_vc.cpu().numpy(), r_kc, r_vc), np.float16)
        assert int(ws[:65536].view(torch.int32).abs().max().item()) == 0


@pytest.mark.parametrize("max_t", [4095, 4096])
@pytest.mark.parametrize("ragged", [False, True])
def test_two_heads_per_kv_head_either_side_of_the_kernel_switch(capi, ref, dev, max_t, ragged):
    """16 query heads over 8 kv heads at head size 128: steps whose longest sequence has 4096 rows or more run on the
    matrix-core kernel, shorter ones on the vector-ALU kernel (onellm_amd/csrc/decode_attn.hip: on_matrix_cores).
    Both sides of that switch, equal and per-sequence lengths, merge launch and fused finish, against the oracle."""
    announce("attn two heads per kv head", max_t, "ragged" if ragged else "equal")
    B, Hq, Hkv, D = 3, 16, 8, 128
    S = 4096
    lens = np.array([max_t, 700, 2500]) if ragged else np.full(B, max_t)
    qkv, bias, kc, vc = _case(np.float16, B, Hq, Hkv, D, S, 1, seed=max_t, std=0.5)
    d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    t_dev = torch.from_numpy(lens.astype(np.int32)).to(dev) if ragged else None
    r_kc, r_vc = kc.copy(), vc.copy()
    want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, lens if ragged else max_t, D, 10000.0)
    for flags in (capi.ATTN_ZEROED_WORKSPACE, 0, capi.ATTN_ZEROED_WORKSPACE):
        d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
        out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
        capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, out, Hq, max_t, D, 10000.0, t_dev=t_dev, max_t=max_t, workspace=ws, flags=flags)
        _assert_parity((out.cpu().numpy(), want, d_kc.cpu().numpy(), d_vc.cpu().numpy(), r_kc, r_vc), np.float16)
        assert int(ws[:65536].view(torch.int32).abs().max().item()) == 0


@pytest.mark.parametrize("B,Hq,Hkv,tmax,ragged", [(8, 32, 32, 2048, True), (12, 32, 32, 2100, True), (6, 32, 32, 1024, False),
                                                   (24, 32, 8, 2048, False), (28, 32, 8, 2500, False), (17, 32, 32, 1100, False),
                                                   (18, 32, 32, 2050, False), (16, 32, 8, 2048, True), (12, 32, 8, 3000, True),
                                                   (16, 16, 8, 2048, True)])
@pytest.mark.parametrize("zeroed", [False, True])
def test_default_dispatch_choices_found_by_interleaved_timing(capi, ref, dev, B, Hq, Hkv, tmax, ragged, zeroed):
    """Shapes at which the launcher's own choice changed after timings on buffers that are never freed: per-sequence
    lengths on the vector-ALU kernel with 2048 rows or more and 8192..50000 items (one equal share per compute unit, a
    unit change charged five items), and equal lengths with 160..255 units (whole units, no split; the matrix-core kernel
    from 176 units at 2048 rows and from 208 beyond); 544 and 576 single-head units (a few more than two per compute unit:
    512 equal shares); per-sequence lengths on the matrix-core kernel with 128 and with 96 units (one share per compute
    unit / the grid schedule) and two-head vector-ALU tiles below 8192 items (the grid schedule).  No tuning keys; against
    the oracle, twice on one workspace."""
    announce("attn dispatch choices", B, Hq, Hkv, tmax, "ragged" if ragged else "equal", "zeroed" if zeroed else "merge launch")
    D, S = 128, tmax
    rng = np.random.default_rng(B * 1000 + tmax)
    lens = rng.integers(tmax // 8, tmax + 1, size=B) if ragged else np.full(B, tmax)
    lens[0] = tmax
    qkv, bias, kc, vc = _case(np.float16, B, Hq, Hkv, D, S, 1, seed=B + tmax, std=0.5)
    d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
    d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
    out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    t_dev = torch.from_numpy(lens.astype(np.int32)).to(dev) if ragged else None
    for _ in range(2):
        capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, out, Hq, tmax, D, 10000.0, t_dev=t_dev, max_t=tmax,
                         flags=capi.ATTN_ZEROED_WORKSPACE if zeroed else 0, workspace=ws)
    r_kc, r_vc = kc.copy(), vc.copy()
    want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, lens if ragged else tmax, D, 10000.0)
    _assert_parity((out.cpu().numpy(), want, d_kc.cpu().numpy(), d_vc.cpu().numpy(), r_kc, r_vc), np.float16)
    assert int(ws[:65536].view(torch.int32).abs().max().item()) == 0


def test_default_dispatch_at_medium_sizes(capi, ref, dev):
    """Sixteen seeded shapes of a few hundred units and a few thousand rows, equal and per-sequence lengths, with and
    without a zeroed workspace, no tuning keys: whatever schedule the launcher picks by itself (grid with or without a
    split, equal shares on an uneven grid, balanced walk, merge launch or fused finish) gives the oracle's result."""
    rng = np.random.default_rng(20240)
    for case in range(16):
        dtype = [np.float16, np.float16, np.float32][int(rng.integers(0, 3))]
        D = int(rng.choice([64, 128, 128, 256]))
        if dtype == np.float32 and D == 256:
            D = 128
        Hkv = int(rng.choice([2, 4, 8, 8, 32, 40]))
        G = int(rng.choice([1, 4, 8, 5])) if Hkv <= 8 else 1
        Hq = Hkv * G
        B = int(rng.integers(1, 17 if Hkv >= 32 else 41))
        tmax = int(rng.integers(200, 1801))
        S = tmax + int(rng.integers(0, 64))
        ragged = bool(rng.integers(0, 2))
        lens = rng.integers(max(1, tmax // 8), tmax + 1, size=B) if ragged else np.full(B, tmax)
        lens[int(rng.integers(0, B))] = tmax
        zeroed = bool(rng.integers(0, 2))
        announce("attn default dispatch", case, dtype.__name__, "B", B, "Hq", Hq, "Hkv", Hkv, "D", D, "t", tmax, "ragged", ragged, "zeroed", zeroed)
        qkv, bias, kc, vc = _case(dtype, B, Hq, Hkv, D, S, 1, seed=7000 + case, std=0.5)
        d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
        d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
        out = torch.zeros(B, Hq * D, dtype=d_qkv.dtype, device=dev)
        ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
        t_dev = torch.from_numpy(lens.astype(np.int32)).to(dev) if ragged else None
        for _ in range(2):                                       # (twice on one workspace: the counters must come back to zero)
            capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, out, Hq, tmax, D, 10000.0, t_dev=t_dev, max_t=tmax,
                             flags=capi.ATTN_ZEROED_WORKSPACE if zeroed else 0, workspace=ws)
        r_kc, r_vc = kc.copy(), vc.copy()
        want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, lens if ragged else tmax, D, 10000.0)
        _assert_parity((out.cpu().numpy(), want, d_kc.cpu().numpy(), d_vc.cpu().numpy(), r_kc, r_vc), dtype)
        assert int(ws[:65536].view(torch.int32).abs().max().item()) == 0


def test_random_shapes_sweep(capi, ref, dev):
    """Eighty seeded random (dtype, heads, group size, head size, lengths, split count, schedule) combinations, ragged lengths
    included: every kernel variant and padded head tile gets shapes nobody picked by hand."""
    rng = np.random.default_rng(2024)
    for case in range(80):
        dtype = [np.float16, np.float32][int(rng.integers(0, 2))]
        D = int(rng.choice([16, 32, 64, 128, 128, 128, 256, 96, 80, 192]))
        Hkv = int(rng.integers(1, 4))
        G = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 20]))
        Hq = Hkv * G
        B = int(rng.integers(1, 5))
        S = int(rng.integers(8, 420))
        lens = rng.integers(1, S + 1, size=B)
        ragged = bool(rng.integers(0, 2))
        t = lens if ragged else int(lens.max())
        nsplit = int(rng.choice([-1, -1, 1, 2, 3, 7]))
        rot = int(rng.choice([D, D, D // 2, 0]))
        balanced = int(rng.choice([-1, 0, 1])) if nsplit == -1 else -1
        nwg = int(rng.choice([-1, 2, 9, 100]))
        announce("attn sweep", case, dtype.__name__, "B", B, "Hq", Hq, "Hkv", Hkv, "D", D, "S", S, "t", t, "nsplit", nsplit, "rot", rot,
                 "balanced", balanced, "nwg", nwg)
        qkv, bias, kc, vc = _case(dtype, B, Hq, Hkv, D, S, 1, seed=5000 + case, std=0.5)
        capi.tune_set("attn_nsplit", nsplit)
        capi.tune_set("attn_balanced", balanced)
        capi.tune_set("attn_balanced_wgs", nwg)
        try:
            _assert_parity(_run_both(capi, ref, dev, qkv, bias, kc, vc, Hq, t, rot), dtype)
        finally:
            capi.tune_set("attn_nsplit", -1)
            capi.tune_set("attn_balanced", -1)
            capi.tune_set("attn_balanced_wgs", -1)
