"""The layout a many-layer model uses: one KV-cache tensor [layers, B, Hkv, S, D] per K and V, as the decoder example
allocates it (examples/cpp/decoder/self_decoder_example.cpp:186-187 of the reference), large enough that the element
offset of the layer slab the step works on does not fit 32 bits.  Decode attention (the single-head vector-ALU kernel
and the grouped-query matrix-core kernel on the balanced schedule), the KV append, the KV repeat and the launcher
shims all run on slab 9 of 11; the oracle is given that one slab as a one-layer cache, so host memory stays ~1 GB.

Bars: outputs within the fp16 tolerance (2e-3 absolute / 1e-2 relative), the slab bit for bit, and every other slab of
the tensor - the ones a 32-bit wrap of the offset would land in - untouched."""
import ctypes
import os

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "tests", "cpp", "liblauncher_harness.so")
TOL = dict(rtol=1e-2, atol=2e-3)
LAYERS, LAYER = 11, 9


def _bits(a):
    return a.view(np.uint16)


def _harness():
    assert os.path.exists(HARNESS), "build it with `python -m onellm_amd.build`"
    L = ctypes.CDLL(HARNESS)
    vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    L.h_last_error.restype = ctypes.c_char_p
    L.h_decode_mha.argtypes = [ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, ci, cf]
    L.h_append.argtypes = [ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci]
    L.h_repeat.argtypes = [ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci]
    return L


def _filled_cache(shape, dev, seed):
    """[layers, B, Hkv, S, D] fp16 ~ N(0, 0.5), filled a slab at a time (no fp32 copy of the whole tensor)."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    c = torch.empty(shape, dtype=torch.float16, device=dev)
    for layer in range(shape[0]):
        c[layer] = torch.randn(shape[1:], device=dev, generator=g).mul_(0.5).half()
    return c


def _others_untouched(cache, snapshot, what):
    for layer in range(LAYERS):
        if layer != LAYER:
            assert torch.equal(cache[layer], snapshot[layer]), f"{what}: slab {layer} was written"


@pytest.mark.parametrize("name,B,Hq,Hkv,S,ragged", [("single_head_valu_kernel", 16, 32, 32, 4096, False),
                                                    ("gqa_mfma_kernel_balanced", 32, 32, 8, 8192, True)])
def test_layer_slab_past_two_to_the_31_elements(capi, ref, dev, name, B, Hq, Hkv, S, ragged):
    D = 128
    slab_elems = B * Hkv * S * D
    assert LAYER * slab_elems > 2 ** 31 and LAYERS * slab_elems * 2 < 2 ** 34      # ~5.9 GB per tensor
    announce("big cache", name, "fill")
    kc = _filled_cache((LAYERS, B, Hkv, S, D), dev, 100)
    vc = _filled_cache((LAYERS, B, Hkv, S, D), dev, 101)
    k_snap, v_snap = kc.clone(), vc.clone()
    rng = np.random.default_rng(9)
    qkv = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * 0.5).astype(np.float16)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(np.float16)
    d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
    if ragged:
        t = rng.integers(S // 8, S - 8, size=B).astype(np.int32)
        t[0], t[1] = S - 8, S // 8
    else:
        t = np.full(B, S - 8, np.int32)
    d_t = torch.from_numpy(t).to(dev)
    # the oracle's cache: slab LAYER alone, as a one-layer tensor
    r_kc = kc[LAYER].cpu().numpy()[None].copy()
    r_vc = vc[LAYER].cpu().numpy()[None].copy()

    # ---- decode attention through the C ABI, the way bench.py and the launcher shim call it (zeroed workspace)
    announce("big cache", name, "decode_attn layer", LAYER)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    capi.decode_attn(d_qkv, d_bias, kc, vc, out, Hq, int(t.max()), D, 10000.0, layer=LAYER,
                     t_dev=d_t if ragged else None, max_t=int(t.max()), flags=capi.ATTN_ZEROED_WORKSPACE, workspace=ws)
    want = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, t if ragged else int(t[0]), D, 10000.0, layer=0)
    np.testing.assert_allclose(out.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL)
    assert np.array_equal(_bits(kc[LAYER].cpu().numpy()), _bits(r_kc[0])), "K slab differs from the oracle's"
    assert np.array_equal(_bits(vc[LAYER].cpu().numpy()), _bits(r_vc[0])), "V slab differs from the oracle's"
    _others_untouched(kc, k_snap, "decode_attn K")
    _others_untouched(vc, v_snap, "decode_attn V")

    # ---- the same step through the launcher shim, which is handed the slab as a 4-D tensor (what the attention
    # layer does) and a host step: equal lengths
    announce("big cache", name, "launchDecoderMaskedMHA on the slab")
    H = _harness()
    step = S - 3
    out_l = torch.zeros_like(out)
    rc = H.h_decode_mha(1, d_qkv.data_ptr(), d_bias.data_ptr(), kc[LAYER].data_ptr(), vc[LAYER].data_ptr(), out_l.data_ptr(),
                        B, Hq, Hkv, D, S, 0, step, 0, D, 10000.0)
    assert rc == 0, H.h_last_error()
    assert H.h_sync_and_check() == 0, H.h_last_error()
    want_l = ref.decode_attn(qkv, bias, r_kc, r_vc, Hq, step, D, 10000.0, layer=0)
    np.testing.assert_allclose(out_l.cpu().numpy().astype(np.float64), want_l.astype(np.float64), **TOL)
    assert np.array_equal(_bits(kc[LAYER].cpu().numpy()), _bits(r_kc[0]))
    assert np.array_equal(_bits(vc[LAYER].cpu().numpy()), _bits(r_vc[0]))
    _others_untouched(kc, k_snap, "launchDecoderMaskedMHA K")
    _others_untouched(vc, v_snap, "launchDecoderMaskedMHA V")

    # ---- KV append into the slab: C ABI, then the launcher with a host layer id
    announce("big cache", name, "kv_append layer", LAYER)
    Q = 3
    ks = (rng.standard_normal((B, Hkv, Q, D)) * 0.5).astype(np.float16)
    vs = (rng.standard_normal((B, Hkv, Q, D)) * 0.5).astype(np.float16)
    cur = rng.integers(0, Q + 1, size=B).astype(np.int32)
    hist = rng.integers(0, S - Q, size=B).astype(np.int32)
    hist[0], cur[0] = S - Q, Q                                       # the slab's last rows
    d_ks, d_vs = torch.from_numpy(ks).to(dev), torch.from_numpy(vs).to(dev)
    d_cur, d_hist = torch.from_numpy(cur).to(dev), torch.from_numpy(hist).to(dev)
    capi.kv_append(d_ks, d_vs, kc, vc, d_cur, d_hist, layer=LAYER)
    ref.kv_append(ks, vs, r_kc, r_vc, cur, hist, layer=0)
    assert np.array_equal(_bits(kc[LAYER].cpu().numpy()), _bits(r_kc[0]))
    assert np.array_equal(_bits(vc[LAYER].cpu().numpy()), _bits(r_vc[0]))
    hist2 = ((hist.astype(np.int64) + 17) % (S - Q)).astype(np.int32)
    d_hist2 = torch.from_numpy(hist2).to(dev)
    rc = H.h_append(1, d_ks.data_ptr(), d_vs.data_ptr(), kc.data_ptr(), vc.data_ptr(), d_cur.data_ptr(), d_hist2.data_ptr(),
                    B, Hkv, Q, S, D, LAYERS, LAYER)
    assert rc == 0, H.h_last_error()
    assert H.h_sync_and_check() == 0, H.h_last_error()
    ref.kv_append(ks, vs, r_kc, r_vc, cur, hist2, layer=0)
    assert np.array_equal(_bits(kc[LAYER].cpu().numpy()), _bits(r_kc[0]))
    assert np.array_equal(_bits(vc[LAYER].cpu().numpy()), _bits(r_vc[0]))
    _others_untouched(kc, k_snap, "kv_append K")
    _others_untouched(vc, v_snap, "kv_append V")

    # ---- KV repeat out of the slab (destination rows clipped to 1024 so the host copy stays small)
    announce("big cache", name, "kv_repeat layer", LAYER)
    MK = 1024
    ctx = rng.integers(1, 1500, size=B).astype(np.int32)
    ctx[0] = MK
    d_ctx = torch.from_numpy(ctx).to(dev)
    for via_launcher in (False, True):
        kd = torch.full((B, Hq, MK, D), 9.0, dtype=torch.float16, device=dev)
        vd = torch.full((B, Hq, MK, D), 9.0, dtype=torch.float16, device=dev)
        if via_launcher:
            rc = H.h_repeat(1, kc.data_ptr(), vc.data_ptr(), kd.data_ptr(), vd.data_ptr(), d_ctx.data_ptr(),
                            B, Hq, Hkv, S, MK, D, LAYERS, LAYER)
            assert rc == 0, H.h_last_error()
            assert H.h_sync_and_check() == 0, H.h_last_error()
        else:
            capi.kv_repeat(kc, vc, kd, vd, d_ctx, layer=LAYER)
        r_kd = np.full((B, Hq, MK, D), 9.0, np.float16)
        r_vd = np.full((B, Hq, MK, D), 9.0, np.float16)
        ref.kv_repeat(r_kc, r_vc, r_kd, r_vd, ctx, layer=0)
        assert np.array_equal(_bits(kd.cpu().numpy()), _bits(r_kd))
        assert np.array_equal(_bits(vd.cpu().numpy()), _bits(r_vd))
    _others_untouched(kc, k_snap, "kv_repeat K")
    _others_untouched(vc, v_snap, "kv_repeat V")
