"""The committed golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py from float64 numpy
models of the mathematics) against BOTH implementations: the CPU oracle (runs anywhere) and the HIP kernels through
the C ABI (marked gpu).  The vectors come from neither, so they pin both.

Bars: fp32 results within 1e-5 relative of the float64 expectation (+2e-6 absolute where values cancel), fp16
results within 2e-3 absolute / 1e-2 relative; the rows written into the KV cache within one rounding of the
storage type of the float64 value; copies (append, repeat) and top-K ids bit-exact."""
import os

import numpy as np
import pytest

from conftest import announce

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = {np.dtype(np.float32): dict(rtol=1e-5, atol=2e-6), np.dtype(np.float16): dict(rtol=1e-2, atol=2e-3)}


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


class OracleBackend:
    """numpy in, numpy out, through oracle/ref.py"""

    def __init__(self, ref):
        self.ref = ref

    def decode_attn(self, f):
        kc, vc = f["k_cache"].copy(), f["v_cache"].copy()
        out = self.ref.decode_attn(f["qkv"], f["bias"], kc, vc, int(f["Hq"]), f["t"], int(f["rotary_dim"]), float(f["base"]),
                                   rope_pos_offset=int(f["pos_offset"]))
        return out, kc, vc

    def rmsnorm(self, x, gamma, eps):
        return self.ref.rmsnorm(x.copy(), gamma, eps)

    def fused_norm(self, res, x, bias, gamma, eps):
        return self.ref.fused_add_bias_residual_rmsnorm(res.copy(), x.copy(), bias, gamma, eps)

    def kv_append(self, ks, vs, kc, vc, cur, hist, layer):
        kc, vc = kc.copy(), vc.copy()
        self.ref.kv_append(ks, vs, kc, vc, cur, hist, layer=layer)
        return kc, vc

    def kv_repeat(self, kc, vc, kd, vd, ctx, layer):
        kd, vd = kd.copy(), vd.copy()
        self.ref.kv_repeat(kc, vc, kd, vd, ctx, layer=layer)
        return kd, vd

    def beam_topk(self, logits, B, beam, K):
        return self.ref.beam_topk(logits, B, beam, K)

    def prefill(self, q, k, v, qkv, bias, po, hist, rd, base):
        self.ref.qkv_bias_rope_transpose(q, k, v, qkv, bias, po, hist, rd, base)
        return q, k, v

    def swiglu(self, inp):
        return self.ref.silu_and_mul(inp, np.zeros((inp.shape[0], inp.shape[2]), inp.dtype))


class GpuBackend:
    """numpy in, numpy out, through the C ABI (onellm_amd/capi.py) on cuda:0"""

    def __init__(self, capi, dev):
        import torch
        self.capi, self.dev, self.torch = capi, dev, torch

    def _t(self, a):
        return self.torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)

    def decode_attn(self, f):
        t = self.torch
        qkv, bias, kc, vc = self._t(f["qkv"]), self._t(f["bias"]), self._t(f["k_cache"]), self._t(f["v_cache"])
        B, _, D = f["qkv"].shape
        Hq = int(f["Hq"])
        out = t.zeros(B, Hq * D, dtype=qkv.dtype, device=self.dev)
        lens = f["t"].astype(np.int32)
        self.capi.decode_attn(qkv, bias, kc, vc, out, Hq, int(lens.max()), int(f["rotary_dim"]), float(f["base"]),
                              t_dev=self._t(lens), max_t=int(lens.max()), rope_pos_offset=int(f["pos_offset"]))
        return out.cpu().numpy(), kc.cpu().numpy(), vc.cpu().numpy()

    def rmsnorm(self, x, gamma, eps):
        return self.capi.rmsnorm(self._t(x), self._t(gamma), eps).cpu().numpy()

    def fused_norm(self, res, x, bias, gamma, eps):
        r, o = self.capi.fused_add_bias_residual_rmsnorm(self._t(res), self._t(x), self._t(bias), self._t(gamma), eps)
        return r.cpu().numpy(), o.cpu().numpy()

    def kv_append(self, ks, vs, kc, vc, cur, hist, layer):
        kc, vc = self._t(kc), self._t(vc)
        self.capi.kv_append(self._t(ks), self._t(vs), kc, vc, self._t(cur), self._t(hist), layer=layer)
        return kc.cpu().numpy(), vc.cpu().numpy()

    def kv_repeat(self, kc, vc, kd, vd, ctx, layer):
        kd, vd = self._t(kd), self._t(vd)
        self.capi.kv_repeat(self._t(kc), self._t(vc), kd, vd, self._t(ctx), layer=layer)
        return kd.cpu().numpy(), vd.cpu().numpy()

    def beam_topk(self, logits, B, beam, K):
        _, vals, ids, fv, fi = self.capi.beam_topk(self._t(logits), B, beam, K)
        return vals.cpu().numpy(), ids.cpu().numpy(), fv.cpu().numpy(), fi.cpu().numpy()

    def prefill(self, q, k, v, qkv, bias, po, hist, rd, base):
        q, k, v = self._t(q), self._t(k), self._t(v)
        self.capi.qkv_bias_rope_transpose(q, k, v, self._t(qkv), self._t(bias), self._t(po), self._t(hist), rd, base)
        return q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()

    def swiglu(self, inp):
        out = self.torch.zeros(inp.shape[0], inp.shape[2], dtype=self._t(inp).dtype, device=self.dev)
        return self.capi.silu_and_mul(self._t(inp), out).cpu().numpy()


@pytest.fixture(params=["oracle", pytest.param("gpu", marks=pytest.mark.gpu)])
def backend(request):
    if request.param == "oracle":
        return OracleBackend(request.getfixturevalue("ref"))
    return GpuBackend(request.getfixturevalue("capi"), request.getfixturevalue("dev"))


def close(got, want, dtype):
    np.testing.assert_allclose(np.asarray(got, np.float64), want, **TOL[np.dtype(dtype)])


def one_rounding(got, want64, dtype):
    """got (storage type) is the float64 value rounded to the storage type, give or take one unit in the last place
    (the float64 model and the fp32 arithmetic of the implementations may fall on different sides of a tie)."""
    got = np.asarray(got)
    lo = np.nextafter(want64.astype(dtype), np.array(-np.inf, dtype)).astype(np.float64)
    hi = np.nextafter(want64.astype(dtype), np.array(np.inf, dtype)).astype(np.float64)
    # fp32 arithmetic before the rounding (a rotated element's error scales with its pair, hence the row maximum)
    slack = 3e-6 * np.abs(want64).max(axis=-1, keepdims=True) + 1e-7
    assert np.all(got.astype(np.float64) >= lo - slack) and np.all(got.astype(np.float64) <= hi + slack)


@pytest.mark.parametrize("name", ["attn_config1_fp32", "attn_gqa_fp16_ragged", "attn_d256_fp16"])
def test_decode_attention(backend, name):
    announce("golden", name, type(backend).__name__)
    f = load(name)
    dtype = f["qkv"].dtype
    out, kc, vc = backend.decode_attn(f)
    close(out, f["out"], dtype)
    B = f["qkv"].shape[0]
    for b in range(B):
        row = int(f["t"][b]) - 1
        one_rounding(kc[0, b, :, row], f["new_k"][b], dtype)
        one_rounding(vc[0, b, :, row], f["new_v"][b], dtype)
        kc[0, b, :, row] = f["k_cache"][0, b, :, row]
        vc[0, b, :, row] = f["v_cache"][0, b, :, row]
    assert np.array_equal(kc, f["k_cache"]) and np.array_equal(vc, f["v_cache"])       # nothing else was written


@pytest.mark.parametrize("name", ["norms_fp16", "norms_fp32"])
def test_norms(backend, name):
    announce("golden", name, type(backend).__name__)
    f = load(name)
    dtype = f["x"].dtype
    close(backend.rmsnorm(f["x"], f["gamma"], float(f["eps"])), f["rmsnorm"], dtype)
    res, out = backend.fused_norm(f["residual"], f["x"], f["bias"], f["gamma"], float(f["eps"]))
    close(out, f["fused_out"], dtype)
    one_rounding(res, f["fused_residual"], dtype)


def test_kv_append_and_repeat(backend):
    announce("golden kv_append_repeat", type(backend).__name__)
    f = load("kv_append_repeat")
    layer = int(f["layer"])
    ka, va = backend.kv_append(f["k_src"], f["v_src"], f["k_cache"], f["v_cache"], f["cur_len"], f["history_len"], layer)
    assert np.array_equal(ka.view(np.uint16), f["k_after_append"].view(np.uint16))
    assert np.array_equal(va.view(np.uint16), f["v_after_append"].view(np.uint16))
    sentinel = np.full_like(f["k_repeated"], 7.0)
    kr, vr = backend.kv_repeat(f["k_after_append"], f["v_after_append"], sentinel, sentinel.copy(), f["context_len"], layer)
    assert np.array_equal(kr.view(np.uint16), f["k_repeated"].view(np.uint16))
    assert np.array_equal(vr.view(np.uint16), f["v_repeated"].view(np.uint16))


def test_beam_topk_with_ties(backend):
    announce("golden beam_topk_ties", type(backend).__name__)
    f = load("beam_topk_ties")
    B, beam, K = int(f["B"]), int(f["beam"]), int(f["K"])
    vals, ids, fv, fi = backend.beam_topk(f["logits"], B, beam, K)
    assert np.array_equal(fi, f["final_ids"])
    assert np.array_equal(fv.view(np.uint32), f["final_vals"].view(np.uint32))
    # stage 1 keeps K per (row, block): their best K per row, under the same order, are the row's top K
    flat = f["logits"].reshape(-1)
    for r in range(B * beam):
        cand = ids[r].reshape(-1)
        cand = cand[cand >= 0]
        order = np.lexsort((cand, -flat[cand].astype(np.float64)))
        assert np.array_equal(cand[order[:K]], f["row_ids"][r])


@pytest.mark.parametrize("name", ["prefill_rope_fp32", "prefill_rope_fp16"])
def test_prefill_rope(backend, name):
    announce("golden", name, type(backend).__name__)
    f = load(name)
    dtype = f["qkv"].dtype
    B, S, Hq = int(f["B"]), int(f["S"]), int(f["Hq"])
    Hkv = (f["qkv"].shape[1] - Hq) // 2
    D = f["qkv"].shape[2]
    q = np.full((B, Hq, S, D), 9.0, dtype)
    k = np.full((B, Hkv, S, D), 9.0, dtype)
    v = np.full((B, Hkv, S, D), 9.0, dtype)
    q, k, v = backend.prefill(q, k, v, f["qkv"], f["bias"], f["padding_offset"], f["history_len"], int(f["rotary_dim"]),
                              float(f["base"]))
    w = f["written"]
    for got, want in ((q, f["q"]), (k, f["k"]), (v, f["v"])):
        for b in range(B):
            # positions up to 3011 rad: the fp32 angle itself carries ~1e-4 absolute error there
            np.testing.assert_allclose(got[b][:, w[b]].astype(np.float64), want[b][:, w[b]], rtol=1e-2 if dtype == np.float16 else 2e-4,
                                       atol=2e-3 if dtype == np.float16 else 3e-4)
            assert np.all(got[b][:, ~w[b]] == 9.0)                                  # padded slots untouched


@pytest.mark.parametrize("name", ["swiglu_fp32", "swiglu_fp16"])
def test_swiglu(backend, name):
    announce("golden", name, type(backend).__name__)
    f = load(name)
    close(backend.swiglu(f["inp"]), f["out"], f["inp"].dtype)
