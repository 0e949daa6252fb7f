"""onellm_decode_attn_static (the entry point that allocates nothing: split partials and arrival counters live in a
fixed device array inside the library) against onellm_decode_attn on the same inputs, through the C ABI.

Both entry points run the same kernels with the same split, and the fused finish merges the pieces of a unit in
piece order, so the outputs are compared bit for bit; the existing entry point is also run with a separate merge
launch (no ZEROED_WORKSPACE flag), which must agree within the fp16 / fp32 parity bars.  Two calls in a row share
the built-in array, the second with a smaller input.  Collected last: a failure here must not hide other tests."""
import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

TOL = {np.float32: dict(rtol=1e-5, atol=1e-6), np.float16: dict(rtol=1e-2, atol=2e-3)}


def _bits(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


def _inputs(dtype, B, Hq, Hkv, D, S, seed):
    rng = np.random.default_rng(seed)
    qkv = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * 0.5).astype(dtype)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(dtype)
    kc = (rng.standard_normal((1, B, Hkv, S, D)) * 0.5).astype(dtype)
    vc = (rng.standard_normal((1, B, Hkv, S, D)) * 0.5).astype(dtype)
    return qkv, bias, kc, vc


def _three_ways(capi, dev, dtype, B, Hq, Hkv, D, S, t, seed):
    """(static entry, existing entry + fused finish, existing entry + merge launch): outputs and caches."""
    qkv, bias, kc, vc = _inputs(dtype, B, Hq, Hkv, D, S, seed)
    ragged = isinstance(t, np.ndarray)
    max_t = int(t.max()) if ragged else int(t)
    res = []
    for way in ("static", "fused", "merge"):
        d_qkv, d_bias = torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev)
        d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
        d_out = torch.zeros(B, Hq * D, dtype=d_qkv.dtype, device=dev)
        t_dev = torch.from_numpy(t.astype(np.int32)).to(dev) if ragged else None
        announce("no-alloc", way, dtype.__name__, "B", B, "Hq", Hq, "Hkv", Hkv, "D", D, "S", S, "max_t", max_t, "ragged", ragged)
        if way == "static":
            capi.decode_attn_static(d_qkv, d_bias, d_kc, d_vc, d_out, Hq, max_t, D, 10000.0, t_dev=t_dev, max_t=max_t)
        else:
            nbytes = capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, max_t)
            ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
            capi.decode_attn(d_qkv, d_bias, d_kc, d_vc, d_out, Hq, max_t, D, 10000.0, t_dev=t_dev, max_t=max_t,
                             flags=capi.ATTN_ZEROED_WORKSPACE if way == "fused" else 0, workspace=ws)
        torch.cuda.synchronize()
        res.append((d_out.cpu().numpy(), d_kc.cpu().numpy(), d_vc.cpu().numpy()))
    return res


def _check(res, dtype):
    (s_out, s_kc, s_vc), (f_out, f_kc, f_vc), (m_out, m_kc, m_vc) = res
    assert np.isfinite(s_out.astype(np.float64)).all()
    np.testing.assert_array_equal(_bits(s_out), _bits(f_out))
    np.testing.assert_array_equal(_bits(s_kc), _bits(f_kc))
    np.testing.assert_array_equal(_bits(s_vc), _bits(f_vc))
    np.testing.assert_allclose(s_out.astype(np.float64), m_out.astype(np.float64), **TOL[dtype])
    np.testing.assert_array_equal(_bits(s_kc), _bits(m_kc))
    np.testing.assert_array_equal(_bits(s_vc), _bits(m_vc))


def test_static_entry_matches_existing_entry_two_calls_in_a_row(capi, dev):
    # first a grouped-query step whose units are each split into several pieces (the scratch holds counters and
    # partials), then a smaller one on the same built-in array: fewer sequences, shorter, another head layout
    _check(_three_ways(capi, dev, np.float16, 4, 32, 8, 128, 4096, 4096, seed=11), np.float16)
    _check(_three_ways(capi, dev, np.float16, 2, 8, 8, 128, 1100, 1024, seed=12), np.float16)
    # per-sequence lengths (balanced schedule: pieces of different units land in one workgroup), then fp32, smaller
    t = np.array([4096, 700, 2300, 1, 1500, 3333], dtype=np.int32)
    _check(_three_ways(capi, dev, np.float16, 6, 32, 8, 128, 4096, t, seed=13), np.float16)
    _check(_three_ways(capi, dev, np.float32, 1, 8, 2, 64, 2048, 2048, seed=14), np.float32)


def test_static_entry_unsplit_step_and_oracle(capi, ref, dev):
    # a step that needs no scratch at all, checked against the CPU oracle
    B, Hq, Hkv, D, S, t = 16, 32, 32, 128, 600, 513
    qkv, bias, kc, vc = _inputs(np.float16, B, Hq, Hkv, D, S, seed=15)
    d_kc, d_vc = torch.from_numpy(kc).to(dev), torch.from_numpy(vc).to(dev)
    d_out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    announce("no-alloc unsplit vs oracle")
    capi.decode_attn_static(torch.from_numpy(qkv).to(dev), torch.from_numpy(bias).to(dev), d_kc, d_vc, d_out, Hq, t, D, 10000.0)
    want = ref.decode_attn(qkv, bias, kc, vc, Hq, t, D, 10000.0)
    np.testing.assert_allclose(d_out.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL[np.float16])
    np.testing.assert_array_equal(_bits(d_kc.cpu().numpy()), _bits(kc))
    np.testing.assert_array_equal(_bits(d_vc.cpu().numpy()), _bits(vc))


def test_static_entry_rejects_a_step_beyond_its_scratch(capi, dev):
    # 16 x 32 heads forced into 64 pieces each: 16*32*64*(128+2)*4 B of partials = 17.0 MB > 16 MiB
    B, Hq, Hkv, D, S, t = 16, 32, 32, 128, 4096, 4096
    need = 64 * 1024 + B * Hq * 64 * (D + 2) * 4
    assert need > capi.DECODE_ATTN_STATIC_SCRATCH_BYTES
    d_qkv = torch.zeros(B, Hq + 2 * Hkv, D, dtype=torch.float16, device=dev)
    d_kc = torch.zeros(1, B, Hkv, S, D, dtype=torch.float16, device=dev)
    d_vc = torch.zeros_like(d_kc)
    d_out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    capi.tune_set("attn_nsplit", 64)
    try:
        announce("no-alloc rejection")
        with pytest.raises(capi.OnellmError) as e:
            capi.decode_attn_static(d_qkv, None, d_kc, d_vc, d_out, Hq, t, D, 10000.0)
        assert e.value.code == capi.ESCRATCH
        assert "built-in scratch" in str(e.value)
    finally:
        capi.tune_set("attn_nsplit", -1)
    torch.cuda.synchronize()
    assert not d_kc.any() and not d_out.any()        # rejected before anything was launched
