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


def _split_step(dev, seed=21, B=4, Hq=32, Hkv=8, D=128, S=4096, t=4096):
    qkv, bias, kc, vc = _inputs(np.float16, B, Hq, Hkv, D, S, seed)
    return dict(qkv=torch.from_numpy(qkv).to(dev), bias=torch.from_numpy(bias).to(dev), kc=torch.from_numpy(kc).to(dev),
                vc=torch.from_numpy(vc).to(dev), out=torch.zeros(B, Hq * D, dtype=torch.float16, device=dev), Hq=Hq, t=t, D=D)


def _static(capi, s, t_dev=None):
    capi.decode_attn_static(s["qkv"], s["bias"], s["kc"], s["vc"], s["out"], s["Hq"], s["t"], s["D"], 10000.0, t_dev=t_dev,
                            max_t=s["t"])


def test_static_entry_leaves_free_device_memory_where_it_was(capi, dev):
    """What the entry point promises: no device memory is allocated or freed by a call.  hipMemGetInfo (through torch)
    before and after split steps of three shapes - equal, per-sequence and long single-sequence lengths - reads the same
    number of free bytes.  Every tensor exists before the first reading and one step has run (code objects loaded)."""
    steps = [_split_step(dev, 21), _split_step(dev, 22, B=6, S=2048, t=2048), _split_step(dev, 23, B=1, Hq=8, Hkv=2, S=8192, t=8192)]
    t_dev = torch.tensor([2048, 300, 1, 999, 1500, 2047], dtype=torch.int32, device=dev)
    announce("no-alloc: free memory, warm-up")
    for s in steps:
        _static(capi, s)
    _static(capi, steps[1], t_dev)
    torch.cuda.synchronize()
    reserved = torch.cuda.memory_reserved()
    free_before, _ = torch.cuda.mem_get_info()
    announce("no-alloc: free memory, measured calls")
    for _ in range(3):
        for s in steps:
            _static(capi, s)
        _static(capi, steps[1], t_dev)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_reserved() == reserved          # (torch itself took nothing in between either)
    assert free_after == free_before, (free_before, free_after)


def test_static_entry_captured_into_a_graph_replays_bit_identically(capi, dev):
    """Its stated use: a split step recorded into a HIP graph (after one ordinary call) and replayed, with eager calls
    on the shared built-in scratch and synchronisations between the replays; every replay gives the eager bits."""
    s = _split_step(dev, 31)
    announce("no-alloc: eager call before capture")
    _static(capi, s)
    torch.cuda.synchronize()
    want = s["out"].clone()
    kc_after, vc_after = s["kc"].clone(), s["vc"].clone()
    other = _split_step(dev, 32, B=2, S=2048, t=1999)
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    announce("no-alloc: capture")
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            _static(capi, s)
    torch.cuda.synchronize()
    for rep in range(4):
        announce("no-alloc: replay", rep)
        s["out"].fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(s["out"], want), "replay %d" % rep
        assert torch.equal(s["kc"], kc_after) and torch.equal(s["vc"], vc_after)
        _static(capi, other)                                  # eager work on the same scratch between replays
        torch.cuda.synchronize()
    del g


_FIRST_CALL_CHILD = r"""
import sys
sys.path.insert(0, sys.argv[1])
import numpy as np
import torch
from onellm_amd import capi

dev = torch.device("cuda:0")
rng = np.random.default_rng(41)
B, Hq, Hkv, D, S, t = 4, 32, 8, 128, 4096, 4096
mk = lambda *shape: torch.from_numpy((rng.standard_normal(shape) * 0.5).astype(np.float16)).to(dev)
qkv, bias, kc, vc = mk(B, Hq + 2 * Hkv, D), mk((Hq + 2 * Hkv) * D), mk(1, B, Hkv, S, D), mk(1, B, Hkv, S, D)
kc2, vc2 = kc.clone(), vc.clone()
out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
L = capi.lib()
torch.cuda.synchronize()
print("CHILD capture begins", flush=True)
side = torch.cuda.Stream()
g = torch.cuda.CUDAGraph()
rc = None
try:
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            # the very first call into the kernel library in this process, on a stream that is being captured
            rc = L.onellm_decode_attn_static(capi.FP16, qkv.data_ptr(), bias.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(),
                                             B, Hq, Hkv, D, S, 0, 1, t, None, t, D, 10000.0, 0, 0, side.cuda_stream)
    captured = True
except RuntimeError as e:
    captured = False
    print("CHILD capture did not end cleanly:", str(e).splitlines()[0], flush=True)
print("CHILD rc", rc, flush=True)
if rc == 0 and captured:
    g.replay()
    torch.cuda.synchronize()
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, t), dtype=torch.uint8, device=dev)
    out2 = torch.zeros_like(out)
    capi.decode_attn(qkv, bias, kc2, vc2, out2, Hq, t, D, 10000.0, flags=capi.ATTN_ZEROED_WORKSPACE, workspace=ws)
    torch.cuda.synchronize()
    same = bool(torch.equal(out, out2) and torch.equal(kc, kc2) and torch.equal(vc, vc2))
    print("CHILD replay equals the eager entry point:", same, flush=True)
    sys.exit(0 if same else 3)
# a refusal must be an error code the library can name, and must leave the process usable
text = L.onellm_error_string(rc).decode() if rc is not None else "no return"
print("CHILD refused:", text, flush=True)
sys.exit(0 if (rc is not None and rc != 0) else 4)
"""


def test_static_entry_as_the_first_call_of_a_process_on_a_capturing_stream(dev):
    """A fresh process whose first call into the library is onellm_decode_attn_static on a stream under capture: the
    symbol of the built-in scratch is resolved and the kernel's code object is loaded inside the capture.  Either
    the step is recorded and its replay equals the existing entry point bit for bit, or the call returns an error code
    with a text; the process must not abort either way."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    announce("no-alloc: first call of a fresh process under capture")
    r = subprocess.run([sys.executable, "-u", "-c", _FIRST_CALL_CHILD, root], capture_output=True, text=True, timeout=600)
    sys.__stderr__.write(r.stdout[-2000:] + r.stderr[-2000:])
    sys.__stderr__.flush()
    assert r.returncode == 0, (r.returncode, r.stdout[-1500:], r.stderr[-1500:])
    assert "CHILD rc" in r.stdout
