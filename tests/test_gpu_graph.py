"""The C ABI neither allocates nor synchronises, so a decode step can be captured into a HIP graph and
replayed.  One layer's worth of the path (RMSNorm -> fused decode attention with a sequence split ->
fused add-bias-residual-RMSNorm -> SwiGLU -> beam top-K) is captured once and replayed several times
with eager work and synchronisations in between; every replay must reproduce the eager result bit for bit."""
import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fused_finish", [False, True])
def test_captured_decode_step_replays_bit_identically(capi, dev, fused_finish):
    # fused_finish: the attention workspace is zero-filled once and declared so; the split sequences are then
    # finished inside the attention kernel (arrival counters, reset by every call) instead of by a merge launch
    announce("graph capture of a decode step, fused finish", fused_finish)
    torch.manual_seed(11)
    B, Hq, Hkv, D, S, t, H, I, V = 4, 32, 8, 128, 2048, 1500, 4096, 2048, 8000
    x0 = torch.randn(B, H, device=dev).half()
    gamma = torch.rand(H, device=dev).add(0.5).half()
    qkv0 = torch.randn(B, Hq + 2 * Hkv, D, device=dev).mul(0.5).half()
    bias = torch.randn((Hq + 2 * Hkv) * D, device=dev).mul(0.5).half()
    kc0 = torch.randn(1, B, Hkv, S, D, device=dev).mul(0.5).half()
    vc0 = torch.randn(1, B, Hkv, S, D, device=dev).mul(0.5).half()
    t_dev = torch.tensor([1500, 700, 33, 1], dtype=torch.int32, device=dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, t), dtype=torch.uint8, device=dev)
    attn_flags = capi.ATTN_ZEROED_WORKSPACE if fused_finish else 0
    act_in0 = torch.randn(B, 2, I, device=dev).half()
    logits = torch.randn(B * 2, V, device=dev)
    topk_ws = torch.empty(capi.beam_topk_workspace_bytes(B, 2, 4) // 4, dtype=torch.float32, device=dev)

    # buffers the step works on (restored before every run so that runs are comparable)
    x, res = x0.clone(), torch.zeros_like(x0)
    kc, vc = kc0.clone(), vc0.clone()
    attn_out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    act_out = torch.zeros(B, I, dtype=torch.float16, device=dev)

    def restore():
        x.copy_(x0); res.zero_(); kc.copy_(kc0); vc.copy_(vc0); attn_out.zero_(); act_out.zero_(); topk_ws.zero_()

    def step():
        capi.rmsnorm(x, gamma, 1e-5)
        capi.decode_attn(qkv0, bias, kc, vc, attn_out, Hq, t, D, 10000.0, t_dev=t_dev, max_t=t, workspace=ws, flags=attn_flags)
        capi.fused_add_bias_residual_rmsnorm(res, x, None, gamma, 1e-5)
        capi.silu_and_mul(act_in0, act_out)
        capi.beam_topk(logits, B, 2, 4, workspace=topk_ws)

    def snapshot():
        torch.cuda.synchronize()
        return [a.clone() for a in (x, res, attn_out, act_out, topk_ws, kc[0, :, :, :1501], vc[0, :, :, :1501])]

    restore()
    step()
    want = snapshot()

    restore()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                    # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    restore()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        step()
    for replay in range(4):
        restore()
        (x0 * 2).sum().item()                     # eager work and a synchronisation between replays
        g.replay()
        got = snapshot()
        for a, b in zip(got, want):
            assert torch.equal(a, b), f"replay {replay} differs from the eager step"
