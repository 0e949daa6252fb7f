"""The bare access-pattern kernels bench.py times as ceilings move exactly the bytes they claim to (a ceiling that
skipped part of its traffic would flatter nothing but itself)."""
import pytest
import torch

import access_ceilings as ac
from conftest import announce

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("policy", range(5))
def test_each_pattern_moves_its_bytes(dev, policy):
    announce("access ceilings policy", policy)
    assert len(ac.policies()) == 5
    g = torch.Generator(device=dev).manual_seed(policy)
    src = torch.randn(1 << 20, device=dev, generator=g)                 # 4 MiB
    dst = torch.zeros_like(src)
    ac.copy(dst, src, policy)
    assert torch.equal(dst, src)
    ac.fill(dst, 3.5, policy)
    assert (dst == 3.5).all()
    sink = torch.zeros(src.numel() * 4 // 16384, device=dev)
    ac.read(src, sink, policy)                                          # reads only; the sink stays as it was
    assert not sink.any()
    fan = torch.zeros(4, src.numel(), device=dev)
    ac.fanout(fan, src, 4, policy)
    assert all(torch.equal(fan[i], src) for i in range(4))
    chunks = torch.zeros(16, 4, src.numel() // 16, device=dev)          # 16 chunks of 256 KiB, four copies side by side
    ac.fanout(chunks, src, 4, policy, chunk=src.numel() * 4 // 16)
    assert all(torch.equal(chunks[:, i].reshape(-1), src) for i in range(4))
    tm = torch.randn(64, 6, 64, device=dev, generator=g)                # 64 tokens x 6 heads x 256 bytes, sequences of 16
    hm = torch.zeros(4, 6, 16, 64, device=dev)
    ac.regroup(hm, tm, 16, policy)
    assert torch.equal(hm, tm.view(4, 16, 6, 64).permute(0, 2, 1, 3).contiguous())
    for row_elems in (2048, 4096, 8192):                                # 8, 16, 32 KiB rows of fp32
        a = torch.randn(64, row_elems, device=dev, generator=g)
        b = torch.randn(64, row_elems, device=dev, generator=g)
        shared = torch.randn(row_elems, device=dev, generator=g)
        a0, b0 = a.clone(), b.clone()
        ac.rows(a, None, None, policy)                                  # one buffer: rewritten with what it held
        assert torch.equal(a, a0)
        ac.rows(a, None, shared, policy)
        assert torch.equal(a, a0)
        ac.rows(a, b, shared, policy)                                   # two buffers: both end up holding the sum
        assert torch.equal(a, a0 + b0) and torch.equal(b, a0 + b0)
