"""GPU parity of KV concat, KV repeat and beam top-K against the CPU oracle (bit-exact), through the C ABI."""
import zlib

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


def _bits(a):
    return a.view(np.uint16 if a.dtype == np.float16 else np.uint32)


# ---------------------------------------------------------------- KV concat

def test_append_reference_unit_vector(capi, dev):
    announce("append unit vector")
    ks = torch.ones(1, 2, 16, 8, device=dev)
    kc = torch.full((1, 1, 2, 32, 8), -9.0, device=dev)
    vc = torch.full((1, 1, 2, 32, 8), -9.0, device=dev)
    capi.kv_append(ks, ks.clone(), kc, vc, torch.tensor([16], dtype=torch.int32, device=dev),
                   torch.tensor([1], dtype=torch.int32, device=dev))
    for c in (kc.cpu().numpy(), vc.cpu().numpy()):
        np.testing.assert_array_equal(c[0, 0, :, 1:17], 1.0)
        np.testing.assert_array_equal(c[0, 0, :, 0], -9.0)
        np.testing.assert_array_equal(c[0, 0, :, 17:], -9.0)


@pytest.mark.parametrize("dtype,D", [(np.float16, 128), (np.float32, 64), (np.float16, 12), (np.float32, 5)])
@pytest.mark.parametrize("Q", [1, 7])
def test_append_matches_oracle(capi, ref, dev, dtype, D, Q):
    announce("append", dtype.__name__, D, Q)
    rng = np.random.default_rng(3)
    L, B, Hkv, S = 2, 5, 3, 40
    ks = rng.standard_normal((B, Hkv, Q, D)).astype(dtype)
    vs = rng.standard_normal((B, Hkv, Q, D)).astype(dtype)
    kc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    vc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    cur = np.minimum(rng.integers(0, Q + 1, B), Q).astype(np.int32)
    cur[0] = Q
    hist = rng.integers(0, S - Q + 1, B).astype(np.int32)
    hist[1] = S - 1          # spills over the end when cur > 1: those rows are dropped
    d = [torch.from_numpy(a).to(dev) for a in (ks, vs, kc, vc, cur, hist)]
    capi.kv_append(*d, layer=1)
    ref.kv_append(ks, vs, kc, vc, cur, hist, layer=1)
    np.testing.assert_array_equal(_bits(d[2].cpu().numpy()), _bits(kc))
    np.testing.assert_array_equal(_bits(d[3].cpu().numpy()), _bits(vc))


def test_append_decode_shape_of_gqa_config(capi, ref, dev):
    # BASELINE config 3, the per-token concat: B32, Hkv8, D128, S8192, one new row per sequence
    announce("append cfg3 decode")
    torch.manual_seed(3)
    B, Hkv, S, D = 32, 8, 8192, 128
    kc = torch.zeros(1, B, Hkv, S, D, dtype=torch.float16, device=dev)
    vc = torch.zeros(1, B, Hkv, S, D, dtype=torch.float16, device=dev)
    ks = torch.randn(B, Hkv, 1, D, device=dev).mul(0.5).half()
    vs = torch.randn(B, Hkv, 1, D, device=dev).mul(0.5).half()
    hist = torch.randint(1023, 8191, (B,), dtype=torch.int32, device=dev)
    capi.kv_append(ks, vs, kc, vc, torch.ones(B, dtype=torch.int32, device=dev), hist)
    idx = hist.long()
    got_k = kc[0, torch.arange(B, device=dev), :, idx]          # [B, Hkv, D]
    got_v = vc[0, torch.arange(B, device=dev), :, idx]
    assert torch.equal(got_k, ks[:, :, 0]) and torch.equal(got_v, vs[:, :, 0])
    assert int(kc.count_nonzero().item()) == int(ks.count_nonzero().item())     # nothing else was written
    assert int(vc.count_nonzero().item()) == int(vs.count_nonzero().item())


# ---------------------------------------------------------------- KV repeat

def test_repeat_reference_unit_vector(capi, dev):
    announce("repeat unit vector")
    src = torch.arange(32, dtype=torch.float32, device=dev).view(2, 1, 2, 4, 2)
    kd = torch.full((1, 2, 2, 2), -1.0, device=dev)
    vd = torch.full((1, 2, 2, 2), -1.0, device=dev)
    capi.kv_repeat(src, src.clone(), kd, vd, torch.tensor([2], dtype=torch.int32, device=dev))
    np.testing.assert_array_equal(kd.cpu().numpy().ravel(), [0, 1, 2, 3, 8, 9, 10, 11])
    np.testing.assert_array_equal(vd.cpu().numpy().ravel(), [0, 1, 2, 3, 8, 9, 10, 11])


@pytest.mark.parametrize("dtype,Hq,Hkv,D", [(np.float16, 32, 8, 128), (np.float32, 4, 4, 64), (np.float16, 6, 1, 12),
                                            (np.float32, 8, 2, 3)])
def test_repeat_matches_oracle(capi, ref, dev, dtype, Hq, Hkv, D):
    announce("repeat", dtype.__name__, Hq, Hkv, D)
    rng = np.random.default_rng(8)
    L, B, S, MK = 2, 4, 50, 44
    kc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    vc = rng.standard_normal((L, B, Hkv, S, D)).astype(dtype)
    lens = np.array([44, 1, 49, 0], np.int32)      # 49 > max_k_len: clipped; 0: nothing written
    kd = np.full((B, Hq, MK, D), 5.0, dtype)
    vd = np.full((B, Hq, MK, D), 5.0, dtype)
    d = [torch.from_numpy(a).to(dev) for a in (kc, vc, kd, vd, lens)]
    capi.kv_repeat(*d, layer=1)
    ref.kv_repeat(kc, vc, kd, vd, lens, layer=1)
    np.testing.assert_array_equal(_bits(d[2].cpu().numpy()), _bits(kd))
    np.testing.assert_array_equal(_bits(d[3].cpu().numpy()), _bits(vd))


# ---------------------------------------------------------------- beam top-K

@pytest.fixture(params=["one_launch-4waves", "two_launches-4waves", "one_launch-8waves", "two_launches-8waves"])
def topk_form(request, capi):
    """Both forms of the second stage - merged by the last stage-1 workgroup of a batch entry, or by a second launch -
    with four and with eight waves per stage-1 workgroup (the launcher picks by shape; here both run on every shape)."""
    form, waves = request.param.split("-")
    capi.tune_set("topk_two_launches", 1 if form == "two_launches" else 0)
    capi.tune_set("topk_waves", 8 if waves == "8waves" else 4)
    yield request.param
    capi.tune_set("topk_two_launches", -1)
    capi.tune_set("topk_waves", -1)


def _lexsort_topk(flat_vals, flat_ids, K):
    order = np.lexsort((flat_ids, -flat_vals.astype(np.float64)))[:K]
    return flat_vals[order], flat_ids[order]


def test_topk_reference_unit_vector(capi, dev, topk_form):
    announce("topk unit vector", topk_form)
    logits = torch.arange(60000, dtype=torch.float32, device=dev).view(2, 30000)
    ws, _, _, fv, fi = capi.beam_topk(logits, 1, 2, 2)
    np.testing.assert_array_equal(fi.cpu().numpy(), [[59999, 59998]])
    np.testing.assert_array_equal(fv.cpu().numpy(), [[59999.0, 59998.0]])
    # where the reference's unit test reads them: vals at 2*B*beam*8*beam, ids B*beam further
    w = ws.cpu().numpy()
    assert w[2 * 1 * 2 * 8 * 2] == 59999.0 and w.view(np.int32)[2 * 1 * 2 * 8 * 2 + 1 * 2] == 59999


def test_topk_config5_planted_ties(capi, ref, dev, topk_form):
    announce("topk cfg5", topk_form)
    rng = np.random.default_rng(5)
    B, beam, V, K = 8, 4, 32000, 4
    logits = (rng.standard_normal((B * beam, V)) * 2.0).astype(np.float32)
    for b in range(B):
        top = logits[b * beam:(b + 1) * beam].max() + 1.0
        for r in (b * beam, b * beam + 3):
            logits[r, [17, 16000, 31999]] = top
    _, v1, i1, fv, fi = capi.beam_topk(torch.from_numpy(logits).to(dev), B, beam, K)
    w1v, w1i, wfv, wfi = ref.beam_topk(logits, B, beam, K)
    np.testing.assert_array_equal(i1.cpu().numpy(), w1i)
    np.testing.assert_array_equal(v1.cpu().numpy().view(np.uint32), w1v.view(np.uint32))
    np.testing.assert_array_equal(fi.cpu().numpy(), wfi)
    np.testing.assert_array_equal(fv.cpu().numpy().view(np.uint32), wfv.view(np.uint32))
    # and against numpy's lexsort directly
    flat = logits.reshape(B, beam * V)
    for b in range(B):
        v, i = _lexsort_topk(flat[b], np.arange(beam * V) + b * beam * V, K)
        np.testing.assert_array_equal(fi.cpu().numpy()[b], i)


@pytest.mark.parametrize("B,beam,V,K", [(1, 1, 1, 1), (2, 3, 100, 8), (3, 2, 257, 5), (1, 4, 2049, 3), (5, 1, 50000, 2),
                                        (2, 2, 128256, 4), (1, 1, 3, 8),
                                        # more survivors per batch entry than one pass of the merging wave holds (256)
                                        (2, 8, 1000, 8), (1, 16, 3000, 4), (1, 40, 500, 2)])
def test_topk_shapes_with_heavy_ties(capi, ref, dev, B, beam, V, K, topk_form):
    announce("topk", B, beam, V, K, topk_form)
    rng = np.random.default_rng(V + K)
    # few distinct values => many ties, the order of equal values is what is being checked
    logits = rng.integers(-3, 4, size=(B * beam, V)).astype(np.float32)
    _, v1, i1, fv, fi = capi.beam_topk(torch.from_numpy(logits).to(dev), B, beam, K)
    w1v, w1i, wfv, wfi = ref.beam_topk(logits, B, beam, K)
    np.testing.assert_array_equal(i1.cpu().numpy(), w1i)
    np.testing.assert_array_equal(fi.cpu().numpy(), wfi)
    np.testing.assert_array_equal(fv.cpu().numpy().view(np.uint32), wfv.view(np.uint32))


def _pattern(name, rows, V, rng):
    if name == "normal":
        return rng.standard_normal((rows, V)).astype(np.float32)
    if name == "ascending":        # every later token beats all earlier ones: nothing can be rejected early
        return (np.arange(rows * V, dtype=np.float32).reshape(rows, V) * 0.25)
    if name == "descending":
        return -(np.arange(rows * V, dtype=np.float32).reshape(rows, V) * 0.25)
    if name == "all_equal":
        return np.full((rows, V), 1.5, np.float32)
    if name == "masked_ranges":    # whole stretches of the vocabulary at -inf, as a banned-token mask leaves them
        a = rng.standard_normal((rows, V)).astype(np.float32)
        for r in range(rows):
            lo = int(rng.integers(0, V))
            a[r, lo:lo + V // 3] = -np.inf
            a[r, ::7] = -np.inf
        return a
    if name == "few_finite":       # fewer finite values than K in some rows
        a = np.full((rows, V), -np.inf, np.float32)
        for r in range(rows):
            idx = rng.integers(0, V, size=r % 4)
            a[r, idx] = rng.standard_normal(len(idx)).astype(np.float32)
        return a
    if name == "sawtooth":         # rising runs of 64 tokens: many lanes of a wave hold a contender at once
        return ((np.arange(rows * V) % 64).astype(np.float32) + rng.integers(0, 3, size=rows * V).astype(np.float32)).reshape(rows, V)
    raise ValueError(name)


@pytest.mark.parametrize("pattern", ["normal", "ascending", "descending", "all_equal", "masked_ranges", "few_finite", "sawtooth"])
@pytest.mark.parametrize("B,beam,V,K", [(2, 2, 32000, 4), (1, 3, 32000, 8), (2, 1, 50257, 2), (1, 2, 128256, 1), (1, 2, 151937, 5)])
def test_topk_data_patterns(capi, ref, dev, topk_form, pattern, B, beam, V, K):
    """What the scan does depends on the data (how many values pass the floor, how many lanes hold a contender at
    once, how many rounds a batch takes); the result must not.  Vocabulary sizes with and without the 16-byte
    path, one to four batches per wave."""
    announce("topk pattern", pattern, B, beam, V, K, topk_form)
    rng = np.random.default_rng(zlib.crc32(("%s %d %d" % (pattern, V, K)).encode()))
    logits = _pattern(pattern, B * beam, V, rng)
    _, v1, i1, fv, fi = capi.beam_topk(torch.from_numpy(logits).to(dev), B, beam, K)
    w1v, w1i, wfv, wfi = ref.beam_topk(logits, B, beam, K)
    np.testing.assert_array_equal(i1.cpu().numpy(), w1i)
    np.testing.assert_array_equal(v1.cpu().numpy().view(np.uint32), w1v.view(np.uint32))
    np.testing.assert_array_equal(fi.cpu().numpy(), wfi)
    np.testing.assert_array_equal(fv.cpu().numpy().view(np.uint32), wfv.view(np.uint32))


def test_topk_nan_inputs_finish_and_keep_the_finite_order(capi, dev, topk_form):
    """NaN has no place in the reference's order (its comparisons are all false for NaN); here a NaN with the sign
    bit clear sorts above +inf and one with it set below -inf.  Checked: the call finishes, the ids are valid, and a
    row's finite values keep their order below the positive NaNs."""
    announce("topk NaN", topk_form)
    B, beam, V, K = 1, 2, 4096, 4
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((B * beam, V)).astype(np.float32)
    logits[0, [10, 2000]] = np.float32(np.nan)
    logits[1, 77] = -np.float32(np.nan)
    logits.view(np.uint32)[1, 77] |= 0x80000000
    _, _, _, fv, fi = capi.beam_topk(torch.from_numpy(logits).to(dev), B, beam, K)
    ids = fi.cpu().numpy()[0]
    assert list(ids[:2]) == [10, 2000] and np.isnan(fv.cpu().numpy()[0, :2]).all()
    finite = logits.reshape(-1).copy()
    finite[[10, 2000, V + 77]] = -np.inf
    order = np.lexsort((np.arange(finite.size), -finite.astype(np.float64)))[:2]
    np.testing.assert_array_equal(ids[2:], order)


def test_topk_negative_infinity_and_run_to_run(capi, ref, dev, topk_form):
    announce("topk -inf", topk_form)
    logits = np.full((2, 1000), -np.inf, np.float32)
    logits[0, 500] = 1.0
    d = torch.from_numpy(logits).to(dev)
    _, _, _, fv, fi = capi.beam_topk(d, 1, 2, 4)
    _, _, wfv, wfi = ref.beam_topk(logits, 1, 2, 4)
    np.testing.assert_array_equal(fi.cpu().numpy(), wfi)
    np.testing.assert_array_equal(fi.cpu().numpy(), [[500, 0, 1, 2]])
    a = fi.clone()
    _, _, _, _, fi2 = capi.beam_topk(d, 1, 2, 4)
    assert torch.equal(a, fi2)


def test_topk_zeros_of_both_signs_and_extreme_values(capi, ref, dev, topk_form):
    """-0.0 and +0.0 tie (the lower index wins) and every stored value carries the bits of the input it came from:
    zeros keep their sign, denormals, the largest finite value and infinities come back unchanged."""
    announce("topk signed zeros and extreme values", topk_form)
    B, beam, V, K = 2, 2, 600, 4
    logits = -np.abs(np.random.default_rng(17).standard_normal((B * beam, V)).astype(np.float32)) - 1.0
    logits[0, [5, 300, 599]] = [-0.0, 0.0, -0.0]                 # three zeros on top: indices 5, 300, 599 in this order
    logits[1, [7, 8]] = [0.0, -0.0]
    logits[2, [1, 2, 3, 4]] = [np.float32(1e-45), np.float32(-1e-45), np.finfo(np.float32).max, np.inf]
    logits[3, [10, 11]] = [np.finfo(np.float32).tiny, -np.inf]
    _, v1, i1, fv, fi = capi.beam_topk(torch.from_numpy(logits).to(dev), B, beam, K)
    w1v, w1i, wfv, wfi = ref.beam_topk(logits, B, beam, K)
    np.testing.assert_array_equal(i1.cpu().numpy(), w1i)
    np.testing.assert_array_equal(v1.cpu().numpy().view(np.uint32), w1v.view(np.uint32))
    np.testing.assert_array_equal(fi.cpu().numpy(), wfi)
    np.testing.assert_array_equal(fv.cpu().numpy().view(np.uint32), wfv.view(np.uint32))
    got_i, got_v = fi.cpu().numpy(), fv.cpu().numpy()
    np.testing.assert_array_equal(got_i[0], [5, 300, 599, V + 7])
    flat = logits.reshape(-1)
    np.testing.assert_array_equal(got_v.view(np.uint32), flat[got_i].view(np.uint32))   # the input's own bits


def test_topk_one_launch_repeats_on_one_workspace_and_falls_back_past_its_limits(capi, ref, dev):
    """The one-launch form leaves its arrival counters as it found them: 150 calls on one workspace, shapes and K
    changing from call to call, all equal to the oracle.  A process that passes more distinct workspaces than there are
    counter sets gets the two-launch form for the surplus ones, with the same results."""
    announce("topk one launch: repeats, changing shapes, more workspaces than counter sets")
    rng = np.random.default_rng(99)
    shapes = [(8, 4, 32000, 4), (3, 2, 257, 5), (1, 4, 2049, 3), (5, 1, 5000, 2), (2, 3, 100, 8), (16, 2, 1024, 1)]
    cases = []
    for B, beam, V, K in shapes:
        logits = rng.integers(-50, 51, size=(B * beam, V)).astype(np.float32)
        cases.append((B, beam, K, torch.from_numpy(logits).to(dev), ref.beam_topk(logits, B, beam, K)))
    big = torch.empty(max(capi.beam_topk_workspace_bytes(B, beam, K) for B, beam, _, K in shapes) // 4, dtype=torch.float32, device=dev)
    launches = set()
    for it in range(150):
        B, beam, K, d, want = cases[it % len(cases)]
        _, v1, i1, fv, fi = capi.beam_topk(d, B, beam, K, workspace=big)
        launches.add(capi.beam_topk_last_launches())
        np.testing.assert_array_equal(i1.cpu().numpy(), want[1], err_msg="call %d" % it)
        np.testing.assert_array_equal(fi.cpu().numpy(), want[3], err_msg="call %d" % it)
        np.testing.assert_array_equal(fv.cpu().numpy().view(np.uint32), want[2].view(np.uint32), err_msg="call %d" % it)
    assert launches == {1}, launches
    assert capi.beam_topk_last_path() == capi.TOPK_PATH_ONE_LAUNCH
    # More workspaces alive than the library has counter sets (64 per GPU): the ones that come too late take two
    # launches and say why; nobody's set is taken from it; released sets are handed out again.
    B, beam, K, d, want = cases[0]
    held = [torch.empty(capi.beam_topk_workspace_bytes(B, beam, K) // 4, dtype=torch.float32, device=dev) for _ in range(80)]
    fallbacks = capi.counter_set_fallbacks()
    seen = []
    try:
        for w in held:
            _, _, _, fv, fi = capi.beam_topk(d, B, beam, K, workspace=w)
            seen.append((capi.beam_topk_last_launches(), capi.beam_topk_last_path()))
            np.testing.assert_array_equal(fi.cpu().numpy(), want[3])
            np.testing.assert_array_equal(fv.cpu().numpy().view(np.uint32), want[2].view(np.uint32))
        served = seen.count((1, capi.TOPK_PATH_ONE_LAUNCH))
        assert 1 <= served <= 63, seen                     # (`big` holds a set as well)
        assert seen == [(1, capi.TOPK_PATH_ONE_LAUNCH)] * served + [(2, capi.TOPK_PATH_NO_COUNTER_SET)] * (80 - served), seen
        assert capi.counter_set_fallbacks() == fallbacks + 80 - served
        # workspaces the table knows keep their one-launch form
        for w in (big, held[0], held[served - 1]):
            capi.beam_topk(d, B, beam, K, workspace=w)
            assert capi.beam_topk_last_path() == capi.TOPK_PATH_ONE_LAUNCH
        # one set given back serves exactly one newcomer
        assert capi.release_workspace(held[0]) == 1 and capi.release_workspace(held[0]) == 0
        for w, path in ((held[79], capi.TOPK_PATH_ONE_LAUNCH), (held[78], capi.TOPK_PATH_NO_COUNTER_SET),
                        (held[0], capi.TOPK_PATH_NO_COUNTER_SET)):
            _, _, _, fv, fi = capi.beam_topk(d, B, beam, K, workspace=w)
            assert capi.beam_topk_last_path() == path
            np.testing.assert_array_equal(fi.cpu().numpy(), want[3])
        # a stream under capture never needs a set
        capi.tune_set("topk_two_launches", 1)
        capi.beam_topk(d, B, beam, K, workspace=held[77])
        assert capi.beam_topk_last_path() == capi.TOPK_PATH_TWO_LAUNCHES
    finally:
        capi.tune_set("topk_two_launches", -1)
        torch.cuda.synchronize()
        for w in held:
            capi.release_workspace(w)


@pytest.mark.parametrize("forced_one_launch", [False, True])
def test_topk_graph_replays(capi, ref, dev, forced_one_launch):
    """Captured once, replayed five times with eager calls on the same workspace (and so the same arrival counters) in
    between: every replay equals the oracle.  A capturing stream gets the two-launch form unless told otherwise."""
    announce("topk under graph replay, one launch forced:", forced_one_launch)
    rng = np.random.default_rng(7)
    B, beam, V, K = 8, 4, 32000, 4
    logits = rng.integers(-1000, 1001, size=(B * beam, V)).astype(np.float32)
    want = ref.beam_topk(logits, B, beam, K)
    d = torch.from_numpy(logits).to(dev)
    ws = torch.empty(capi.beam_topk_workspace_bytes(B, beam, K) // 4, dtype=torch.float32, device=dev)
    capi.beam_topk(d, B, beam, K, workspace=ws)
    assert capi.beam_topk_last_launches() == 1
    torch.cuda.synchronize()
    capi.tune_set("topk_two_launches", 0 if forced_one_launch else -1)
    try:
        side = torch.cuda.Stream()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                capi.beam_topk(d, B, beam, K, workspace=ws)
            assert capi.beam_topk_last_launches() == (1 if forced_one_launch else 2)
    finally:
        capi.tune_set("topk_two_launches", -1)
    torch.cuda.synchronize()
    n1 = B * beam * 8 * K
    for rep in range(5):
        ws.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        fv = ws[2 * n1:2 * n1 + B * K].view(B, K).cpu().numpy()
        fi = ws[2 * n1 + B * K:2 * n1 + 2 * B * K].view(torch.int32).view(B, K).cpu().numpy()
        np.testing.assert_array_equal(fi, want[3], err_msg="replay %d" % rep)
        np.testing.assert_array_equal(fv.view(np.uint32), want[2].view(np.uint32), err_msg="replay %d" % rep)
        _, _, _, _, fi2 = capi.beam_topk(d, B, beam, K, workspace=ws)      # eager, same counters
        np.testing.assert_array_equal(fi2.cpu().numpy(), want[3])
    torch.cuda.synchronize()
    del g
    assert capi.release_workspace(ws) == 1
