"""The decode-side layers (include/onellm/layers.h: launchLinearGemm, LLaMASelfAttentionLayer, LLaMAFFNLayer,
LlamaSelfDecoder) and the projection C ABI under them (include/onellm_gemm.h), driven through the layers' C surface
(include/onellm_layers.h), which builds Tensor / TensorMap / LlamaLayerWeight objects the way
examples/cpp/decoder/self_decoder_example.cpp does.
Host-side behaviour runs without a GPU; parity against the CPU oracle (oracle/ref.py: linear, self_decoder_step — the
latter pinned on an independent library implementation in tests/test_oracle_layers.py) is marked gpu."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import announce

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_GEMM = os.path.join(ROOT, "onellm_amd", "libonellm_gemm.so")
LIB_LAYERS = os.path.join(ROOT, "onellm_amd", "libonellm_layers.so")


@pytest.fixture(scope="module")
def H():
    assert os.path.exists(LIB_LAYERS), "build it with `python -m onellm_amd.build`"
    import torch  # noqa: F401  first, so that the HIP runtime and BLAS library torch ships are the ones this process uses
    L = ctypes.CDLL(LIB_LAYERS)
    vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    pp = ctypes.POINTER(ctypes.c_void_p)
    L.onellm_layers_last_error.restype = ctypes.c_char_p
    L.onellm_layers_linear.argtypes = [ci, vp, vp, vp, ci, ci, ci, ci, ci, ci]
    L.onellm_decoder_create.restype = vp
    L.onellm_decoder_create.argtypes = [ci] * 9 + [cf, cf, ci] + [pp] * 10 + [vp]
    L.onellm_decoder_forward.argtypes = [vp, ci, vp, vp, vp, vp]
    L.onellm_decoder_destroy.argtypes = [vp]
    return L


@pytest.fixture(scope="module")
def G():
    import torch  # noqa: F401  (see H)
    L = ctypes.CDLL(LIB_GEMM)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    L.onellm_linear.argtypes = [ci, vp, vp, vp, ci, ci, ci, ci, ci, vp, ctypes.c_size_t, vp]
    L.onellm_linear_workspace_bytes.restype = ctypes.c_size_t
    return L


# ---------------------------------------------------------------- host only

def test_gemm_library_exports_what_its_header_declares(G):
    text = open(os.path.join(ROOT, "include", "onellm_gemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(onellm_[a-z0-9_]+)\s*\(", text)))
    assert names == ["onellm_linear", "onellm_linear_allow_plain", "onellm_linear_last_path", "onellm_linear_pair",
                     "onellm_linear_pair_tune", "onellm_linear_tune", "onellm_linear_workspace_bytes"]
    for n in names:
        assert hasattr(G, n)
    assert G.onellm_linear_workspace_bytes() > 0


def test_linear_rejects_bad_arguments_before_any_launch(G):
    fake = ctypes.c_void_p(0x1000)
    assert G.onellm_linear(7, fake, fake, fake, 2, 4, 4, 0, 0, None, 0, None) == -1        # unknown dtype
    assert G.onellm_linear(0, None, fake, fake, 2, 4, 4, 0, 0, None, 0, None) == -1        # null input
    assert G.onellm_linear(0, fake, fake, fake, 2, 0, 4, 0, 0, None, 0, None) == -1        # empty inner size
    assert G.onellm_linear(0, fake, fake, fake, 2, 4, 4, 3, 0, None, 0, None) == -1        # row stride below N
    assert G.onellm_linear(0, fake, fake, fake, 0, 4, 4, 0, 0, None, 0, None) == 0         # no rows: nothing to do


def test_layers_library_exports_its_c_surface(H):
    text = open(os.path.join(ROOT, "include", "onellm_layers.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(onellm_[a-z0-9_]+)\s*\(", text)))
    assert names == ["onellm_decoder_create", "onellm_decoder_destroy", "onellm_decoder_forward", "onellm_layers_allow_plain_gemm",
                     "onellm_layers_gemm_workspace_count", "onellm_layers_last_error", "onellm_layers_linear",
                     "onellm_layers_release_gemm_workspace"]
    for n in names:
        assert hasattr(H, n)


def test_layers_library_exports_reference_signatures():
    out = subprocess.run(["nm", "-DC", LIB_LAYERS], capture_output=True, text=True, check=True).stdout
    for sig in ["launchLinearGemm(Tensor*, BaseWeight&, Tensor*, bool, bool, bool)",
                "LLaMASelfAttentionLayer::forward(TensorMap&, TensorMap&, LLaMAattentionWeights&, LLaMAAttentionDynParams&)",
                "LLaMAFFNLayer::forward(TensorMap&, TensorMap&, LLaMAFFNWeights&, LLaMAAttentionDynParams&)",
                "LlamaSelfDecoder::forward(TensorMap&, std::vector<LlamaLayerWeight*, std::allocator<LlamaLayerWeight*> > const&, TensorMap&, LLaMAAttentionDynParams&)",
                "LlamaSelfDecoder::LlamaSelfDecoder(int, int, int, int, int, LLaMAAttentionStaticParams const&, float, ihipStream_t*, cublasWrapper*, BaseAllocator*, bool)"]:
        assert sig in out, sig


def test_linear_launcher_precondition_failures_throw(H):
    fake = ctypes.c_void_p(0x1000)
    assert H.onellm_layers_linear(0, None, fake, fake, 2, 4, 4, 0, 0, 0) == 1
    assert b"null tensor or weight" in H.onellm_layers_last_error()
    assert H.onellm_layers_linear(0, fake, fake, fake, 2, 4, 4, 0, 0, 1) == 1                          # second slot without a pair buffer
    assert b"shared_out_buf" in H.onellm_layers_last_error()


# ---------------------------------------------------------------- GPU parity

TOL = {np.float32: dict(rtol=2e-5, atol=2e-5), np.float16: dict(rtol=1e-2, atol=2e-3)}


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("M,K,N", [(1, 16, 16), (2, 32, 64), (3, 7, 5), (16, 4096, 12288), (16, 4096, 4096), (16, 11008, 4096),
                                   (5, 100, 36), (64, 256, 512)])
def test_linear_matches_the_oracle(H, G, ref, dtype, M, K, N):
    import torch
    announce("linear", dtype.__name__, M, K, N)
    rng = np.random.default_rng(M * 7 + N)
    if (M, K, N) == (1, 16, 16):                       # tests/unittests/test_linear.cu:60-98
        x, w = np.ones((M, K), dtype), np.ones((K, N), dtype)
    else:
        x = (rng.standard_normal((M, K)) * 0.5).astype(dtype)
        w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(dtype)
    want = ref.linear(x, w)
    dx, dw = _dev(torch, x), _dev(torch, w)
    y = torch.full((M, N), 7.0, dtype=dx.dtype, device=dx.device)
    code = 1 if dtype == np.float16 else 0
    assert H.onellm_layers_linear(code, dx.data_ptr(), dw.data_ptr(), y.data_ptr(), M, K, N, 0, 0, 0) == 0, H.onellm_layers_last_error()
    np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL[dtype])
    if K >= 4096:
        # (the library GEMM, or this library's few-row kernel where the timing run of the layer shim chose it)
        assert G.onellm_linear_last_path() in (1, 2), "the projection shapes of a 7B layer must not run the plain kernel"
    # W given as [N, K]
    dwt = _dev(torch, w.T)
    y2 = torch.zeros_like(y)
    assert H.onellm_layers_linear(code, dx.data_ptr(), dwt.data_ptr(), y2.data_ptr(), M, K, N, 1, 0, 0) == 0, H.onellm_layers_last_error()
    np.testing.assert_allclose(y2.cpu().numpy().astype(np.float64), want.astype(np.float64), **TOL[dtype])
    # the gate/up pair buffer: two projections into the two slots of [M, 2, N]
    w2 = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(dtype)
    pair = torch.full((M, 2, N), -3.0, dtype=dx.dtype, device=dx.device)
    assert H.onellm_layers_linear(code, dx.data_ptr(), dw.data_ptr(), pair.data_ptr(), M, K, N, 0, 1, 0) == 0, H.onellm_layers_last_error()
    assert H.onellm_layers_linear(code, dx.data_ptr(), _dev(torch, w2).data_ptr(), pair.data_ptr(), M, K, N, 0, 1, 1) == 0, H.onellm_layers_last_error()
    got = pair.cpu().numpy().astype(np.float64)
    np.testing.assert_allclose(got[:, 0], want.astype(np.float64), **TOL[dtype])
    np.testing.assert_allclose(got[:, 1], ref.linear(x, w2).astype(np.float64), **TOL[dtype])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,M,K,N,ldy", [
    (np.float16, 1, 64, 8, 0), (np.float16, 3, 128, 72, 0), (np.float16, 16, 4096, 4096, 0), (np.float16, 16, 11008, 4096, 0),
    (np.float16, 7, 4096, 12288, 0), (np.float16, 16, 4096, 11008, 22016), (np.float16, 32, 4096, 4096, 0),
    (np.float16, 17, 256, 136, 140), (np.float16, 16, 1024, 200, 0), (np.float16, 4, 4096, 32000, 0),
    (np.float32, 1, 64, 8, 0), (np.float32, 5, 128, 36, 40), (np.float32, 16, 4096, 4096, 0), (np.float32, 16, 11008, 4096, 0),
    (np.float32, 9, 4096, 11008, 22016), (np.float32, 32, 1024, 520, 0), (np.float32, 20, 256, 100, 0)])
def test_few_row_kernel_matches_the_oracle_in_every_configuration(G, ref, dtype, M, K, N, ldy):
    """onellm_linear's own kernel for a decode step's rows, forced (tuning key gemm_skinny = 1) through every kernel
    variant and every number of slices along K that takes the problem: parity with the oracle at the element type's
    bar, untouched padding columns, the same bits on a second call (the sliced runs reuse one workspace and its
    arrival counters)."""
    import torch
    from onellm_amd import capi
    announce("few-row linear", dtype.__name__, M, K, N, ldy)
    rng = np.random.default_rng(M * 131 + N)
    x = (rng.standard_normal((M, K)) * 0.5).astype(dtype)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(dtype)
    want = ref.linear(x, w).astype(np.float64)
    dx, dw = _dev(torch, x), _dev(torch, w)
    ld = ldy or N
    ws = torch.empty(capi.linear_workspace_bytes(), dtype=torch.uint8, device=dx.device)
    ran = []
    capi.tune_set("gemm_skinny", 1)
    try:
        for variant in range(13):
            for splits in (1, 2, 3, 4, 6, 8, 16):
                capi.tune_set("gemm_skinny_config", 100 * variant + splits)
                outs = []
                for rep in range(2):
                    y = torch.full((M, ld), float("nan"), dtype=dx.dtype, device=dx.device)
                    capi.linear(dx, dw, y, ldy=ld, workspace=ws)
                    torch.cuda.synchronize()
                    outs.append(y.cpu().numpy())
                if G.onellm_linear_last_path() != 2:
                    continue                               # (this configuration does not take the problem: the library ran)
                ran.append((variant, splits))
                got = outs[0]
                np.testing.assert_allclose(got[:, :N].astype(np.float64), want, err_msg=str((variant, splits)), **TOL[dtype])
                assert np.isnan(got[:, N:]).all(), (variant, splits)
                assert np.array_equal(outs[0][:, :N], outs[1][:, :N]), (variant, splits)
    finally:
        capi.tune_set("gemm_skinny", -1)
        capi.tune_set("gemm_skinny_config", -1)
    assert len(ran) >= 3, ran
    assert any(s > 1 for _, s in ran) or K < 128, ran


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,M,K,N", [(np.float16, 16, 4096, 11008), (np.float16, 5, 256, 72), (np.float16, 20, 512, 200),
                                         (np.float32, 16, 4096, 1408), (np.float32, 3, 256, 36)])
def test_pair_of_projections_in_one_launch_matches_two_calls_and_the_oracle(G, ref, dtype, M, K, N):
    """onellm_linear_pair (the gate / up projections into the [M, 2, N] buffer the SwiGLU kernel reads): forced through
    the one-launch configurations, both halves match the oracle and are bit-identical to two onellm_linear calls
    with the same configuration; after a tuning run the chosen form still matches."""
    import torch
    from onellm_amd import capi
    announce("linear pair", dtype.__name__, M, K, N)
    rng = np.random.default_rng(N + M)
    x = (rng.standard_normal((M, K)) * 0.5).astype(dtype)
    w0 = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(dtype)
    w1 = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(dtype)
    want0, want1 = ref.linear(x, w0).astype(np.float64), ref.linear(x, w1).astype(np.float64)
    dx, d0, d1 = _dev(torch, x), _dev(torch, w0), _dev(torch, w1)
    ws = torch.empty(capi.linear_workspace_bytes(), dtype=torch.uint8, device=dx.device)

    def run_pair():
        pair = torch.full((M, 2, N), float("nan"), dtype=dx.dtype, device=dx.device)
        capi.linear_pair(dx, d0, d1, pair, pair.view(-1)[N:], ldy=2 * N, workspace=ws)
        torch.cuda.synchronize()
        return pair.cpu().numpy()

    ran = 0
    capi.tune_set("gemm_skinny", 1)
    try:
        for variant in range(13):
            for splits in (1, 2, 4, 8):
                capi.tune_set("gemm_skinny_config", 100 * variant + splits)
                got = run_pair()
                if G.onellm_linear_last_path() != 3:
                    continue
                ran += 1
                np.testing.assert_allclose(got[:, 0].astype(np.float64), want0, err_msg=str((variant, splits)), **TOL[dtype])
                np.testing.assert_allclose(got[:, 1].astype(np.float64), want1, err_msg=str((variant, splits)), **TOL[dtype])
                two = torch.full((M, 2, N), float("nan"), dtype=dx.dtype, device=dx.device)
                capi.linear(dx, d0, two, ldy=2 * N, workspace=ws)
                capi.linear(dx, d1, two.view(-1)[N:], ldy=2 * N, workspace=ws)
                torch.cuda.synchronize()
                assert G.onellm_linear_last_path() == 2
                assert np.array_equal(got, two.cpu().numpy()), (variant, splits)
    finally:
        capi.tune_set("gemm_skinny", -1)
        capi.tune_set("gemm_skinny_config", -1)
    assert ran >= 3
    best, two_calls = capi.linear_pair_tune(capi.FP16 if dtype == np.float16 else capi.FP32, M, K, N, ldy=2 * N, workspace=ws)
    assert 0 < best <= two_calls
    got = run_pair()
    np.testing.assert_allclose(got[:, 0].astype(np.float64), want0, **TOL[dtype])
    np.testing.assert_allclose(got[:, 1].astype(np.float64), want1, **TOL[dtype])


@pytest.mark.gpu
def test_few_row_kernel_cut_runs_back_to_back_on_one_workspace(G, ref):
    """300 cut runs of mixed shapes and configurations queued back to back on one workspace (its partial sums and
    arrival counters are reused from launch to launch with nothing in between but stream order), then every output
    compared bit for bit with what the same (shape, configuration) gave when it ran alone, which in turn matches the
    oracle."""
    import torch
    from onellm_amd import capi
    announce("few-row linear, back to back")
    rng = np.random.default_rng(11)
    dev = torch.device("cuda:0")
    ws = torch.empty(capi.linear_workspace_bytes(), dtype=torch.uint8, device=dev)
    shapes = [(16, 1024, 512), (8, 2048, 1024), (16, 4096, 4096), (32, 512, 256), (3, 4096, 1536)]
    ops = []
    for M, K, N in shapes:
        x = (rng.standard_normal((M, K)) * 0.5).astype(np.float16)
        w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
        ops.append((M, K, N, _dev(torch, x), _dev(torch, w), ref.linear(x, w).astype(np.float64)))
    capi.tune_set("gemm_skinny", 1)
    try:
        alone = {}
        for si, (M, K, N, dx, dw, want) in enumerate(ops):
            for variant in range(7):
                for splits in (2, 3, 4, 8):
                    capi.tune_set("gemm_skinny_config", 100 * variant + splits)
                    y = torch.zeros((M, N), dtype=torch.float16, device=dev)
                    capi.linear(dx, dw, y, workspace=ws)
                    torch.cuda.synchronize()
                    if G.onellm_linear_last_path() != 2:
                        continue
                    got = y.cpu().numpy()
                    np.testing.assert_allclose(got.astype(np.float64), want, **TOL[np.float16])
                    alone[(si, variant, splits)] = got
        keys = sorted(alone)
        assert len(keys) >= 40, len(keys)
        order = [keys[i] for i in rng.integers(0, len(keys), size=300)]
        outs = []
        for n, (si, variant, splits) in enumerate(order):
            M, K, N, dx, dw, _ = ops[si]
            capi.tune_set("gemm_skinny_config", 100 * variant + splits)
            # every fifth call hands its sums over in the formally ordered way (release on the counter add, acquire
            # fence in the slice that reads them back); the default relies on written-through stores and an add
            # executed at memory.  Same sums in the same order: same bits.
            capi.tune_set("gemm_ordered_finish", 1 if n % 5 == 4 else -1)
            y = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
            capi.linear(dx, dw, y, workspace=ws)
            outs.append(y)
        torch.cuda.synchronize()
        for k, y in zip(order, outs):
            assert np.array_equal(y.cpu().numpy(), alone[k]), k
    finally:
        capi.tune_set("gemm_skinny", -1)
        capi.tune_set("gemm_skinny_config", -1)
        capi.tune_set("gemm_ordered_finish", -1)


@pytest.mark.gpu
def test_few_row_kernel_without_a_free_counter_set_runs_uncut_and_says_so(G, ref):
    """A run cut along K counts its slices in one of the library's 128 counter sets per GPU, owned by the workspace
    from its first cut run on.  The 129th workspace gets none: the call runs the same kernel uncut (path 4), with the
    same result to the tolerance, never with somebody else's counters; after onellm_release_workspace of one owner
    the next workspace is served again."""
    import torch
    from onellm_amd import capi
    announce("few-row linear, counter sets exhausted")
    rng = np.random.default_rng(12)
    dev = torch.device("cuda:0")
    M, K, N = 16, 1024, 512
    x = (rng.standard_normal((M, K)) * 0.5).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    want = ref.linear(x, w).astype(np.float64)
    dx, dw = _dev(torch, x), _dev(torch, w)
    # one allocation cut into 1 MiB workspaces: distinct pointers, all alive (what the kernel needs here is 256 KiB)
    pool = torch.empty(140 << 20, dtype=torch.uint8, device=dev)
    spaces = [pool[i << 20:(i + 1) << 20] for i in range(140)]
    capi.tune_set("gemm_skinny", 1)
    capi.tune_set("gemm_skinny_config", 100 * 0 + 4)
    fallbacks = capi.counter_set_fallbacks()
    try:
        paths = []
        for ws in spaces[:132]:
            y = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
            capi.linear(dx, dw, y, workspace=ws)
            paths.append(G.onellm_linear_last_path())
            np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), want, **TOL[np.float16])
        owners = paths.count(2)
        assert 1 <= owners <= 128 and paths[:owners] == [2] * owners and set(paths[owners:]) == {4}, paths
        assert capi.counter_set_fallbacks() == fallbacks + (132 - owners)
        # an owner keeps being served while strangers are turned away
        y = torch.zeros((M, N), dtype=torch.float16, device=dev)
        capi.linear(dx, dw, y, workspace=spaces[0])
        assert G.onellm_linear_last_path() == 2
        # give one set back: exactly one more workspace can run cut
        assert capi.release_workspace(spaces[1]) == 1
        for ws, expect in ((spaces[135], 2), (spaces[136], 4), (spaces[1], 4)):
            y = torch.full((M, N), float("nan"), dtype=torch.float16, device=dev)
            capi.linear(dx, dw, y, workspace=ws)
            assert G.onellm_linear_last_path() == expect
            np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), want, **TOL[np.float16])
    finally:
        capi.tune_set("gemm_skinny", -1)
        capi.tune_set("gemm_skinny_config", -1)
        for ws in spaces:
            capi.release_workspace(ws)


@pytest.mark.gpu
def test_few_row_kernel_declines_what_it_is_not_built_for(G, ref):
    """Forced or not, a problem outside the kernel's rules (rows of W that are not whole 16-byte pieces, W as [N, K],
    too many rows, K not in whole 64-row blocks, a misaligned operand) runs the library as before."""
    import torch
    from onellm_amd import capi
    capi.tune_set("gemm_skinny", 1)
    try:
        for dtype, M, K, N, nk, shift in [(np.float32, 4, 128, 66, False, 0), (np.float16, 4, 128, 64, True, 0), (np.float16, 33, 128, 64, False, 0),
                                          (np.float16, 4, 96, 64, False, 0), (np.float16, 4, 128, 68, False, 0), (np.float16, 4, 128, 64, False, 1)]:
            announce("few-row linear declines", dtype.__name__, M, K, N, nk, shift)
            rng = np.random.default_rng(K + N)
            x = (rng.standard_normal((M, K)) * 0.5).astype(dtype)
            w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(dtype)
            dx = _dev(torch, x)
            wbuf = torch.zeros(K * N + 8, dtype=dx.dtype, device=dx.device)
            dw = wbuf[shift:shift + K * N].view(N, K) if nk else wbuf[shift:shift + K * N].view(K, N)
            dw.copy_(_dev(torch, w.T if nk else w))
            y = torch.zeros((M, N), dtype=dx.dtype, device=dx.device)
            rc = G.onellm_linear(1 if dtype == np.float16 else 0, dx.data_ptr(), dw.data_ptr(), y.data_ptr(), M, K, N, 0, int(nk), None, 0, None)
            torch.cuda.synchronize()
            assert rc == 0 and G.onellm_linear_last_path() != 2
            np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), ref.linear(x, w).astype(np.float64), **TOL[dtype])
    finally:
        capi.tune_set("gemm_skinny", -1)


@pytest.mark.gpu
def test_tuning_run_times_the_few_row_kernel_and_keeps_results_right(G, ref):
    """onellm_linear_tune on a decode-step projection (cold weights: it rotates over copies of W) leaves a plan -
    the library's algorithm or this library's kernel, whichever was faster - that still matches the oracle; with
    gemm_skinny = 0 the plan is the library's."""
    import torch
    from onellm_amd import capi
    M, K, N = 16, 2048, 4096
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((M, K)) * 0.5).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    want = ref.linear(x, w).astype(np.float64)
    dx, dw = _dev(torch, x), _dev(torch, w)
    ws = torch.empty(capi.linear_workspace_bytes(), dtype=torch.uint8, device=dx.device)
    announce("linear tune", M, K, N)
    best, first = capi.linear_tune(capi.FP16, M, K, N, workspace=ws)
    assert 0 < best <= first * 1.5
    y = torch.zeros((M, N), dtype=torch.float16, device=dx.device)
    capi.linear(dx, dw, y, workspace=ws)
    torch.cuda.synchronize()
    assert G.onellm_linear_last_path() in (1, 2)
    np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), want, **TOL[np.float16])
    capi.tune_set("gemm_skinny", 0)
    try:
        y.zero_()
        capi.linear(dx, dw, y, workspace=ws)
        torch.cuda.synchronize()
        assert G.onellm_linear_last_path() == 1
        np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), want, **TOL[np.float16])
    finally:
        capi.tune_set("gemm_skinny", -1)


def _random_layers(rng, dtype, Hq, Hkv, D, I, L, bias=True):
    hidden = Hq * D
    out = []
    for _ in range(L):
        out.append({
            "attn_norm": rng.uniform(0.5, 1.5, hidden).astype(dtype), "ffn_norm": rng.uniform(0.5, 1.5, hidden).astype(dtype),
            "wqkv": (rng.standard_normal((hidden, (Hq + 2 * Hkv) * D)) / np.sqrt(hidden)).astype(dtype),
            "bqkv": (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.1).astype(dtype) if bias else None,
            "wo": (rng.standard_normal((hidden, hidden)) / np.sqrt(hidden)).astype(dtype),
            "bo": (rng.standard_normal(hidden) * 0.1).astype(dtype) if bias else None,
            "wgate": (rng.standard_normal((hidden, I)) / np.sqrt(hidden)).astype(dtype),
            "wup": (rng.standard_normal((hidden, I)) / np.sqrt(hidden)).astype(dtype),
            "wdown": (rng.standard_normal((I, hidden)) / np.sqrt(I)).astype(dtype),
            "bdown": (rng.standard_normal(hidden) * 0.1).astype(dtype) if bias else None,
        })
    return out


class GpuDecoder:
    """capi.SelfDecoder over device copies of numpy `layers`."""

    def __init__(self, H, torch, dtype, B, Hq, Hkv, D, I, S, rotary_dim, base, eps, layers, output_norm, attn_bias=True):
        from onellm_amd import capi
        self.torch = torch
        dl = [{k: (None if v is None else _dev(torch, v)) for k, v in w.items()} for w in layers]
        self.dec = capi.SelfDecoder(1 if dtype == np.float16 else 0, B, Hq, Hkv, D, I, S, rotary_dim, base, eps, dl,
                                    _dev(torch, output_norm), attn_bias=attn_bias)

    def forward(self, step, x, y, kc, vc):
        self.dec.forward(step, x, y, kc, vc)
        self.torch.cuda.synchronize()

    def close(self):
        self.dec.close()


STEP_TOL = {np.float32: dict(rtol=2e-4, atol=2e-4), np.float16: dict(rtol=3e-2, atol=3e-2)}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,B,Hq,Hkv,D,I,L,S,t,rotary", [
    (np.float32, 2, 4, 2, 8, 12, 2, 12, 3, 128),        # examples/cpp/decoder/self_decoder_example.cpp:10-27
    (np.float32, 3, 8, 2, 64, 172, 2, 40, 33, 64),
    (np.float16, 4, 8, 2, 128, 1024, 2, 300, 257, 128),
    (np.float16, 2, 32, 32, 128, 1408, 1, 64, 64, 128),
    (np.float16, 1, 4, 4, 64, 96, 3, 16, 1, 64),
])
@pytest.mark.parametrize("projections", ["tuned", "library_only"])
def test_decoder_step_matches_the_oracle(H, ref, dtype, B, Hq, Hkv, D, I, L, S, t, rotary, projections):
    """`library_only` (tuning key gemm_skinny = 0) is the path the task statement names: every projection on hipBLASLt.
    `tuned` lets the tuning run pick this library's few-row kernel where it measured faster (an extension)."""
    import torch
    from onellm_amd import capi
    announce("decoder step", dtype.__name__, B, Hq, Hkv, D, I, L, S, "t", t, projections)
    capi.tune_set("gemm_skinny", 0 if projections == "library_only" else -1)
    try:
        _decoder_step_case(H, ref, torch, dtype, B, Hq, Hkv, D, I, L, S, t, rotary)
    finally:
        capi.tune_set("gemm_skinny", -1)


def _decoder_step_case(H, ref, torch, dtype, B, Hq, Hkv, D, I, L, S, t, rotary):
    rng = np.random.default_rng(B * 1000 + Hq * 10 + t)
    hidden, eps = Hq * D, 1e-5
    layers = _random_layers(rng, dtype, Hq, Hkv, D, I, L)
    out_norm = rng.uniform(0.5, 1.5, hidden).astype(dtype)
    x = rng.standard_normal((B, hidden)).astype(dtype)
    kc = np.zeros((L, B, Hkv, S, D), dtype)
    vc = np.zeros((L, B, Hkv, S, D), dtype)
    kc[:, :, :, :t - 1] = (rng.standard_normal((L, B, Hkv, t - 1, D)) * 0.5).astype(dtype)
    vc[:, :, :, :t - 1] = (rng.standard_normal((L, B, Hkv, t - 1, D)) * 0.5).astype(dtype)

    r_x, r_kc, r_vc = x.copy(), kc.copy(), vc.copy()
    want = ref.self_decoder_step(r_x, layers, out_norm, r_kc, r_vc, Hq, t, rotary, 10000.0, eps)

    dec = GpuDecoder(H, torch, dtype, B, Hq, Hkv, D, I, S, rotary, 10000.0, eps, layers, out_norm)
    try:
        g_x, g_kc, g_vc = _dev(torch, x), _dev(torch, kc), _dev(torch, vc)
        g_y = torch.zeros_like(g_x)
        dec.forward(t, g_x, g_y, g_kc, g_vc)
        f64 = lambda a: a.cpu().numpy().astype(np.float64)
        np.testing.assert_allclose(f64(g_y), want.astype(np.float64), **STEP_TOL[dtype])
        np.testing.assert_allclose(f64(g_x), r_x.astype(np.float64), **STEP_TOL[dtype])            # residual stream
        np.testing.assert_allclose(f64(g_kc), r_kc.astype(np.float64), **STEP_TOL[dtype])          # row t-1 of every layer
        np.testing.assert_allclose(f64(g_vc), r_vc.astype(np.float64), **STEP_TOL[dtype])
        assert np.abs(f64(g_y) - want.astype(np.float64)).mean() < (2e-5 if dtype == np.float32 else 4e-3)
        # history rows and rows past t are untouched, bit for bit
        got_k = g_kc.cpu().numpy()
        np.testing.assert_array_equal(got_k[:, :, :, :t - 1].view(np.uint8), kc[:, :, :, :t - 1].view(np.uint8))
        assert not got_k[:, :, :, t:].any()
        # a second step on the grown cache, buffers recycled by the allocator
        x2 = rng.standard_normal((B, hidden)).astype(dtype)
        if t < S:
            r_x2 = x2.copy()
            want2 = ref.self_decoder_step(r_x2, layers, out_norm, r_kc, r_vc, Hq, t + 1, rotary, 10000.0, eps)
            g_x2 = _dev(torch, x2)
            dec.forward(t + 1, g_x2, g_y, g_kc, g_vc)
            np.testing.assert_allclose(f64(g_y), want2.astype(np.float64), **STEP_TOL[dtype])
    finally:
        dec.close()


@pytest.mark.gpu
def test_decoder_without_attention_bias_and_reference_rope_position(H, ref):
    """attn_bias = false drops the qkv / output biases (src/weights/llama/layer_weights.cc:26-29)."""
    import torch
    announce("decoder step without biases")
    rng = np.random.default_rng(5)
    dtype, B, Hq, Hkv, D, I, L, S, t = np.float32, 2, 4, 2, 16, 24, 2, 10, 6
    hidden = Hq * D
    layers = _random_layers(rng, dtype, Hq, Hkv, D, I, L, bias=False)
    out_norm = rng.uniform(0.5, 1.5, hidden).astype(dtype)
    x = rng.standard_normal((B, hidden)).astype(dtype)
    kc = (rng.standard_normal((L, B, Hkv, S, D)) * 0.5).astype(dtype)
    vc = (rng.standard_normal((L, B, Hkv, S, D)) * 0.5).astype(dtype)
    r_x, r_kc, r_vc = x.copy(), kc.copy(), vc.copy()
    want = ref.self_decoder_step(r_x, layers, out_norm, r_kc, r_vc, Hq, t, D, 10000.0, 1e-5)
    dec = GpuDecoder(H, torch, dtype, B, Hq, Hkv, D, I, S, D, 10000.0, 1e-5, layers, out_norm, attn_bias=False)
    try:
        g_x, g_kc, g_vc = _dev(torch, x), _dev(torch, kc), _dev(torch, vc)
        g_y = torch.zeros_like(g_x)
        dec.forward(t, g_x, g_y, g_kc, g_vc)
        np.testing.assert_allclose(g_y.cpu().numpy(), want, **STEP_TOL[dtype])
        np.testing.assert_allclose(g_kc.cpu().numpy(), r_kc, **STEP_TOL[dtype])
    finally:
        dec.close()


@pytest.mark.gpu
def test_standalone_cpp_driver_matches_the_oracle(ref):
    """tests/cpp/self_decoder_driver.cpp is a C++ program written against onellm/layers.h with the shapes and constants
    of examples/cpp/decoder/self_decoder_example.cpp; it runs in its own process (system HIP runtime and hipBLASLt, no
    PyTorch) and prints its results."""
    announce("stand-alone C++ decoder driver")
    exe = os.path.join(ROOT, "tests", "cpp", "self_decoder_driver")
    assert os.path.exists(exe), "build it with `python -m onellm_amd.build`"
    run = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
    rows = {}
    for line in run.stdout.splitlines():
        name, *vals = line.split()
        rows.setdefault(name, []).append(np.array([float(v) for v in vals], np.float32))

    B, Hq, Hkv, D, I, L, S, t = 2, 4, 2, 8, 12, 2, 12, 3
    hidden, f = Hq * D, np.float32
    layer = {"attn_norm": np.ones(hidden, f), "ffn_norm": np.ones(hidden, f), "wqkv": np.ones((hidden, (Hq + 2 * Hkv) * D), f),
             "bqkv": np.full((Hq + 2 * Hkv) * D, 2, f), "wo": np.ones((hidden, hidden), f), "bo": np.full(hidden, 2, f),
             "wgate": np.full((hidden, I), 2, f), "wup": np.ones((hidden, I), f), "wdown": np.full((I, hidden), 2, f),
             "bdown": np.zeros(hidden, f)}
    x = np.ones((B, hidden), f)
    kc, vc = np.ones((L, B, Hkv, S, D), f), np.ones((L, B, Hkv, S, D), f)
    want = ref.self_decoder_step(x, [layer] * L, np.full(hidden, 2, f), kc, vc, Hq, t, 128, 10000.0, 1e-16)
    np.testing.assert_allclose(rows["decoder_output"][0], want.reshape(-1), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(rows["residual"][0], x.reshape(-1), rtol=1e-4)
    for l in range(L):
        np.testing.assert_allclose(rows["k_row"][l], kc[l, 0, 0, t - 1], rtol=1e-4, atol=1e-4)
        np.testing.assert_allclose(rows["v_row"][l], vc[l, 0, 0, t - 1], rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
def test_decoder_step_captured_into_a_graph_replays_identically(H, ref):
    """A decoder built on a side stream: after one ordinary step (buffers, attention workspace and GEMM plans exist)
    a step is captured into a HIP graph and replayed with eager work and synchronisations in between; every replay
    must reproduce the eager step bit for bit (output, residual stream and caches)."""
    import torch
    from onellm_amd import capi
    announce("decoder step under graph capture")
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(77)
    dtype, B, Hq, Hkv, D, I, L, S, t = np.float16, 4, 16, 4, 128, 1536, 2, 600, 577
    hidden = Hq * D
    layers = _random_layers(rng, dtype, Hq, Hkv, D, I, L)
    out_norm = rng.uniform(0.5, 1.5, hidden).astype(dtype)
    x0 = _dev(torch, rng.standard_normal((B, hidden)).astype(dtype))
    kc0 = _dev(torch, (rng.standard_normal((L, B, Hkv, S, D)) * 0.5).astype(dtype))
    vc0 = _dev(torch, (rng.standard_normal((L, B, Hkv, S, D)) * 0.5).astype(dtype))
    side = torch.cuda.Stream()
    dl = [{k: (None if v is None else _dev(torch, v)) for k, v in w.items()} for w in layers]
    dec = capi.SelfDecoder(capi.FP16, B, Hq, Hkv, D, I, S, D, 10000.0, 1e-5, dl, _dev(torch, out_norm), stream=side.cuda_stream)
    x, y, kc, vc = x0.clone(), torch.zeros_like(x0), kc0.clone(), vc0.clone()

    def restore():
        x.copy_(x0); y.zero_(); kc.copy_(kc0); vc.copy_(vc0)

    def snapshot():
        torch.cuda.synchronize()
        return [a.clone() for a in (x, y, kc, vc)]

    try:
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            restore()
            dec.forward(t, x, y, kc, vc)                   # eager, on the decoder's stream: also the warm-up
        want = snapshot()
        # against the oracle too, so that "identical" is not "identically wrong"
        r_x, r_kc, r_vc = x0.cpu().numpy().copy(), kc0.cpu().numpy().copy(), vc0.cpu().numpy().copy()
        r_y = ref.self_decoder_step(r_x, layers, out_norm, r_kc, r_vc, Hq, t, D, 10000.0, 1e-5)
        np.testing.assert_allclose(want[1].cpu().numpy().astype(np.float64), r_y.astype(np.float64), **STEP_TOL[dtype])

        restore()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            dec.forward(t, x, y, kc, vc)
        for replay in range(4):
            restore()
            (x0.float() * 2).sum().item()                  # eager work and a synchronisation between replays
            g.replay()
            got = snapshot()
            for a, b in zip(got, want):
                assert torch.equal(a, b), f"replay {replay} differs from the eager step"
    finally:
        torch.cuda.synchronize()
        dec.close()


# ---------------------------------------------------------------- slow or unsafe paths are loud

def _harness():
    L = ctypes.CDLL(os.path.join(ROOT, "tests", "cpp", "liblauncher_harness.so"))
    L.h_set_launch_stream.argtypes = [ctypes.c_void_p]
    L.h_set_launch_stream.restype = None
    return L


def test_new_error_codes_have_text():
    from onellm_amd import capi
    L = capi.lib()
    assert b"plain kernel" in L.onellm_error_string(capi.ENOGEMMKERNEL)
    assert b"captured" in L.onellm_error_string(capi.ECAPTURING)


@pytest.mark.gpu
def test_a_large_projection_without_a_library_kernel_is_an_error_not_a_slow_success(H, G, ref):
    """With the GEMM library out of the picture (a test knob makes onellm_linear behave as if it had declined the
    problem) a tiny product still runs - on the plain kernel, as unit-test and example sizes always did - while a
    projection of a real model's size is refused with its own code, through the C entry point and as an exception of
    launchLinearGemm, until the caller allows the hundred-times-slower kernel."""
    import torch
    from onellm_amd import capi
    announce("linear without a library kernel")
    rng = np.random.default_rng(1)
    capi.tune_set("gemm_no_library", 1)
    try:
        # (40 rows: more than this library's own few-row kernel takes, which would otherwise step in for the library)
        for (M, K, N), big in (((3, 40, 24), False), ((40, 2048, 1024), True)):
            x = (rng.standard_normal((M, K)) * 0.5).astype(np.float16)
            w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
            dx, dw = _dev(torch, x), _dev(torch, w)
            y = torch.zeros((M, N), dtype=dx.dtype, device=dx.device)
            rc = G.onellm_linear(1, dx.data_ptr(), dw.data_ptr(), y.data_ptr(), M, K, N, 0, 0, None, 0, None)
            if not big:
                assert rc == 0 and G.onellm_linear_last_path() == 0
            else:
                assert rc == capi.ENOGEMMKERNEL
                assert H.onellm_layers_linear(1, dx.data_ptr(), dw.data_ptr(), y.data_ptr(), M, K, N, 0, 0, 0) == 1
                assert b"plain kernel" in H.onellm_layers_last_error()
                torch.cuda.synchronize()
                assert not y.any()                                   # nothing ran
                assert H.onellm_layers_allow_plain_gemm(1) == 0
                try:
                    assert H.onellm_layers_linear(1, dx.data_ptr(), dw.data_ptr(), y.data_ptr(), M, K, N, 0, 0, 0) == 0, H.onellm_layers_last_error()
                    assert G.onellm_linear_last_path() == 0
                finally:
                    H.onellm_layers_allow_plain_gemm(0)
            np.testing.assert_allclose(y.cpu().numpy().astype(np.float64), ref.linear(x, w).astype(np.float64), **TOL[np.float16])
    finally:
        capi.tune_set("gemm_no_library", -1)


@pytest.mark.gpu
def test_gemm_workspace_is_per_launch_stream_and_never_created_under_capture(H):
    """Two decoders or threads that queue on different streams of one GPU must not share the library's split-K
    scratch: every launch stream gets its own buffer.  Creating one allocates, so the first projection on a stream
    that is being captured is refused with a message instead of recording an allocation into the graph."""
    import torch
    announce("gemm workspace keying")
    harness = _harness()
    dev = torch.device("cuda:0")
    x = torch.randn(4, 64, device=dev).half()
    w = torch.randn(64, 32, device=dev).half()
    y = torch.zeros(4, 32, dtype=torch.float16, device=dev)
    run = lambda: H.onellm_layers_linear(1, x.data_ptr(), w.data_ptr(), y.data_ptr(), 4, 64, 32, 0, 0, 0)
    s1, s2, s3 = torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()
    try:
        assert run() == 0                                            # null stream
        torch.cuda.synchronize()
        want = y.clone()
        before = H.onellm_layers_gemm_workspace_count()
        for k, s in enumerate((s1, s2, s1, s2)):
            harness.h_set_launch_stream(s.cuda_stream)
            y.zero_()
            torch.cuda.synchronize()
            assert run() == 0, H.onellm_layers_last_error()
            torch.cuda.synchronize()
            assert torch.equal(y, want)
            assert H.onellm_layers_gemm_workspace_count() == before + min(k + 1, 2)
        # a stream seen for the first time while it is being captured
        harness.h_set_launch_stream(s3.cuda_stream)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s3):
            x.add_(0)                                                # (something for the graph to hold)
            rc = run()
            msg = H.onellm_layers_last_error()
        assert rc == 1 and b"captured" in msg, msg
        assert H.onellm_layers_gemm_workspace_count() == before + 2
        torch.cuda.synchronize()
        assert run() == 0                                            # an ordinary call afterwards is fine
        torch.cuda.synchronize()
        assert torch.equal(y, want)
        # a stream that is about to be destroyed gives its workspace (and that workspace's counter sets) back
        count = H.onellm_layers_gemm_workspace_count()
        assert H.onellm_layers_release_gemm_workspace(ctypes.c_void_p(s1.cuda_stream)) == 1
        assert H.onellm_layers_release_gemm_workspace(ctypes.c_void_p(s1.cuda_stream)) == 0
        assert H.onellm_layers_gemm_workspace_count() == count - 1
        harness.h_set_launch_stream(s1.cuda_stream)                  # ... and gets a new one if it is used again after all
        assert run() == 0, H.onellm_layers_last_error()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
        assert H.onellm_layers_gemm_workspace_count() == count
    finally:
        harness.h_set_launch_stream(None)
