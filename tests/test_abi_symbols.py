"""The C-ABI library loads without a GPU and exports every function include/onellm_hip.h declares;
argument checks that happen before any launch are exercised here too (no compute calls)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "onellm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(onellm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ["onellm_decode_attn", "onellm_decode_attn_workspace_bytes", "onellm_rmsnorm",
                 "onellm_fused_add_bias_residual_rmsnorm", "onellm_kv_append", "onellm_kv_repeat",
                 "onellm_beam_topk", "onellm_beam_topk_workspace_bytes", "onellm_beam_topk_last_launches", "onellm_error_string", "onellm_hip_version",
                 "onellm_qkv_bias_rope_transpose", "onellm_silu_and_mul", "onellm_topk_sample",
                 "onellm_decode_attn_static"]:
        assert must in names


def test_library_exports_every_declared_symbol(capi):
    L = ctypes.CDLL(capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(L, name), f"{name} declared in onellm_hip.h but not exported"
    assert set(declared_functions()) == set(capi.SYMBOLS), "ctypes table and header disagree"


def test_launcher_library_exports_reference_signatures(capi):
    import subprocess
    out = subprocess.run(["nm", "-DC", capi.LAUNCHERS_PATH], capture_output=True, text=True, check=True).stdout
    for sig in ["launchDecoderMaskedMHA(Tensor*, BaseWeight&, Tensor*, Tensor*, Tensor*, Tensor*, Tensor*, LLaMAAttentionStaticParams&)",
                "launchRMSNorm(Tensor*, LayerNormWeight&, float)",
                "void launchFusedAddBiasResidualRMSNorm<float>(float*, float*, float const*, float const*, float, int, int)",
                "void launchFusedAddBiasResidualRMSNorm<__half>(__half*, __half*, __half const*, __half const*, float, int, int)",
                "launchAppendKVCache(Tensor*, Tensor*, Tensor*, Tensor*, Tensor*, Tensor*, Tensor*)",
                "launchTransposeKVCache(Tensor*, Tensor*, Tensor*, Tensor*, Tensor*, Tensor*)",
                "launchTopKforBeamSearch(float const*, int, int, float*)",
                "launchAddFusedQKVBiasTransposeAndRoPE(Tensor*, Tensor*, Tensor*, Tensor*, BaseWeight&, Tensor*, Tensor*, Tensor*, LLaMAAttentionStaticParams&)",
                "void launchAct<float>(float const*, float*, int, int)",
                "void launchAct<__half>(__half const*, __half*, int, int)",
                "launchSampling(Tensor*, Tensor*, Tensor*, Tensor*, Tensor*, std::unordered_map<"]:
        assert sig in out, sig


def test_version_and_error_strings(capi):
    L = capi.lib()
    assert L.onellm_hip_version() >= 1000
    assert b"invalid argument" in L.onellm_error_string(capi.EINVAL)
    assert b"workspace" in L.onellm_error_string(capi.EWORKSPACE)
    assert b"built-in scratch" in L.onellm_error_string(capi.ESCRATCH)
    assert L.onellm_error_string(0) == b"success"
    assert L.onellm_error_string(-99)


def test_argument_rejection_happens_before_any_launch(capi):
    L = capi.lib()
    fake = ctypes.c_void_p(0x1000)   # never dereferenced: every call below is rejected on the host
    assert L.onellm_rmsnorm(capi.FP16, None, fake, 1e-5, 4, 64, None) == capi.EINVAL
    assert L.onellm_rmsnorm(7, fake, fake, 1e-5, 4, 64, None) == capi.EINVAL
    assert L.onellm_fused_add_bias_residual_rmsnorm(capi.FP16, fake, None, None, fake, 1e-5, 4, 64, None) == capi.EINVAL
    # t > S, Hq % Hkv != 0, odd row size, missing workspace
    args = dict(dtype=capi.FP16, B=1, Hq=4, Hkv=2, D=128, S=64, layer=0, L=1, t=65)
    def attn(**kw):
        a = dict(args); a.update(kw)
        return L.onellm_decode_attn(a["dtype"], fake, None, fake, fake, fake, a["B"], a["Hq"], a["Hkv"], a["D"], a["S"],
                                    a["layer"], a["L"], a["t"], None, a["t"], 128, 10000.0, 0, 0, None, 0, None)
    assert attn() == capi.EINVAL
    assert attn(t=0) == capi.EINVAL
    assert attn(t=8, Hq=3) == capi.EINVAL
    assert attn(t=8, layer=1) == capi.EINVAL
    assert attn(t=8, D=1024) == capi.EUNSUPPORTED        # head sizes above 512 are not built
    assert attn(t=4096, S=4096) == capi.EWORKSPACE      # needs a sequence split, no workspace given
    assert L.onellm_beam_topk(fake, 1, 2, 100, 9, fake, None) == capi.EUNSUPPORTED
    assert L.onellm_beam_topk(fake, 1, 2, 0, 2, fake, None) == capi.EINVAL
    assert L.onellm_kv_append(capi.FP16, fake, fake, fake, fake, None, fake, 1, 1, 1, 8, 8, 0, 1, None) == capi.EINVAL
    assert L.onellm_kv_repeat(capi.FP16, fake, fake, fake, fake, fake, 1, 3, 2, 8, 8, 8, 0, 1, None) == capi.EINVAL


def test_workspace_size_queries(capi):
    assert capi.decode_attn_workspace_bytes(16, 32, 32, 128, 4096) >= 16 * 32 * (128 + 2) * 4
    assert capi.decode_attn_workspace_bytes(16, 32, 32, 128, 4096) % 256 == 0
    # reference layout: (2*B*beam*8*K + 2*B*K) floats (tests/unittests/test_beamsearch_topK.cu:22 in the reference tree)
    assert capi.beam_topk_workspace_bytes(1, 2, 2) == 4 * (2 * 1 * 2 * 8 * 2 + 2 * 1 * 2)
