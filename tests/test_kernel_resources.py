"""Register, occupancy and scratch budgets of the gfx950 kernels, read from the remarks hipcc leaves during the
build (-Rpass-analysis=kernel-resource-usage, kept by onellm_amd/build.py next to the objects).  No GPU needed.

A kernel that quietly grows past a budget still computes the right numbers - and runs with half the waves per SIMD, or
spills its loop state to scratch memory.  The finish code of the attention kernels has done that once (64 loads in
flight in the fused merge pushed the balanced grouped-query kernels from two waves per SIMD to one), so the budgets
the measured figures rely on are pinned here."""
import os
import re

import pytest

from onellm_amd import build

SOURCES = ["decode_attn.hip", "norms.hip", "kv_cache.hip", "beam_topk.hip", "prefill_rope.hip", "activation.hip", "sampling.hip",
           "skinny_gemm.hip"]


@pytest.fixture(scope="module")
def resources():
    if not all(os.path.exists(build.resources_file(s)) for s in SOURCES):
        build.build(force=True)
    return {s: build.kernel_resources(s) for s in SOURCES}


def _matching(res, pattern):
    hits = {k: v for k, v in res.items() if re.search(pattern, k)}
    assert hits, "no kernel matches %r" % pattern
    return hits


def test_every_source_reports_its_kernels(resources):
    for src, res in resources.items():
        assert res, src
        for name, r in res.items():
            assert r["vgprs"] is not None and r["occupancy"] is not None and r["scratch"] is not None, (src, name)


def test_no_kernel_spills_to_scratch(resources):
    for src, res in resources.items():
        for name, r in res.items():
            assert r["scratch"] == 0, "%s: %s uses %d bytes of scratch per lane" % (src, name, r["scratch"])


@pytest.mark.parametrize("pattern,min_occupancy", [
    # the headline kernel (one query head per kv head, fp16, D = 128) and its balanced form: four waves per SIMD
    (r"decode_attn_split_kernelI6__halfLi16ELi1ELi4ELi4ELb[01]E", 4),
    # grouped-query heads on the matrix cores, fp16 D = 64 and 128, grid and balanced schedule: two workgroups per CU
    (r"decode_attn_gqa_mfma_kernelILi(64|128)ELi(4|8|16)E", 2),
    (r"decode_attn_gqa_mfma_kernelILi256E", 1),
    (r"decode_attn_gqa_mfma_f32_kernelILi128E", 2),
    (r"decode_attn_gqa_mfma_f32_kernelILi64E", 3),
    # merge kernels: one wave per (sequence, head), many per CU
    (r"decode_attn_merge(_balanced)?_kernel", 8),
])
def test_attention_kernels_keep_their_occupancy(resources, pattern, min_occupancy):
    for name, r in _matching(resources["decode_attn.hip"], pattern).items():
        assert r["occupancy"] >= min_occupancy, "%s: %d waves per SIMD (VGPRs %d, AGPRs %d)" % (name, r["occupancy"], r["vgprs"], r["agprs"])


def test_streaming_kernels_keep_full_occupancy(resources):
    # norm rows of up to 16 KiB (the measured shapes): 512 threads per row, four workgroups per CU = eight waves per SIMD
    for name, r in _matching(resources["norms.hip"], r"norm_row_kernelI(f|6__half)Li[12]ELi512E").items():
        assert r["occupancy"] == 8 and r["vgprs"] <= 64, (name, r)
    for src in ("kv_cache.hip", "activation.hip", "sampling.hip"):
        for name, r in resources[src].items():
            assert r["occupancy"] == 8, (src, name, r)
    # beam top-K: one 4-wave workgroup per CU is all a launch brings; the wave-wide list lives in scalar registers
    for name, r in resources["beam_topk.hip"].items():
        assert r["occupancy"] >= 4 and r["vgprs"] <= 64, (name, r)
    for name, r in _matching(resources["prefill_rope.hip"], r"rows_kernel").items():
        assert r["occupancy"] >= 4, (name, r)


def test_few_row_gemm_keeps_two_workgroups_per_compute_unit(resources):
    # the projection kernel's variants up to 16 rows: one stage of 128 columns or two of 64 leave room for two 4-wave
    # workgroups per CU (the cut runs launch 256-768 of them); the two-stage 128-column form is the one-per-CU variant
    res = resources["skinny_gemm.hip"]
    for name, r in _matching(res, r"skinny_gemm_kernelILi1ELi(1ELi4ELi8|2ELi4ELi4|1ELi4ELi4)E").items():
        assert r["occupancy"] >= 2, (name, r)
    for name, r in res.items():
        assert r["vgprs"] + r["agprs"] <= 512 and r["scratch"] == 0, (name, r)
