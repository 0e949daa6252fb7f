// Library version, error strings and the internal tuning table.
#include <string.h>
#include <atomic>
#include <hip/hip_runtime_api.h>
#include "onellm_hip.h"

namespace onellm {

namespace {
struct Knob {
    const char* key;
    std::atomic<int> value;
};
// -1 = let the launcher decide.  Meant for benchmarks and sweeps, not part of the stable ABI.
Knob g_knobs[] = {
    {"norm_tpr", {-1}},          // threads per row of the norm kernels: 64 .. 1024
    {"attn_target_wgs", {-1}},   // workgroups the sequence split of decode attention aims for
    {"attn_nsplit", {-1}},       // force the number of sequence splits
    {"attn_balanced", {-1}},     // 1 / 0: force the balanced workgroup schedule of decode attention on / off
    {"attn_balanced_wgs", {-1}}, // workgroups of the balanced schedule
    {"attn_balanced_cost", {-1}}, // items a change of unit is charged with in the balanced schedule
    {"attn_fused_finish", {-1}}, // 0: keep the separate merge launch even when the workspace is declared zeroed
    {"prefill_generic", {-1}},   // 1: the index-walking prefill kernel also where the row-walking one applies
    {"attn_gqa_valu", {-1}},     // 1: grouped-query heads on the vector ALU kernel instead of the MFMA one
    {"gemm_skinny", {-1}},       // onellm_linear's own few-row kernel: 0 = never (not timed either), 1 = wherever it takes the problem; default: where the tuning run chose it
    {"gemm_skinny_config", {-1}}, // with gemm_skinny = 1: 100 * kernel variant + slices along K, instead of the timed or default choice (tests)
    {"gemm_no_library", {-1}},   // 1: onellm_linear behaves as if the GEMM library had declined the problem (tests)
    {"attn_ordered_finish", {-1}}, // 1: release on the fused finish's counter add + acquire fence in the merging piece
    {"attn_early_look", {-1}},   // 1 / 0: a piece that finds the unit's other pieces arrived merges it from its registers / never looks
    {"topk_two_launches", {-1}}, // beam top-K: 1 = always a second launch for the merge of the survivors, 0 = one launch wherever it can be (also under capture)
    {"gemm_ordered_finish", {-1}}, // 1: release on the few-row projection kernel's counter add + acquire fence in the slice that reads the sums back
    {"topk_waves", {-1}},        // beam top-K: 4 / 8 waves per stage-1 workgroup instead of the launcher's choice
    {"attn_turns", {-1}},        // 0: co-resident attention workgroups do not take turns at wave priority
};
}  // namespace

int tune_get(const char* key)
{
    for (auto& k : g_knobs)
        if (strcmp(k.key, key) == 0) return k.value.load(std::memory_order_relaxed);
    return -1;
}

}  // namespace onellm

// 1.1: ONELLM_ATTN_ZEROED_WORKSPACE, 64 KiB of arrival counters at the front of the attention workspace
// 1.2: onellm_decode_attn_static
// 1.3: onellm_release_workspace, onellm_counter_set_fallbacks, onellm_beam_topk_last_path
extern "C" int onellm_hip_version(void) { return 1003; }

extern "C" int onellm_tune_set(const char* key, int value)
{
    if (!key) return ONELLM_EINVAL;
    for (auto& k : onellm::g_knobs)
        if (strcmp(k.key, key) == 0) {
            k.value.store(value, std::memory_order_relaxed);
            return 0;
        }
    return ONELLM_EINVAL;
}

extern "C" const char* onellm_error_string(int code)
{
    switch (code) {
        case 0: return "success";
        case ONELLM_EINVAL: return "onellm: invalid argument (null pointer, non-positive size or unknown enum)";
        case ONELLM_EUNSUPPORTED: return "onellm: shape or alignment not supported by the gfx950 kernels";
        case ONELLM_EWORKSPACE: return "onellm: workspace missing or too small";
        case ONELLM_ESCRATCH: return "onellm: the step's split partials exceed the library's built-in scratch "
                                     "(ONELLM_DECODE_ATTN_STATIC_SCRATCH_BYTES); use onellm_decode_attn with a workspace";
        case ONELLM_ENOGEMMKERNEL: return "onellm: the GEMM library has no kernel for this problem; onellm_linear_allow_plain(1) permits the "
                        "plain kernel (about a hundred times slower)";
        case ONELLM_ECAPTURING: return "onellm: the call has to allocate or synchronise and its stream is being captured; run one "
                        "ordinary step on this stream first";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "onellm: unknown error code";
}
