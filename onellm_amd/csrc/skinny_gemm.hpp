// y[M, N] = x[M, K] . W[K, N] for a handful of rows (a decode step's batch): fp16 or fp32 operands, fp32 accumulation
// on the matrix cores, the weights streamed once.  Host interface; the kernel is in skinny_gemm.hip.
// (internal to libonellm_gemm.so: onellm_linear and onellm_linear_tune are its callers)
#pragma once
#include <stddef.h>
#include <hip/hip_runtime.h>

namespace onellm {

constexpr int kSkinnyMaxRows = 32;          // M above this goes to the library

// how one problem is run: which instantiation of the kernel, and in how many slices along K
struct SkinnyConfig {
    int variant = -1;                       // -1: not this kernel
    int splits = 0;
};

// Whether the kernel takes the problem at all (shape and layout only; pointers are checked at launch).
bool skinny_shape_ok(int dtype, int M, int K, int N, int ldy, int w_is_nk);

// Configurations worth timing for a problem - or for `problems` = 2 of them that share x and shape and go out in one
// launch - `max` at most; with_workspace_bytes bounds the slices along K (a sliced run keeps its partial sums in the
// caller's workspace).  Returns how many were written.
int skinny_candidates(int dtype, int M, int K, int N, size_t with_workspace_bytes, int problems, SkinnyConfig* out, int max);

// A reasonable configuration without timing anything (what a forced run uses); variant -1 if there is none.
SkinnyConfig skinny_default(int dtype, int M, int K, int N, size_t with_workspace_bytes, int problems);

// skinny_launch: a run cut along K found every arrival-counter set of the device owned by other workspaces; nothing
// was launched.  The caller runs the same variant uncut, or the library.
constexpr int kSkinnyNoCounterSet = -1000;

// Queues the multiplication.  0, ONELLM_EUNSUPPORTED (this kernel does not take the problem as given: alignment,
// workspace too small for a sliced run - the caller goes on to the library), kSkinnyNoCounterSet or a hipError_t.
// A sliced run (splits > 1) uses `workspace` for partial sums; calls that share a workspace must not overlap, which
// is the library's rule for the same buffer as well.
// With w_second / y_second the launch also computes y_second = x . w_second (same shape and row stride): the gate and
// up projections of a feed-forward block in one go.
int skinny_launch(SkinnyConfig c, int dtype, const void* x, const void* w, void* y, const void* w_second, void* y_second, int M, int K,
                  int N, int ldy, void* workspace, size_t workspace_bytes, hipStream_t stream);

}  // namespace onellm
