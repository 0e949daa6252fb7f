"""Compiles the gfx950 HIP kernels and the C++ launcher shims into in-tree shared libraries.

    python -m onellm_amd.build            # build what is out of date
    python -m onellm_amd.build --force    # rebuild everything
    python -m onellm_amd.build --stamps   # only tests/cpp/libonellm_hip_stamps.so (attention timeline build)

Outputs (next to this file): libonellm_hip.so (the C ABI of include/onellm_hip.h), libonellm_launchers.so (the
launch* functions with oneLLM's own signatures), libonellm_gemm.so (the C ABI of include/onellm_gemm.h, over
hipBLASLt) and libonellm_layers.so (the decode-side layers of include/onellm/layers.h).
hipcc cross-compiles for gfx950 without a GPU.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
INCLUDE = os.path.join(ROOT, "include")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

LIB_HIP = os.path.join(HERE, "libonellm_hip.so")
LIB_LAUNCH = os.path.join(HERE, "libonellm_launchers.so")
LIB_GEMM = os.path.join(HERE, "libonellm_gemm.so")
LIB_LAYERS = os.path.join(HERE, "libonellm_layers.so")
# test-only: a C wrapper that drives the launcher shims with oneLLM-style Tensor objects
HARNESS_SRC = os.path.join(ROOT, "tests", "cpp", "launcher_harness.cpp")
LIB_HARNESS = os.path.join(ROOT, "tests", "cpp", "liblauncher_harness.so")
# test-only: bare access-pattern kernels (what the memory system gives each kernel's access mix); timed by bench.py
CEILINGS_SRC = os.path.join(ROOT, "tests", "cpp", "access_ceilings.hip")
LIB_CEILINGS = os.path.join(ROOT, "tests", "cpp", "libaccess_ceilings.so")
# test-only, built on request (--stamps): the kernel library with per-workgroup timeline stamps in the attention kernels
LIB_STAMPS = os.path.join(ROOT, "tests", "cpp", "libonellm_hip_stamps.so")
# test-only: a stand-alone C++ program that runs one decode step through the layers, like the reference's example driver
DRIVER_SRC = os.path.join(ROOT, "tests", "cpp", "self_decoder_driver.cpp")
DRIVER_BIN = os.path.join(ROOT, "tests", "cpp", "self_decoder_driver")

KERNEL_SOURCES = ["decode_attn.hip", "norms.hip", "kv_cache.hip", "beam_topk.hip", "prefill_rope.hip", "activation.hip", "sampling.hip",
                  "tuning.cpp", "counter_sets.cpp"]
LAUNCHER_SOURCES = ["launchers.cpp"]
GEMM_SOURCES = ["linear.hip", "skinny_gemm.hip"]
LAYER_SOURCES = ["layers.cpp", "layers_capi.cpp"]

# packed fp32 VALU forms are switched off on purpose (code generation only; scalar fp32 code is
# what the kernels are written in)
COMMON = ["-O3", "-std=c++17", "-fPIC", "-I" + INCLUDE, "-I" + CSRC, "-Wall", "-Wno-unused-function"]
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# Kernels whose workgroups live a few microseconds get their first kernel arguments handed over in scalar
# registers at wave launch instead of fetching them first (gfx950 kernel-argument preload, up to 16 dwords;
# the code object keeps the ordinary fetch as its entry for a loader that does not preload).  Measured on
# MI355X: RMSNorm 8192 x 4096 fp16 22.2 -> 21.7 us.
PRELOAD_KERNARGS = ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
PRELOAD_SOURCES = {"norms.hip", "activation.hip", "kv_cache.hip", "prefill_rope.hip"}


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))]
    for d, _, fs in os.walk(INCLUDE):
        hs += [os.path.join(d, f) for f in fs if f.endswith(".h")]
    return hs


def _compile(src, force):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if not force and not _newer(obj, [path] + _headers()):
        return obj
    cmd = [HIPCC, "-c", path, "-o", obj] + COMMON
    if src.endswith(".hip"):
        # (the compiler's per-kernel register / occupancy / scratch remarks are kept next to the object:
        # tests/test_kernel_resources.py holds the kernels to their budgets)
        cmd += DEVICE + ["-Rpass-analysis=kernel-resource-usage"]
        if src in PRELOAD_SOURCES and os.environ.get("ONELLM_NO_KERNARG_PRELOAD") != "1":
            cmd += PRELOAD_KERNARGS
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr[-4000:]))
    if src.endswith(".hip"):
        with open(resources_file(src), "w") as f:
            f.write(r.stderr)
    return obj


def resources_file(src):
    """Where the build leaves hipcc's kernel-resource-usage remarks of one .hip source."""
    return os.path.join(OBJ, os.path.splitext(src)[0] + ".resources.txt")


def kernel_resources(src):
    """{demangled-ish kernel symbol: {"vgprs", "agprs", "sgprs", "occupancy", "scratch", "lds"}} from the last build of src."""
    import re
    out = {}
    with open(resources_file(src)) as f:
        text = f.read()
    for block in re.split(r"remark: [^\n]*Function Name: ", text)[1:]:
        name = block.split("\n")[0].split(" ")[0]

        def field(label):
            m = re.search(label + r": (\d+)", block)
            return int(m.group(1)) if m else None
        out[name] = dict(vgprs=field("VGPRs"), agprs=field("AGPRs"), sgprs=field("SGPRs"),
                         occupancy=field(r"Occupancy \[waves/SIMD\]"), scratch=field(r"ScratchSize \[bytes/lane\]"),
                         lds=field(r"LDS Size \[bytes/block\]"))
    return out


def build_stamps():
    """The kernel library once more with -DONELLM_ATTN_STAMPS (tests/attn_timeline.py loads it): every attention
    workgroup records when it started and ended and which XCD it ran on."""
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    for src in KERNEL_SOURCES:
        obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".stamps.o")
        cmd = [HIPCC, "-c", os.path.join(CSRC, src), "-o", obj, "-DONELLM_ATTN_STAMPS"] + COMMON
        if src.endswith(".hip"):
            cmd += DEVICE + (PRELOAD_KERNARGS if src in PRELOAD_SOURCES else [])
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s (stamps):\n%s" % (src, r.stderr[-4000:]))
        objs.append(obj)
    subprocess.run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_STAMPS] + objs, check=True)
    return LIB_STAMPS


def build(force=False, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=6) as ex:
        kobjs = list(ex.map(lambda s: _compile(s, force), KERNEL_SOURCES))
        lobjs = list(ex.map(lambda s: _compile(s, force), LAUNCHER_SOURCES))
        gobjs = list(ex.map(lambda s: _compile(s, force), GEMM_SOURCES))
        yobjs = list(ex.map(lambda s: _compile(s, force), LAYER_SOURCES))
    if force or _newer(LIB_HIP, kobjs):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_HIP] + kobjs
        subprocess.run(cmd, check=True, capture_output=not verbose)
    if force or _newer(LIB_LAUNCH, lobjs + [LIB_HIP]):
        cmd = [HIPCC, "-shared", "-fPIC", "-o", LIB_LAUNCH] + lobjs + \
              ["-L" + HERE, "-lonellm_hip", "-Wl,-rpath,$ORIGIN"]
        subprocess.run(cmd, check=True, capture_output=not verbose)
    if os.path.exists(HARNESS_SRC) and (force or _newer(LIB_HARNESS, [HARNESS_SRC, LIB_LAUNCH] + _headers())):
        cmd = [HIPCC, "-shared", "-fPIC", "-O2", "-std=c++17", "-I" + INCLUDE, "-I" + CSRC, HARNESS_SRC, "-o", LIB_HARNESS,
               "-L" + HERE, "-lonellm_launchers", "-lonellm_hip", "-Wl,-rpath,$ORIGIN/../../onellm_amd"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for the launcher harness:\n" + r.stderr[-4000:])
    if os.path.exists(CEILINGS_SRC) and (force or _newer(LIB_CEILINGS, [CEILINGS_SRC])):
        cmd = [HIPCC, "-shared", "-fPIC", "-O3", "-std=c++17", CEILINGS_SRC, "-o", LIB_CEILINGS] + DEVICE + PRELOAD_KERNARGS
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for the access-ceiling kernels:\n" + r.stderr[-4000:])
    if force or _newer(LIB_GEMM, gobjs + [LIB_HIP]):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_GEMM] + gobjs + \
              ["-L" + HERE, "-lonellm_hip", "-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,$ORIGIN"]
        subprocess.run(cmd, check=True, capture_output=not verbose)
    if force or _newer(LIB_LAYERS, yobjs + [LIB_GEMM, LIB_LAUNCH]):
        cmd = [HIPCC, "-shared", "-fPIC", "-o", LIB_LAYERS] + yobjs + \
              ["-L" + HERE, "-lonellm_gemm", "-lonellm_launchers", "-lonellm_hip", "-Wl,-rpath,$ORIGIN"]
        subprocess.run(cmd, check=True, capture_output=not verbose)
    if os.path.exists(DRIVER_SRC) and (force or _newer(DRIVER_BIN, [DRIVER_SRC, LIB_LAYERS] + _headers())):
        cmd = [HIPCC, "-O2", "-std=c++17", "-I" + INCLUDE, DRIVER_SRC, "-o", DRIVER_BIN, "-L" + HERE, "-lonellm_layers",
               "-lonellm_gemm", "-lonellm_launchers", "-lonellm_hip", "-Wl,-rpath,$ORIGIN/../../onellm_amd"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for the decoder driver:\n" + r.stderr[-4000:])
    return LIB_HIP, LIB_LAUNCH, LIB_GEMM, LIB_LAYERS


if __name__ == "__main__":
    if "--stamps" in sys.argv:
        print(build_stamps())
    else:
        libs = build(force="--force" in sys.argv, verbose=True)
        print("\n".join(libs))
