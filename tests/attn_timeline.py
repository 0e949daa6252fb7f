"""Per-workgroup timeline of a decode-attention launch: when each workgroup ended and on which XCD it ran.

    python -m onellm_amd.build --stamps          # builds tests/cpp/libonellm_hip_stamps.so (once)
    python tests/attn_timeline.py [config2|config2_ctx512|config2_ctx16|config3|config3_full] [phases] [knob=value ...]

Runs the kernel library built with -DONELLM_ATTN_STAMPS (the product sources plus two clock stamps per workgroup and
the XCC id register) on synthetic inputs of the named BASELINE shape and prints, per XCD and per dispatch half
(workgroups i and i + 256 land on the same compute unit), the mean / min / max end time in microseconds after the
first workgroup's entry, over eight launches on rotating cache sets.  With `phases` (matrix-core kernels: config3,
config3_full) it also prints, for the workgroups grouped by the number of unit pieces in their share, when each piece
was begun, how long its set-up, its streaming loop and its finish took, and how long a change of unit takes from the
last row of one piece to the first score of the next.  A measurement aid for the tables under profiles/, not a test:
pytest does not collect it."""
import ctypes
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from onellm_amd import capi  # noqa: E402

SHAPES = {
    "config2": dict(B=16, Hq=32, Hkv=32, S=4096, t=4096, ragged=False, nsets=4),
    "config2_ctx512": dict(B=16, Hq=32, Hkv=32, S=4096, t=512, ragged=False, nsets=4),
    "config2_ctx16": dict(B=16, Hq=32, Hkv=32, S=4096, t=16, ragged=False, nsets=4),       # launch and drain only
    "config3": dict(B=32, Hq=32, Hkv=8, S=8192, t=8192, ragged=True, nsets=3),
    "config3_full": dict(B=32, Hq=32, Hkv=8, S=8192, t=8192, ragged=False, nsets=3),
}


def main():
    name = sys.argv[1] if len(sys.argv) > 1 else "config2"
    c = SHAPES[name]
    lib_path = os.path.join(ROOT, "tests", "cpp", "libonellm_hip_stamps.so")
    assert os.path.exists(lib_path), "build it first: python -m onellm_amd.build --stamps"
    capi.LIB_PATH = lib_path
    L = capi.lib()
    L.onellm_attn_set_stamp_buffer.argtypes = [ctypes.c_void_p]
    L.onellm_attn_set_stamp_buffer.restype = None
    phases = "phases" in sys.argv[2:]
    for kv in [x for x in sys.argv[2:] if x != "phases"]:      # internal tuning knobs, e.g. attn_balanced_wgs=512
        key, value = kv.split("=")
        capi.tune_set(key, int(value))
        print("knob", key, "=", value)
    dev = torch.device("cuda:0")
    D = 128
    B, Hq, Hkv, S, t = c["B"], c["Hq"], c["Hkv"], c["S"], c["t"]
    torch.manual_seed(2)
    sets = [(torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half(), torch.randn(1, B, Hkv, S, D, device=dev).mul_(0.5).half())
            for _ in range(c["nsets"])]
    qkv = torch.randn(B, Hq + 2 * Hkv, D, device=dev).mul_(0.5).half()
    bias = torch.randn((Hq + 2 * Hkv) * D, device=dev).mul_(0.5).half()
    out = torch.zeros(B, Hq * D, dtype=torch.float16, device=dev)
    t_dev = None
    if c["ragged"]:
        t_dev = torch.from_numpy(np.random.default_rng(3).integers(1024, S + 1, size=B).astype(np.int32)).to(dev)
    ws = torch.zeros(capi.decode_attn_workspace_bytes(B, Hq, Hkv, D, S), dtype=torch.uint8, device=dev)
    EVENTS = 16                                                # phase stamps per workgroup, behind the four words of each
    stamps = torch.zeros(8192 * (4 + EVENTS), dtype=torch.int64, device=dev)

    def step(i):
        kc, vc = sets[i % len(sets)]
        capi.decode_attn(qkv, bias, kc, vc, out, Hq, t, D, 10000.0, t_dev=t_dev, max_t=t, workspace=ws,
                         flags=capi.ATTN_ZEROED_WORKSPACE)

    for i in range(5):
        step(i)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for i in range(50):
        step(i)
    ev1.record()
    torch.cuda.synchronize()
    print("%s: %.1f us per step (HIP events, 50 steps, stamps off)" % (name, ev0.elapsed_time(ev1) / 50 * 1e3))
    ends, xcc, cu, alone, phase_runs = [], None, None, [], []
    for rep in range(8):
        stamps.zero_()
        torch.cuda.synchronize()
        L.onellm_attn_set_stamp_buffer(stamps.data_ptr())
        ev0.record()
        step(rep)
        ev1.record()
        torch.cuda.synchronize()
        alone.append(ev0.elapsed_time(ev1) * 1e3)
        L.onellm_attn_set_stamp_buffer(None)
        raw = stamps.cpu().numpy()
        d = raw[:8192 * 4].reshape(-1, 4)
        # a workgroup's record is (entry, end, XCD id, hardware id); the phase stamps that follow the records are clock
        # values in every word, so the records are the leading rows whose third word is an XCD id
        used = (d[:, 0] != 0) & (d[:, 2] < 16) & (d[:, 3] < 2 ** 32)
        n = int(np.argmin(used)) if not used.all() else len(used)
        if phases:
            ev = raw[n * 4:n * 4 + n * EVENTS].reshape(n, EVENTS).astype(np.float64)
            t0 = d[:n, 0].min()
            phase_runs.append(((d[:n, 0] - t0) / 100.0, (d[:n, 1] - t0) / 100.0, np.where(ev > 0, (ev - t0) / 100.0, np.nan)))
        st, en = d[:n, 0], d[:n, 1]
        xcc = d[:n, 2] & 0xF
        cu = ((d[:n, 3] >> 8) & 0xFF) | (xcc << 8)      # (XCD, shader engine, array, unit)
        ends.append((en - st.min()) / 100.0)           # 100 MHz clock
        last_start = (st.max() - st.min()) / 100.0
    e = np.mean(ends, axis=0)
    n = len(e)
    idx = np.arange(n)
    print("one launch at a time, between two events: %.1f us (median of %d)" % (float(np.median(alone)), len(alone)))
    print("workgroups %d; all started by %.1f us; end: mean %.1f, max %.1f, min %.1f us" % (n, last_start, e.mean(), e.max(), e.min()))
    half = n // 2 if n >= 512 else n
    for x in range(8):
        a = e[(xcc == x) & (idx < half)]
        line = "XCD %d: workgroups 0..%d end mean %.1f (min %.1f, max %.1f)" % (x, half - 1, a.mean(), a.min(), a.max())
        if half < n:
            b = e[(xcc == x) & (idx >= half)]
            line += " | %d..%d end mean %.1f (min %.1f, max %.1f)" % (half, n - 1, b.mean(), b.min(), b.max())
        print(line)
    by_compute_unit(ends[-1], cu)
    if phases:
        phase_table(phase_runs)


def phase_table(runs):
    """Four stamps per unit piece (begun, set-up done, last row consumed, finished), averaged over the launches, for the
    workgroups grouped by how many pieces their share holds."""
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        entry = np.mean([r[0] for r in runs], 0)
        end = np.mean([r[1] for r in runs], 0)
        ev = np.nanmean([r[2] for r in runs], 0)
    npieces = (~np.isnan(ev)).sum(1) // 4
    print("workgroups by number of pieces in their share:", {int(k): int(v) for k, v in zip(*np.unique(npieces, return_counts=True))})
    for n in sorted(set(npieces)):
        if n == 0:
            continue
        sel = npieces == n
        e = ev[sel]
        print("-- %d piece(s), %d workgroups: end mean %.1f us; entry -> first piece begun %.2f us"
              % (n, sel.sum(), end[sel].mean(), np.nanmean(e[:, 0] - entry[sel])))
        for p in range(n):
            b, s, l, f = e[:, 4 * p], e[:, 4 * p + 1], e[:, 4 * p + 2], e[:, 4 * p + 3]
            line = "   piece %d: begun at %5.1f; set-up %.2f; streaming %.2f; finish %.2f" % (p, np.nanmean(b), np.nanmean(s - b), np.nanmean(l - s), np.nanmean(f - l))
            if p + 1 < n:
                line += "; last row -> next piece's first score %.2f" % np.nanmean(e[:, 4 * (p + 1) + 1] - l)
            print(line)



def by_compute_unit(e, cu):
    """How the workgroups of the last launch were spread over the compute units, and when those of a unit with one, two,
    three ... of them ended."""
    units, counts = np.unique(cu, return_counts=True)
    print("compute units used: %d; workgroups per unit: %s" % (len(units), dict(zip(*np.unique(counts, return_counts=True)))))
    per_unit = dict(zip(units, counts))
    share = np.array([per_unit[c] for c in cu])
    for k in sorted(set(share)):
        a = e[share == k]
        print("  units with %d workgroup(s): %d workgroups end mean %.1f (min %.1f, max %.1f)" % (k, a.size, a.mean(), a.min(), a.max()))
    # when a compute unit is done with all it was given: the step ends with the last of them
    last = np.array([e[cu == c].max() for c in units])
    first = np.array([e[cu == c].min() for c in units])
    print("  a compute unit's last workgroup ends: mean %.1f, min %.1f, max %.1f, 10th / 90th percentile %.1f / %.1f; its first: mean %.1f"
          % (last.mean(), last.min(), last.max(), np.percentile(last, 10), np.percentile(last, 90), first.mean()))


if __name__ == "__main__":
    main()
