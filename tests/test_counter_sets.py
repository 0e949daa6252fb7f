"""The table that hands out sets of arrival counters (onellm_amd/csrc/counter_sets.hpp) - the one policy of the
one-launch beam top-K and of the few-row projection kernel's runs cut along K.  Plain host logic: driven here through
the C++ test harness, no GPU.  What must hold: a set belongs to its (device, workspace) until that workspace is
released and never changes hands before; a full table answers -1 (the caller's counter-free form) and counts it;
released sets are handed out again; onellm_release_workspace reaches every table on the process-wide list."""
import ctypes
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "tests", "cpp", "liblauncher_harness.so")


@pytest.fixture(scope="module")
def H():
    assert os.path.exists(HARNESS), "build it with `python -m onellm_amd.build`"
    import torch  # noqa: F401  first, so that the HIP runtime torch ships is the one this process uses
    L = ctypes.CDLL(HARNESS)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    L.h_counter_table_new.restype = vp
    L.h_counter_table_new.argtypes = [ci, ci]
    L.h_counter_table_delete.argtypes = [vp]
    L.h_counter_table_acquire.argtypes = [vp, ci, vp, ci]
    L.h_counter_table_release.argtypes = [vp, vp]
    L.h_counter_table_stats.argtypes = [vp, ci, ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.POINTER(ctypes.c_long)]
    return L


def _stats(H, t, device=0):
    o, c, f = ctypes.c_int(), ctypes.c_int(), ctypes.c_long()
    H.h_counter_table_stats(t, device, ctypes.byref(o), ctypes.byref(c), ctypes.byref(f))
    return o.value, c.value, f.value


def _ws(i):
    return ctypes.c_void_p(0x10000 + 0x100 * i)       # never dereferenced


def test_a_workspace_keeps_its_set_and_a_full_table_says_so(H, capfd):
    t = H.h_counter_table_new(4, 0)
    try:
        sets = [H.h_counter_table_acquire(t, 0, _ws(i), 0) for i in range(4)]
        assert sorted(sets) == [0, 1, 2, 3]
        # exhaustion: a fifth workspace gets nothing, as often as it asks, and is counted; one notice on stderr
        assert H.h_counter_table_acquire(t, 0, _ws(4), 0) == -1
        assert H.h_counter_table_acquire(t, 0, _ws(5), 0) == -1
        assert _stats(H, t) == (4, 0, 2)
        err = capfd.readouterr().err
        assert err.count("[oneLLM][WARN]") == 1 and "onellm_release_workspace" in err
        # ... and nobody lost a set to it: every owner still gets the set it had
        assert [H.h_counter_table_acquire(t, 0, _ws(i), 0) for i in range(4)] == sets
        assert _stats(H, t) == (4, 0, 2)
    finally:
        H.h_counter_table_delete(t)


def test_release_frees_exactly_the_workspaces_sets(H):
    t = H.h_counter_table_new(3, 0)
    try:
        a, b, c = (H.h_counter_table_acquire(t, 0, _ws(i), 0) for i in range(3))
        assert H.h_counter_table_release(t, _ws(7)) == 0                 # unknown workspace: nothing happens
        assert H.h_counter_table_release(t, _ws(1)) == 1
        assert _stats(H, t)[0] == 2
        assert H.h_counter_table_acquire(t, 0, _ws(0), 0) == a and H.h_counter_table_acquire(t, 0, _ws(2), 0) == c
        assert H.h_counter_table_acquire(t, 0, _ws(3), 0) == b           # the freed set, and only that one, is reused
        assert H.h_counter_table_acquire(t, 0, _ws(1), 0) == -1          # the released workspace is a stranger now
        assert H.h_counter_table_release(t, _ws(3)) == 1
        assert H.h_counter_table_acquire(t, 0, _ws(1), 0) == b
    finally:
        H.h_counter_table_delete(t)


def test_sets_recorded_into_a_graph_are_remembered_and_never_taken(H):
    t = H.h_counter_table_new(2, 0)
    try:
        s0 = H.h_counter_table_acquire(t, 0, _ws(0), 1)                  # handed to a launch on a capturing stream
        s1 = H.h_counter_table_acquire(t, 0, _ws(1), 0)
        assert _stats(H, t)[:2] == (2, 1)
        assert H.h_counter_table_acquire(t, 0, _ws(1), 1) == s1          # a later captured launch marks it too
        assert _stats(H, t)[:2] == (2, 2)
        for i in range(2, 40):                                           # any number of other workspaces come and go
            assert H.h_counter_table_acquire(t, 0, _ws(i), 0) == -1
        assert H.h_counter_table_acquire(t, 0, _ws(0), 0) == s0 and H.h_counter_table_acquire(t, 0, _ws(1), 0) == s1
        assert _stats(H, t)[:2] == (2, 2)                                # (the mark stays for as long as the set is owned)
        assert H.h_counter_table_release(t, _ws(0)) == 1                 # the owner says its graphs are gone
        assert _stats(H, t)[:2] == (1, 1)
    finally:
        H.h_counter_table_delete(t)


def test_every_device_has_its_own_sets(H):
    t = H.h_counter_table_new(2, 0)
    try:
        assert H.h_counter_table_acquire(t, 0, _ws(0), 0) == 0 and H.h_counter_table_acquire(t, 0, _ws(1), 0) == 1
        assert H.h_counter_table_acquire(t, 1, _ws(2), 0) == 0           # device 1 starts with all of its sets
        assert H.h_counter_table_acquire(t, 1, _ws(0), 0) == 1           # the same pointer on another device: another owner
        assert H.h_counter_table_acquire(t, 0, _ws(2), 0) == -1
        assert H.h_counter_table_release(t, _ws(0)) == 2                 # released on every device
        assert _stats(H, t, 0)[0] == 1 and _stats(H, t, 1)[0] == 1
    finally:
        H.h_counter_table_delete(t)


def test_release_workspace_reaches_listed_tables_only(H, capi):
    L = capi.lib()
    listed, private = H.h_counter_table_new(1, 1), H.h_counter_table_new(1, 0)
    try:
        before = L.onellm_counter_set_fallbacks()
        assert H.h_counter_table_acquire(listed, 0, _ws(0), 0) == 0 and H.h_counter_table_acquire(private, 0, _ws(0), 0) == 0
        assert H.h_counter_table_acquire(listed, 0, _ws(1), 0) == -1
        assert L.onellm_counter_set_fallbacks() == before + 1            # (the private table's are not counted)
        assert H.h_counter_table_acquire(private, 0, _ws(1), 0) == -1
        assert L.onellm_counter_set_fallbacks() == before + 1
        assert L.onellm_release_workspace(_ws(0)) == 1
        assert L.onellm_release_workspace(_ws(0)) == 0
        assert L.onellm_release_workspace(None) == 0
        assert H.h_counter_table_acquire(listed, 0, _ws(1), 0) == 0
        assert H.h_counter_table_acquire(private, 0, _ws(1), 0) == -1
    finally:
        H.h_counter_table_delete(listed)
        H.h_counter_table_delete(private)
    assert L.onellm_release_workspace(_ws(1)) == 0                       # a deleted table is off the list
