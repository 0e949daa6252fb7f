"""ctypes binding of tests/cpp/libaccess_ceilings.so: bare access-pattern kernels (pure read, fill, copy, in-place
row read-reduce-write, one-read-G-stores, token-major to head-major regrouping) whose measured rate is the ceiling of the product kernel with the same
access mix on the GPU at hand.  Test-side only: bench.py times them beside the product kernels, a GPU test checks
that each moves the bytes it claims to."""
import ctypes
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "libaccess_ceilings.so")
_vp, _ci, _sz, _cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_float
SYMBOLS = {
    "ceiling_policy_count": (_ci, []),
    "ceiling_policy_name": (ctypes.c_char_p, [_ci]),
    "ceiling_read": (_ci, [_vp, _sz, _vp, _ci, _vp]),
    "ceiling_fill": (_ci, [_vp, _sz, _cf, _ci, _vp]),
    "ceiling_copy": (_ci, [_vp, _vp, _sz, _ci, _vp]),
    "ceiling_rows": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "ceiling_fanout": (_ci, [_vp, _vp, _sz, _ci, _sz, _sz, _ci, _vp]),
    "ceiling_regroup": (_ci, [_vp, _vp, _ci, _ci, _ci, _ci, _vp]),
}
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m onellm_amd.build`")
        import torch  # noqa: F401  (its HIP runtime first, as for the product library)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _ok(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with code {rc}")


def policies():
    L = lib()
    return [L.ceiling_policy_name(i).decode() for i in range(L.ceiling_policy_count())]


def read(src, sink, policy):
    _ok(lib().ceiling_read(src.data_ptr(), src.numel() * src.element_size(), sink.data_ptr(), policy, _stream()), "ceiling_read")


def fill(dst, value, policy):
    _ok(lib().ceiling_fill(dst.data_ptr(), dst.numel() * dst.element_size(), value, policy, _stream()), "ceiling_fill")


def copy(dst, src, policy):
    assert dst.numel() * dst.element_size() == src.numel() * src.element_size()
    _ok(lib().ceiling_copy(dst.data_ptr(), src.data_ptr(), src.numel() * src.element_size(), policy, _stream()), "ceiling_copy")


def rows(a, b, shared, policy):
    """a (and b, if given) [rows, row] updated in place; shared (if given) one row-sized vector every workgroup reads."""
    n, row_bytes = a.shape[0], a.shape[1] * a.element_size()
    _ok(lib().ceiling_rows(a.data_ptr(), b.data_ptr() if b is not None else None,
                           shared.data_ptr() if shared is not None else None, n, row_bytes, policy, _stream()), "ceiling_rows")


def fanout(dst, src, G, policy, chunk=0):
    """dst [G, ...src.shape] <- src repeated G times; with chunk (bytes) the source is a row of chunks and dst holds the
    G copies of each chunk side by side ([chunks, G, chunk])."""
    nbytes = src.numel() * src.element_size()
    assert dst.numel() * dst.element_size() == G * nbytes
    _ok(lib().ceiling_fanout(dst.data_ptr(), src.data_ptr(), nbytes, G, nbytes, chunk, policy, _stream()), "ceiling_fanout")


def regroup(dst, src, seq_tokens, policy):
    """src [tokens, heads, 256 bytes] -> dst [tokens // seq_tokens, heads, seq_tokens, 256 bytes]."""
    tokens, heads = src.shape[0], src.shape[1]
    assert src[0, 0].numel() * src.element_size() == 256 and dst.numel() == src.numel()
    _ok(lib().ceiling_regroup(dst.data_ptr(), src.data_ptr(), tokens, heads, seq_tokens, policy, _stream()), "ceiling_regroup")
