"""ctypes binding of libonellm_hip.so (the C ABI in include/onellm_hip.h) for torch tensors.

Every wrapper passes raw device pointers and launches on torch's current stream.  There is no
fallback: if the library is not built, loading raises.
"""
import ctypes
import os
import weakref

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libonellm_hip.so")
LAUNCHERS_PATH = os.path.join(_HERE, "libonellm_launchers.so")

FP32, FP16 = 0, 1
EINVAL, EUNSUPPORTED, EWORKSPACE, ESCRATCH, ENOGEMMKERNEL, ECAPTURING = -1, -2, -3, -4, -5, -6
DECODE_ATTN_STATIC_SCRATCH_BYTES = 16 << 20
ATTN_NO_V_BIAS = 0x1
ATTN_NO_CACHE_WRITE = 0x2
ATTN_ZEROED_WORKSPACE = 0x4
TOPK_BLOCKS_PER_ROW = 8
TOPK_PATH_ONE_LAUNCH, TOPK_PATH_TWO_LAUNCHES, TOPK_PATH_NO_COUNTER_SET = 1, 2, 3

# every symbol include/onellm_hip.h declares: name -> (restype, argtypes)
_vp, _ci, _cf, _cu, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_uint, ctypes.c_size_t
SYMBOLS = {
    "onellm_hip_version": (_ci, []),
    "onellm_error_string": (ctypes.c_char_p, [_ci]),
    "onellm_tune_set": (_ci, [ctypes.c_char_p, _ci]),
    "onellm_decode_attn": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _vp, _ci,
                                 _ci, _cf, _ci, _cu, _vp, _sz, _vp]),
    "onellm_decode_attn_workspace_bytes": (_sz, [_ci, _ci, _ci, _ci, _ci]),
    "onellm_decode_attn_static": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _vp, _ci,
                                        _ci, _cf, _ci, _cu, _vp]),
    "onellm_rmsnorm": (_ci, [_ci, _vp, _vp, _cf, _ci, _ci, _vp]),
    "onellm_fused_add_bias_residual_rmsnorm": (_ci, [_ci, _vp, _vp, _vp, _vp, _cf, _ci, _ci, _vp]),
    "onellm_kv_append": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _vp]),
    "onellm_kv_repeat": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _vp]),
    "onellm_beam_topk": (_ci, [_vp, _ci, _ci, _ci, _ci, _vp, _vp]),
    "onellm_beam_topk_workspace_bytes": (_sz, [_ci, _ci, _ci]),
    "onellm_beam_topk_last_launches": (_ci, []),
    "onellm_beam_topk_last_path": (_ci, []),
    "onellm_release_workspace": (_ci, [_vp]),
    "onellm_counter_set_fallbacks": (ctypes.c_long, []),
    "onellm_qkv_bias_rope_transpose": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci,
                                             _cf, _vp]),
    "onellm_silu_and_mul": (_ci, [_ci, _vp, _vp, _ci, _ci, _vp]),
    "onellm_topk_sample": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _ci, ctypes.c_ulonglong, _ci, _ci, _vp]),
}

_lib = None


class OnellmError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        msg = lib().onellm_error_string(code).decode()
        super().__init__(f"{what} failed with code {code}: {msg}")


def lib():
    """Load the HIP library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m onellm_amd.build` "
                               "(there is no CPU fallback)")
        # torch first: its wheel ships a HIP runtime of its own under the same soname, and the copy that is loaded
        # first is the one every library of the process has to share (tensors come from torch's)
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def tune_set(key, value):
    """Internal tuning knob (benchmarks only); -1 restores the automatic choice."""
    rc = lib().onellm_tune_set(key.encode(), int(value))
    if rc:
        raise OnellmError(rc, f"tune_set({key})")


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _dt(t):
    import torch
    if t.dtype == torch.float32:
        return FP32
    if t.dtype == torch.float16:
        return FP16
    raise TypeError(f"unsupported dtype {t.dtype}")


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensors only"
    return t.data_ptr()


def _check(rc, what):
    if rc != 0:
        raise OnellmError(rc, what)


def decode_attn_workspace_bytes(B, Hq, Hkv, D, max_t):
    return lib().onellm_decode_attn_workspace_bytes(B, Hq, Hkv, D, max_t)


def decode_attn(qkv, bias, k_cache, v_cache, out, Hq, t, rotary_dim, rope_base, layer=0, t_dev=None,
                max_t=None, rope_pos_offset=0, flags=0, workspace=None):
    """qkv [B, Hq+2Hkv, D]; caches [L, B, Hkv, S, D]; out [B, Hq*D]; t host int (or max of t_dev).
    `workspace` is a uint8 device tensor; allocated here when None."""
    import torch
    B, QKVH, D = qkv.shape
    L, _, Hkv, S, _ = k_cache.shape
    assert QKVH == Hq + 2 * Hkv
    if max_t is None:
        max_t = t
    if workspace is None:
        workspace = torch.empty(decode_attn_workspace_bytes(B, Hq, Hkv, D, max_t), dtype=torch.uint8, device=qkv.device)
    rc = lib().onellm_decode_attn(_dt(qkv), _ptr(qkv), _ptr(bias), _ptr(k_cache), _ptr(v_cache), _ptr(out),
                                  B, Hq, Hkv, D, S, layer, L, int(t), _ptr(t_dev), int(max_t),
                                  rotary_dim, rope_base, rope_pos_offset, flags,
                                  _ptr(workspace), workspace.numel(), _stream())
    _check(rc, "onellm_decode_attn")
    return out


def decode_attn_static(qkv, bias, k_cache, v_cache, out, Hq, t, rotary_dim, rope_base, layer=0, t_dev=None,
                       max_t=None, rope_pos_offset=0, flags=0):
    """decode_attn through the entry point that uses the library's built-in scratch (allocates nothing)."""
    B, QKVH, D = qkv.shape
    L, _, Hkv, S, _ = k_cache.shape
    assert QKVH == Hq + 2 * Hkv
    if max_t is None:
        max_t = t
    rc = lib().onellm_decode_attn_static(_dt(qkv), _ptr(qkv), _ptr(bias), _ptr(k_cache), _ptr(v_cache), _ptr(out),
                                         B, Hq, Hkv, D, S, layer, L, int(t), _ptr(t_dev), int(max_t),
                                         rotary_dim, rope_base, rope_pos_offset, flags, _stream())
    _check(rc, "onellm_decode_attn_static")
    return out


def rmsnorm(x, gamma, eps):
    N, H = x.shape
    _check(lib().onellm_rmsnorm(_dt(x), _ptr(x), _ptr(gamma), eps, N, H, _stream()), "onellm_rmsnorm")
    return x


def fused_add_bias_residual_rmsnorm(residual, out, bias, gamma, eps):
    N, H = out.shape
    _check(lib().onellm_fused_add_bias_residual_rmsnorm(_dt(out), _ptr(residual), _ptr(out), _ptr(bias), _ptr(gamma),
                                                        eps, N, H, _stream()), "onellm_fused_add_bias_residual_rmsnorm")
    return residual, out


def kv_append(k_src, v_src, k_cache, v_cache, cur_len, history_len, layer=0):
    B, Hkv, max_q_len, D = k_src.shape
    L, _, _, S, _ = k_cache.shape
    _check(lib().onellm_kv_append(_dt(k_src), _ptr(k_src), _ptr(v_src), _ptr(k_cache), _ptr(v_cache), _ptr(cur_len),
                                  _ptr(history_len), B, Hkv, max_q_len, S, D, layer, L, _stream()), "onellm_kv_append")


def kv_repeat(k_cache, v_cache, k_dst, v_dst, context_len, layer=0):
    L, B, Hkv, S, D = k_cache.shape
    _, Hq, max_k_len, _ = k_dst.shape
    _check(lib().onellm_kv_repeat(_dt(k_cache), _ptr(k_cache), _ptr(v_cache), _ptr(k_dst), _ptr(v_dst),
                                  _ptr(context_len), B, Hq, Hkv, S, max_k_len, D, layer, L, _stream()),
           "onellm_kv_repeat")


def beam_topk_workspace_bytes(B, beam, K):
    return lib().onellm_beam_topk_workspace_bytes(B, beam, K)


def beam_topk_last_launches():
    return lib().onellm_beam_topk_last_launches()


def beam_topk_last_path():
    return lib().onellm_beam_topk_last_path()


def release_workspace(workspace):
    """Give the arrival-counter sets of a workspace (a tensor or a raw pointer) back; returns how many were freed."""
    ptr = workspace if isinstance(workspace, int) else workspace.data_ptr()
    return lib().onellm_release_workspace(ptr)


def counter_set_fallbacks():
    return lib().onellm_counter_set_fallbacks()


def beam_topk(logits, B, beam, K, workspace=None):
    """logits [B*beam, V] fp32.  Returns (workspace, round1_vals, round1_ids, final_vals, final_ids) as views."""
    import torch
    rows, V = logits.shape
    assert rows == B * beam and logits.dtype == torch.float32
    if workspace is None:
        workspace = torch.empty(beam_topk_workspace_bytes(B, beam, K) // 4, dtype=torch.float32, device=logits.device)
        # a workspace made here gives its counter set back when the tensor dies (the caller of the C function does
        # that itself, with onellm_release_workspace, when it frees a workspace)
        weakref.finalize(workspace, lib().onellm_release_workspace, workspace.data_ptr())
    _check(lib().onellm_beam_topk(_ptr(logits), B, beam, V, K, _ptr(workspace), _stream()), "onellm_beam_topk")
    n1 = B * beam * TOPK_BLOCKS_PER_ROW * K
    vals = workspace[:n1].view(B * beam, TOPK_BLOCKS_PER_ROW, K)
    ids = workspace[n1:2 * n1].view(torch.int32).view(B * beam, TOPK_BLOCKS_PER_ROW, K)
    fv = workspace[2 * n1:2 * n1 + B * K].view(B, K)
    fi = workspace[2 * n1 + B * K:2 * n1 + 2 * B * K].view(torch.int32).view(B, K)
    return workspace, vals, ids, fv, fi


def qkv_bias_rope_transpose(q_buf, k_buf, v_buf, qkv, bias, padding_offset, history_length, rotary_dim, rope_base):
    """qkv [token_num, Hq+2Hkv, D]; q_buf [B, Hq, seq_len, D]; k_buf / v_buf [B, Hkv, seq_len, D]."""
    token_num, QKVH, D = qkv.shape
    B, Hq, seq_len, _ = q_buf.shape
    Hkv = k_buf.shape[1]
    assert QKVH == Hq + 2 * Hkv
    _check(lib().onellm_qkv_bias_rope_transpose(_dt(qkv), _ptr(q_buf), _ptr(k_buf), _ptr(v_buf), _ptr(qkv), _ptr(bias),
                                                _ptr(padding_offset), _ptr(history_length), B, seq_len, token_num, Hq,
                                                Hkv, D, rotary_dim, rope_base, _stream()),
           "onellm_qkv_bias_rope_transpose")


def silu_and_mul(inp, out):
    B, two, I = inp.shape
    assert two == 2
    _check(lib().onellm_silu_and_mul(_dt(inp), _ptr(inp), _ptr(out), B, I, _stream()), "onellm_silu_and_mul")
    return out


def topk_sample(topk_id, topk_val, output_id, seqlen, is_finished, seed, end_id, vocab_size):
    """topk_id int32 [B, K]; topk_val fp32 [B, K]; output_id, seqlen int32 [B]; is_finished bool/uint8 [B]."""
    B, K = topk_id.shape
    _check(lib().onellm_topk_sample(_ptr(topk_id), _ptr(topk_val), _ptr(output_id), _ptr(seqlen), _ptr(is_finished), B, K,
                                    int(seed), end_id, vocab_size, _stream()), "onellm_topk_sample")
    return output_id


# ---------------------------------------------------------------- projection GEMMs (include/onellm_gemm.h)
GEMM_PATH = os.path.join(_HERE, "libonellm_gemm.so")
LAYERS_PATH = os.path.join(_HERE, "libonellm_layers.so")
GEMM_SYMBOLS = {
    "onellm_linear": (_ci, [_ci, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _sz, _vp]),
    "onellm_linear_tune": (_ci, [_ci, _ci, _ci, _ci, _ci, _ci, _vp, _sz, _vp, ctypes.POINTER(_cf), ctypes.POINTER(_cf)]),
    "onellm_linear_workspace_bytes": (_sz, []),
    "onellm_linear_last_path": (_ci, []),
    "onellm_linear_pair": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _sz, _vp]),
    "onellm_linear_pair_tune": (_ci, [_ci, _ci, _ci, _ci, _ci, _ci, _vp, _sz, _vp, ctypes.POINTER(_cf), ctypes.POINTER(_cf)]),
    "onellm_linear_allow_plain": (_ci, [_ci]),
}
_gemm = None


def gemm_lib():
    """Load the projection library (once); it brings in hipBLASLt, so it is separate from lib()."""
    global _gemm
    if _gemm is None:
        if not os.path.exists(GEMM_PATH):
            raise RuntimeError(f"{GEMM_PATH} is missing: build it with `python -m onellm_amd.build`")
        import torch  # noqa: F401  first: the process must end up with one HIP runtime and one BLAS library
        L = ctypes.CDLL(GEMM_PATH)
        for name, (res, args) in GEMM_SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _gemm = L
    return _gemm


def linear_workspace_bytes():
    return gemm_lib().onellm_linear_workspace_bytes()


def linear_tune(dtype_code, M, K, N, ldy=0, w_is_nk=False, workspace=None):
    """Time the library's candidates for this problem once and keep the fastest; returns (best_us, first_us)."""
    best, first = _cf(0.0), _cf(0.0)
    rc = gemm_lib().onellm_linear_tune(dtype_code, M, K, N, int(ldy), int(bool(w_is_nk)), _ptr(workspace),
                                       workspace.numel() if workspace is not None else 0, _stream(), ctypes.byref(best),
                                       ctypes.byref(first))
    _check(rc, "onellm_linear_tune")
    return best.value, first.value


def linear_pair_tune(dtype_code, M, K, N, ldy=0, w_is_nk=False, workspace=None):
    """Tune the single projection, then time the one-launch forms of a pair against two calls; returns
    (best_us, two_calls_us)."""
    best, two = _cf(0.0), _cf(0.0)
    rc = gemm_lib().onellm_linear_pair_tune(dtype_code, M, K, N, int(ldy), int(bool(w_is_nk)), _ptr(workspace),
                                            workspace.numel() if workspace is not None else 0, _stream(), ctypes.byref(best),
                                            ctypes.byref(two))
    _check(rc, "onellm_linear_pair_tune")
    return best.value, two.value


def linear_pair(x, w_first, w_second, y_first, y_second, w_is_nk=False, ldy=0, workspace=None):
    """y_first = x . w_first and y_second = x . w_second (same shapes, row stride ldy): the gate / up pair."""
    M, K = x.shape
    N = w_first.shape[0] if w_is_nk else w_first.shape[1]
    assert w_first.shape == w_second.shape and (w_first.shape[1] if w_is_nk else w_first.shape[0]) == K
    assert x.dtype == w_first.dtype == w_second.dtype == y_first.dtype == y_second.dtype
    assert x.is_cuda and x.is_contiguous() and w_first.is_contiguous() and w_second.is_contiguous()
    rc = gemm_lib().onellm_linear_pair(_dt(x), x.data_ptr(), w_first.data_ptr(), w_second.data_ptr(), y_first.data_ptr(),
                                       y_second.data_ptr(), M, K, N, int(ldy), int(bool(w_is_nk)), _ptr(workspace),
                                       workspace.numel() if workspace is not None else 0, _stream())
    _check(rc, "onellm_linear_pair")


def linear(x, w, y, w_is_nk=False, ldy=0, workspace=None):
    """y[M, N] = x[M, K] . W (W [K, N], or [N, K] with w_is_nk); y may be a strided view given by its first element
    and `ldy`.  `workspace`: uint8 device tensor or None."""
    M, K = x.shape
    N = w.shape[0] if w_is_nk else w.shape[1]
    assert (w.shape[1] if w_is_nk else w.shape[0]) == K and x.dtype == w.dtype == y.dtype
    assert x.is_cuda and x.is_contiguous() and w.is_contiguous()
    rc = gemm_lib().onellm_linear(_dt(x), x.data_ptr(), w.data_ptr(), y.data_ptr(), M, K, N, int(ldy), int(bool(w_is_nk)),
                                  _ptr(workspace), workspace.numel() if workspace is not None else 0, _stream())
    _check(rc, "onellm_linear")
    return y


# ---------------------------------------------------------------- decode-side layers (include/onellm_layers.h)
_layers = None


def layers_lib():
    global _layers
    if _layers is None:
        if not os.path.exists(LAYERS_PATH):
            raise RuntimeError(f"{LAYERS_PATH} is missing: build it with `python -m onellm_amd.build`")
        gemm_lib()
        L = ctypes.CDLL(LAYERS_PATH)
        pp = ctypes.POINTER(ctypes.c_void_p)
        L.onellm_layers_last_error.restype = ctypes.c_char_p
        L.onellm_layers_linear.argtypes = [_ci, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci]
        L.onellm_decoder_create.restype = _vp
        L.onellm_decoder_create.argtypes = [_ci] * 9 + [_cf, _cf, _ci] + [pp] * 10 + [_vp, _vp]
        L.onellm_decoder_forward.argtypes = [_vp, _ci, _vp, _vp, _vp, _vp]
        L.onellm_decoder_destroy.argtypes = [_vp]
        _layers = L
    return _layers


class SelfDecoder:
    """LlamaSelfDecoder over device tensors.  `layers`: list of dicts of torch device tensors with the keys attn_norm,
    ffn_norm, wqkv, bqkv, wo, bo, wdown, bdown, wgate, wup (weights [in, out]; a bias may be None).  `stream`: raw
    stream handle every step is queued on (None = the null stream)."""

    ORDER = ["attn_norm", "ffn_norm", "wqkv", "bqkv", "wo", "bo", "wdown", "bdown", "wgate", "wup"]

    def __init__(self, dtype_code, B, Hq, Hkv, D, inter_size, S, rotary_dim, rope_base, eps, layers, output_norm, attn_bias=True,
                 stream=None):
        self.L = layers_lib()
        self._keep = (layers, output_norm)
        n = len(layers)
        arrays = []
        for name in self.ORDER:
            arr = (ctypes.c_void_p * n)()
            for l, w in enumerate(layers):
                arr[l] = None if w[name] is None else _ptr(w[name])
            arrays.append(arr)
        self.handle = self.L.onellm_decoder_create(dtype_code, B, Hq, Hkv, D, inter_size, n, S, rotary_dim, rope_base, eps,
                                                   int(attn_bias), *arrays, _ptr(output_norm), stream)
        if not self.handle:
            raise RuntimeError(self.L.onellm_layers_last_error().decode())

    def forward(self, step, decoder_input, decoder_output, k_cache, v_cache):
        rc = self.L.onellm_decoder_forward(self.handle, int(step), _ptr(decoder_input), _ptr(decoder_output), _ptr(k_cache),
                                           _ptr(v_cache))
        if rc != 0:
            raise RuntimeError(self.L.onellm_layers_last_error().decode())

    def close(self):
        if self.handle:
            self.L.onellm_decoder_destroy(self.handle)
            self.handle = None
