"""ctypes binding of the CPU oracle (oracle/libonellm_ref.so).  TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg import this module;
the product package never does.  Every function works on numpy arrays in place, exactly as the
C functions do, and raises on a non-zero return code.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ONELLM_REF_LIB selects another build of the same source, e.g. oracle/libonellm_ref_asan.so (`make -C oracle
# check-asan` runs the oracle's tests against it under AddressSanitizer + UBSan)
_LIB_PATH = os.environ.get("ONELLM_REF_LIB") or os.path.join(_HERE, "libonellm_ref.so")

FP32, FP16 = 0, 1
ATTN_NO_V_BIAS = 0x1
ATTN_NO_CACHE_WRITE = 0x2


def build(force=False):
    """Compile the oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(
            os.path.join(_HERE, "onellm_ref.c")):
        subprocess.run(["make", "-C", _HERE, "-B", os.path.basename(_LIB_PATH)], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, ci, cf, cu = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_uint
        L.onellm_ref_sincosf.argtypes = [cf, ctypes.POINTER(cf), ctypes.POINTER(cf)]
        L.onellm_ref_sincosf.restype = None
        L.onellm_ref_rope_freqs.argtypes = [vp, ci, ci, cf]
        L.onellm_ref_rope_freqs.restype = None
        L.onellm_ref_rope_row.argtypes = [vp, ci, ci, vp, ci]
        L.onellm_ref_rope_row.restype = None
        L.onellm_ref_decode_attn.argtypes = [ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp, ci, cf, ci, cu]
        L.onellm_ref_rmsnorm.argtypes = [ci, vp, vp, cf, ci, ci]
        L.onellm_ref_fused_add_bias_residual_rmsnorm.argtypes = [ci, vp, vp, vp, vp, cf, ci, ci, ci]
        L.onellm_ref_kv_append.argtypes = [ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci]
        L.onellm_ref_kv_repeat.argtypes = [ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci]
        L.onellm_ref_beam_topk.argtypes = [vp, ci, ci, ci, ci, ci, vp]
        L.onellm_ref_qkv_bias_rope_transpose.argtypes = [ci, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, cf]
        L.onellm_ref_silu_and_mul.argtypes = [ci, vp, vp, ci, ci]
        L.onellm_ref_philox4x32_10.argtypes = [vp, vp, vp]
        L.onellm_ref_philox4x32_10.restype = None
        L.onellm_ref_uniform_from_u32.argtypes = [ctypes.c_uint32]
        L.onellm_ref_uniform_from_u32.restype = cf
        L.onellm_ref_exp_fixed.argtypes = [cf]
        L.onellm_ref_exp_fixed.restype = cf
        L.onellm_ref_topk_sample.argtypes = [vp, vp, vp, vp, vp, ci, ci, ctypes.c_ulonglong, ci, ci]
        _lib = L
    return _lib


def _dt(a):
    if a.dtype == np.float32:
        return FP32
    if a.dtype == np.float16:
        return FP16
    raise TypeError(f"unsupported dtype {a.dtype}")


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle needs C-contiguous arrays"
    return a.ctypes.data


def _chk(rc, name):
    if rc != 0:
        raise RuntimeError(f"oracle {name} rejected its arguments (rc={rc})")


def sincosf(x):
    s, c = ctypes.c_float(), ctypes.c_float()
    lib().onellm_ref_sincosf(ctypes.c_float(x), ctypes.byref(s), ctypes.byref(c))
    return s.value, c.value


def sincosf_array(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    s = np.empty_like(x)
    c = np.empty_like(x)
    L = lib()
    cs, cc = ctypes.c_float(), ctypes.c_float()
    for i, v in enumerate(x.ravel()):
        L.onellm_ref_sincosf(ctypes.c_float(float(v)), ctypes.byref(cs), ctypes.byref(cc))
        s.ravel()[i] = cs.value
        c.ravel()[i] = cc.value
    return s, c


def rope_freqs(rotary_dim, base, D=None):
    D = rotary_dim if D is None else D
    f = np.zeros(D // 2 + 1, dtype=np.float32)
    lib().onellm_ref_rope_freqs(_p(f), D, rotary_dim, base)
    return f[: min(rotary_dim, D) // 2]


def rope_row(x, rotary_dim, base, pos):
    """Rotate one fp32 row in place."""
    assert x.dtype == np.float32 and x.ndim == 1
    f = np.zeros(x.shape[0] // 2 + 1, dtype=np.float32)
    lib().onellm_ref_rope_freqs(_p(f), x.shape[0], rotary_dim, base)
    lib().onellm_ref_rope_row(_p(x), x.shape[0], rotary_dim, _p(f), pos)
    return x


def decode_attn(qkv, bias, k_cache, v_cache, Hq, t, rotary_dim, rope_base, layer=0,
                rope_pos_offset=0, flags=0):
    """qkv [B, Hq+2Hkv, D]; caches [L, B, Hkv, S, D] (modified in place); t int or int array [B].
    Returns out [B, Hq*D]."""
    B, QKVH, D = qkv.shape
    L, Bc, Hkv, S, Dc = k_cache.shape
    assert Bc == B and Dc == D and QKVH == Hq + 2 * Hkv and v_cache.shape == k_cache.shape
    assert k_cache.dtype == qkv.dtype == v_cache.dtype
    out = np.zeros((B, Hq * D), dtype=qkv.dtype)
    if np.isscalar(t) or isinstance(t, (int, np.integer)):
        t_host, t_arr = int(t), None
    else:
        t_arr = np.ascontiguousarray(t, dtype=np.int32)
        t_host = int(t_arr.max())
    rc = lib().onellm_ref_decode_attn(_dt(qkv), _p(qkv), _p(bias), _p(k_cache), _p(v_cache), _p(out),
                                      B, Hq, Hkv, D, S, layer, L, t_host, _p(t_arr),
                                      rotary_dim, rope_base, rope_pos_offset, flags)
    _chk(rc, "decode_attn")
    return out


def rmsnorm(x, gamma, eps):
    N, H = x.shape
    assert gamma.dtype == x.dtype
    _chk(lib().onellm_ref_rmsnorm(_dt(x), _p(x), _p(gamma), eps, N, H), "rmsnorm")
    return x


def fused_add_bias_residual_rmsnorm(residual, out, bias, gamma, eps, as_written=False):
    N, H = out.shape
    assert residual.shape == out.shape and residual.dtype == out.dtype == gamma.dtype
    _chk(lib().onellm_ref_fused_add_bias_residual_rmsnorm(_dt(out), _p(residual), _p(out), _p(bias), _p(gamma),
                                                          eps, N, H, int(as_written)), "fused_norm")
    return residual, out


def kv_append(k_src, v_src, k_cache, v_cache, cur_len, history_len, layer=0):
    B, Hkv, max_q_len, D = k_src.shape
    L, _, _, S, _ = k_cache.shape
    cur_len = np.ascontiguousarray(cur_len, dtype=np.int32)
    history_len = np.ascontiguousarray(history_len, dtype=np.int32)
    _chk(lib().onellm_ref_kv_append(_dt(k_src), _p(k_src), _p(v_src), _p(k_cache), _p(v_cache), _p(cur_len),
                                    _p(history_len), B, Hkv, max_q_len, S, D, layer, L), "kv_append")


def kv_repeat(k_cache, v_cache, k_dst, v_dst, context_len, layer=0):
    L, B, Hkv, S, D = k_cache.shape
    _, Hq, max_k_len, _ = k_dst.shape
    context_len = np.ascontiguousarray(context_len, dtype=np.int32)
    _chk(lib().onellm_ref_kv_repeat(_dt(k_cache), _p(k_cache), _p(v_cache), _p(k_dst), _p(v_dst), _p(context_len),
                                    B, Hq, Hkv, S, max_k_len, D, layer, L), "kv_repeat")


def beam_topk(logits, B, beam, K, nblk=8):
    """Returns (round1_vals [B*beam,nblk,K], round1_ids, final_vals [B,K], final_ids [B,K])."""
    rows, V = logits.shape
    assert rows == B * beam and logits.dtype == np.float32
    n1 = B * beam * nblk * K
    ws = np.zeros(2 * n1 + 2 * B * K, dtype=np.float32)
    _chk(lib().onellm_ref_beam_topk(_p(logits), B, beam, V, K, nblk, _p(ws)), "beam_topk")
    vals = ws[:n1].reshape(B * beam, nblk, K).copy()
    ids = ws[n1:2 * n1].view(np.int32).reshape(B * beam, nblk, K).copy()
    fv = ws[2 * n1:2 * n1 + B * K].reshape(B, K).copy()
    fi = ws[2 * n1 + B * K:].view(np.int32).reshape(B, K).copy()
    return vals, ids, fv, fi


def qkv_bias_rope_transpose(q_buf, k_buf, v_buf, qkv, bias, padding_offset, history_length, rotary_dim, rope_base):
    """qkv [token_num, Hq+2Hkv, D]; q_buf [B, Hq, seq_len, D]; k_buf/v_buf [B, Hkv, seq_len, D] (written in place)."""
    token_num, QKVH, D = qkv.shape
    B, Hq, seq_len, _ = q_buf.shape
    Hkv = k_buf.shape[1]
    assert QKVH == Hq + 2 * Hkv
    po = np.ascontiguousarray(padding_offset, dtype=np.int32)
    hl = np.ascontiguousarray(history_length, dtype=np.int32)
    _chk(lib().onellm_ref_qkv_bias_rope_transpose(_dt(qkv), _p(q_buf), _p(k_buf), _p(v_buf), _p(qkv), _p(bias), _p(po),
                                                  _p(hl), B, seq_len, token_num, Hq, Hkv, D, rotary_dim, rope_base),
         "qkv_bias_rope_transpose")


def silu_and_mul(inp, out):
    B, two, I = inp.shape
    assert two == 2 and out.shape == (B, I) and out.dtype == inp.dtype
    _chk(lib().onellm_ref_silu_and_mul(_dt(inp), _p(inp), _p(out), B, I), "silu_and_mul")
    return out


def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32).copy()
    k = np.asarray(key, dtype=np.uint32).copy()
    out = np.zeros(4, np.uint32)
    lib().onellm_ref_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def uniform_from_u32(x):
    return lib().onellm_ref_uniform_from_u32(int(x))


def exp_fixed(x):
    return lib().onellm_ref_exp_fixed(float(x))


def topk_sample(topk_id, topk_val, seqlen, is_finished, seed, end_id, vocab_size):
    """topk_id int32 [B, K], topk_val fp32 [B, K] sorted best-first; seqlen int32 [B] and is_finished uint8 [B]
    are updated in place.  Returns output_id int32 [B]."""
    B, K = topk_id.shape
    assert topk_id.dtype == np.int32 and topk_val.dtype == np.float32 and seqlen.dtype == np.int32
    assert is_finished.dtype == np.uint8
    out = np.zeros(B, np.int32)
    _chk(lib().onellm_ref_topk_sample(_p(topk_id), _p(topk_val), _p(out), _p(seqlen), _p(is_finished), B, K,
                                      int(seed), end_id, vocab_size), "topk_sample")
    return out


def linear(x, w, w_is_nk=False):
    """y[M, N] = x[M, K] . W with W [K, N] (or [N, K] when w_is_nk), accumulated in float64 and rounded once to
    x.dtype — the projection of src/kernels/qkv_linear.cu:8-66 with the weight layout of
    src/weights/llama/layer_weights.cc:21-41 (shape = {in, out}).  Pinned by the all-ones case of
    tests/unittests/test_linear.cu:60-98 and by brute-force triple loops."""
    assert x.dtype == w.dtype and x.ndim == 2 and w.ndim == 2
    wm = w.astype(np.float64)
    y = x.astype(np.float64) @ (wm.T if w_is_nk else wm)
    return y.astype(x.dtype)


def self_decoder_step(x, layers, output_norm, k_cache, v_cache, Hq, t, rotary_dim, rope_base, eps, rope_pos_offset=-1):
    """One decode step of the LLaMA decoder stack (src/layers/decoder/self_decoder.cpp:15-78 with
    src/layers/attention/masked_self_attention.cpp:51-82 and src/layers/ffn/ffn.cpp:53-73), built from the
    per-kernel restatements above plus linear().  The data flow is the pre-norm decoder the reference is written
    towards (x stays the residual stream; the snapshot normalises it in place, drops the FFN result and addresses
    cache layer 0 for every layer).  The new token is rotated as position t + rope_pos_offset: -1 is the 0-based
    position the context phase gives that row (src/kernels/qkv_bias_and_RoPE.cu:140), 0 what the decode kernel does
    on its own (src/kernels/decoder_masked_attn.cu:186).

    x [B, hidden] (updated in place: the residual stream); layers: list of dicts with attn_norm, ffn_norm, wqkv
    [hidden, (Hq+2Hkv)D], bqkv, wo [hidden, hidden], bo, wgate/wup [hidden, I], wdown [I, hidden], bdown (biases
    may be None); caches [L, B, Hkv, S, D] (row t-1 of every layer written).  Returns y [B, hidden]."""
    B, hidden = x.shape
    L, _, Hkv, S, D = k_cache.shape
    assert len(layers) == L and hidden == Hq * D
    zeros = np.zeros(hidden, dtype=x.dtype)
    y = rmsnorm(x.copy(), layers[0]["attn_norm"], eps)
    for l, w in enumerate(layers):
        qkv = linear(y, w["wqkv"]).reshape(B, Hq + 2 * Hkv, D)
        a = decode_attn(qkv, w["bqkv"], k_cache, v_cache, Hq, t, rotary_dim, rope_base, layer=l,
                        rope_pos_offset=rope_pos_offset)
        y = linear(a, w["wo"])
        fused_add_bias_residual_rmsnorm(x, y, w["bo"] if w["bo"] is not None else zeros, w["ffn_norm"], eps)
        gate, up = linear(y, w["wgate"]), linear(y, w["wup"])
        pair = np.ascontiguousarray(np.stack([gate, up], axis=1))           # [B, 2, I]
        act = silu_and_mul(pair, np.empty_like(gate))
        y = linear(act, w["wdown"])
        gamma = layers[l + 1]["attn_norm"] if l + 1 < L else output_norm
        fused_add_bias_residual_rmsnorm(x, y, w["bdown"] if w["bdown"] is not None else zeros, gamma, eps)
    return y


def set_threads(n):
    """Host threads the oracle's OpenMP loops may use; returns the previous setting."""
    return lib().onellm_ref_set_threads(int(n))
