#!/usr/bin/env python3
"""Writes the golden vectors in this directory (small .npz files: inputs and expected outputs).

    python tests/golden/make_fixtures.py

The expected outputs come from float64 numpy models written here from the mathematics of each operation
(softmax(q K^T / sqrt(D)) V with rotary embedding as a complex multiplication, root-mean-square
normalisation, slice assignment, np.repeat, np.lexsort, x * sigmoid(x) * y), not from the CPU oracle under
oracle/ and not from the HIP kernels: they pin both.  Shapes include BASELINE config 1 (fp32, batch 1,
8 heads x 64, 16 cached steps + the current token, seed 0) exactly.  Nothing here reads the reference.

The files are data only (numpy arrays, loaded with allow_pickle=False).
"""
import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def rope64(x, rotary_dim, base, pos):
    """(x[2i] + i x[2i+1]) * exp(i * pos / base**(2i/rotary_dim)) for 2i < rotary_dim."""
    x = np.asarray(x, dtype=np.float64).copy()
    n = min(rotary_dim, x.shape[-1]) // 2
    if n:
        z = (x[..., 0:2 * n:2] + 1j * x[..., 1:2 * n:2]) * np.exp(1j * pos * np.power(float(base), -np.arange(n) * 2.0 / rotary_dim))
        x[..., 0:2 * n:2], x[..., 1:2 * n:2] = z.real, z.imag
    return x


def attention_case(dtype, B, Hq, Hkv, D, S, t, rotary_dim, base, seed, std, pos_offset=0):
    rng = np.random.default_rng(seed)
    qkv = (rng.standard_normal((B, Hq + 2 * Hkv, D)) * std).astype(dtype)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * std).astype(dtype)
    kc = (rng.standard_normal((1, B, Hkv, S, D)) * std).astype(dtype)
    vc = (rng.standard_normal((1, B, Hkv, S, D)) * std).astype(dtype)
    t = np.broadcast_to(np.asarray(t, np.int32), (B,)).copy()
    G = Hq // Hkv
    b64 = bias.astype(np.float64).reshape(Hq + 2 * Hkv, D)
    out = np.zeros((B, Hq * D))
    new_k = np.zeros((B, Hkv, D))
    new_v = np.zeros((B, Hkv, D))
    for b in range(B):
        x = qkv[b].astype(np.float64) + b64
        pos = int(t[b]) + pos_offset
        q = rope64(x[:Hq], rotary_dim, base, pos)
        k = rope64(x[Hq:Hq + Hkv], rotary_dim, base, pos).astype(dtype).astype(np.float64)   # stored, then used
        v = x[Hq + Hkv:].astype(dtype).astype(np.float64)
        new_k[b], new_v[b] = k, v
        for h in range(Hq):
            kvh = h // G
            K = np.concatenate([kc[0, b, kvh, :t[b] - 1].astype(np.float64), k[kvh][None]])
            V = np.concatenate([vc[0, b, kvh, :t[b] - 1].astype(np.float64), v[kvh][None]])
            s = K @ q[h] / math.sqrt(D)
            p = np.exp(s - s.max())
            out[b, h * D:(h + 1) * D] = (p / p.sum()) @ V
    return dict(qkv=qkv, bias=bias, k_cache=kc, v_cache=vc, t=t, Hq=np.int32(Hq), rotary_dim=np.int32(rotary_dim),
                base=np.float64(base), pos_offset=np.int32(pos_offset), out=out, new_k=new_k, new_v=new_v)


def norm_case(dtype, N, H, eps, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, H)).astype(dtype)
    res = rng.standard_normal((N, H)).astype(dtype)
    bias = rng.standard_normal(H).astype(dtype)
    gamma = rng.uniform(0.5, 1.5, H).astype(dtype)
    x64, g64 = x.astype(np.float64), gamma.astype(np.float64)
    y = g64 * x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + eps)
    r = x64 + res.astype(np.float64) + bias.astype(np.float64)
    fy = g64 * r / np.sqrt((r ** 2).mean(-1, keepdims=True) + eps)
    return dict(x=x, residual=res, bias=bias, gamma=gamma, eps=np.float64(eps), rmsnorm=y, fused_residual=r, fused_out=fy)


def kv_case(seed):
    rng = np.random.default_rng(seed)
    B, Hkv, G, S, D, L, max_q = 3, 2, 3, 24, 16, 2, 5
    kc = rng.integers(-2000, 2000, (L, B, Hkv, S, D)).astype(np.float16)
    vc = rng.integers(-2000, 2000, (L, B, Hkv, S, D)).astype(np.float16)
    ks = rng.integers(-2000, 2000, (B, Hkv, max_q, D)).astype(np.float16)
    vs = rng.integers(-2000, 2000, (B, Hkv, max_q, D)).astype(np.float16)
    cur = np.array([5, 1, 0], np.int32)
    hist = np.array([3, 19, 7], np.int32)
    layer = 1
    ka, va = kc.copy(), vc.copy()
    for b in range(B):
        ka[layer, b, :, hist[b]:hist[b] + cur[b]] = ks[b, :, :cur[b]]
        va[layer, b, :, hist[b]:hist[b] + cur[b]] = vs[b, :, :cur[b]]
    ctx = (hist + cur).astype(np.int32)
    max_k = 22
    kr = np.full((B, Hkv * G, max_k, D), 7.0, np.float16)        # rows past the length keep this sentinel
    vr = np.full((B, Hkv * G, max_k, D), 7.0, np.float16)
    for b in range(B):
        n = min(ctx[b], max_k)
        kr[b, :, :n] = np.repeat(ka[layer, b, :, :n], G, axis=0)
        vr[b, :, :n] = np.repeat(va[layer, b, :, :n], G, axis=0)
    return dict(k_cache=kc, v_cache=vc, k_src=ks, v_src=vs, cur_len=cur, history_len=hist, layer=np.int32(layer),
                k_after_append=ka, v_after_append=va, context_len=ctx, G=np.int32(G), k_repeated=kr, v_repeated=vr)


def topk_case(seed):
    rng = np.random.default_rng(seed)
    B, beam, V, K = 3, 4, 2000, 4
    logits = (rng.standard_normal((B * beam, V)) * 2).astype(np.float32)
    for r in range(B * beam):                                     # planted equal maxima: the lower index must win
        logits[r, [17, V // 2, V - 1]] = logits[r].max() + 1.0
    logits[0:beam] = logits[0]                                    # a whole batch entry of identical rows
    logits[beam, 5] = logits[beam + 3, 5] = 100.0                 # the same value in two beams of one entry
    flat = np.arange(B * beam * V, dtype=np.int64).reshape(B * beam, V)
    row_ids = np.zeros((B * beam, K), np.int32)
    for r in range(B * beam):
        order = np.lexsort((flat[r], -logits[r].astype(np.float64)))
        row_ids[r] = flat[r][order[:K]]
    fin_ids = np.zeros((B, K), np.int32)
    fin_vals = np.zeros((B, K), np.float32)
    lf = logits.reshape(-1)
    for b in range(B):
        idx = flat[b * beam:(b + 1) * beam].reshape(-1)
        order = np.lexsort((idx, -lf[idx].astype(np.float64)))
        fin_ids[b] = idx[order[:K]]
        fin_vals[b] = lf[fin_ids[b]]
    return dict(logits=logits, B=np.int32(B), beam=np.int32(beam), K=np.int32(K), row_ids=row_ids, final_ids=fin_ids,
                final_vals=fin_vals)


def prefill_case(dtype, seed):
    rng = np.random.default_rng(seed)
    B, S, Hq, Hkv, D, rd, base = 3, 12, 4, 2, 16, 12, 10000.0
    lens = [12, 5, 1]
    hist = np.array([0, 40, 3000], np.int32)
    T = sum(lens)
    qkv = (rng.standard_normal((T, Hq + 2 * Hkv, D)) * 0.5).astype(dtype)
    bias = (rng.standard_normal((Hq + 2 * Hkv) * D) * 0.5).astype(dtype)
    po, tok = [], 0
    for b, n in enumerate(lens):
        for s in range(n):
            po.append(b * S + s - tok)
            tok += 1
    po = np.array(po, np.int32)
    q = np.zeros((B, Hq, S, D))
    k = np.zeros((B, Hkv, S, D))
    v = np.zeros((B, Hkv, S, D))
    written = np.zeros((B, S), bool)
    b64 = bias.astype(np.float64).reshape(Hq + 2 * Hkv, D)
    for tkn in range(T):
        dst = tkn + po[tkn]
        b, s = dst // S, dst % S
        x = qkv[tkn].astype(np.float64) + b64
        pos = int(hist[b]) + s
        q[b, :, s] = rope64(x[:Hq], rd, base, pos)
        k[b, :, s] = rope64(x[Hq:Hq + Hkv], rd, base, pos)
        v[b, :, s] = x[Hq + Hkv:]
        written[b, s] = True
    return dict(qkv=qkv, bias=bias, padding_offset=po, history_len=hist, rotary_dim=np.int32(rd), base=np.float64(base),
                B=np.int32(B), S=np.int32(S), Hq=np.int32(Hq), q=q, k=k, v=v, written=written)


def swiglu_case(dtype, seed):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((5, 2, 24)) * 2).astype(dtype)
    g, u = x[:, 0].astype(np.float64), x[:, 1].astype(np.float64)
    return dict(inp=x, out=g / (1.0 + np.exp(-g)) * u)


def main():
    save = lambda name, d: np.savez_compressed(os.path.join(HERE, name + ".npz"), **d)
    # BASELINE config 1: fp32, batch 1, 8 heads x 64, cache of 16 steps + the current token, rotary 64, seed 0
    save("attn_config1_fp32", attention_case(np.float32, 1, 8, 8, 64, 32, 17, 64, 10000.0, seed=0, std=1.0))
    # grouped-query fp16 with per-sequence lengths (7 query heads per kv head: a padded head tile), 0-based rotary position
    save("attn_gqa_fp16_ragged", attention_case(np.float16, 4, 14, 2, 128, 136, [1, 2, 77, 136], 128, 10000.0, seed=1, std=0.5,
                                                pos_offset=-1))
    # partial rotation, another base, head size 256, equal lengths
    save("attn_d256_fp16", attention_case(np.float16, 2, 6, 3, 256, 72, 70, 64, 500000.0, seed=2, std=0.5))
    save("norms_fp16", norm_case(np.float16, 6, 256, 1e-5, seed=4))
    save("norms_fp32", norm_case(np.float32, 3, 100, 1e-6, seed=5))
    save("kv_append_repeat", kv_case(seed=6))
    save("beam_topk_ties", topk_case(seed=7))
    save("prefill_rope_fp32", prefill_case(np.float32, seed=8))
    save("prefill_rope_fp16", prefill_case(np.float16, seed=9))
    save("swiglu_fp32", swiglu_case(np.float32, seed=10))
    save("swiglu_fp16", swiglu_case(np.float16, seed=11))


if __name__ == "__main__":
    main()
