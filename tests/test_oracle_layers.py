"""Pins the oracle's projection and its whole decode step (oracle/ref.py: linear, self_decoder_step) on the CPU.

* linear: the all-ones case the reference tests (tests/unittests/test_linear.cu:60-98: 16x16 ones times ones = 16)
  and a brute-force triple loop.
* self_decoder_step: against an independent library implementation of the same architecture — the Hugging Face
  LlamaModel (random weights, fp32, CPU).  The library rotates the pairs (i, i + D/2) of a head, the reference the
  pairs (2i, 2i+1) (src/kernels/decoder_masked_attn.cu:111-131); a fixed permutation of the q/k output columns maps
  one onto the other without changing any dot product, so the decoder outputs must agree and the cached K rows must
  agree up to that permutation.  This checks the step's data flow, the [in, out] weight layout, the GQA head
  mapping, the RoPE convention and position (t - 1), and the fused-norm chaining in one go.
"""
import numpy as np
import pytest


def test_linear_reference_known_answer(ref):
    x = np.ones((1, 16), np.float32)
    w = np.ones((16, 16), np.float32)
    np.testing.assert_array_equal(ref.linear(x, w), np.full((1, 16), 16.0, np.float32))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_linear_brute_force(ref, dtype):
    rng = np.random.default_rng(0)
    M, K, N = 3, 7, 5
    x = rng.standard_normal((M, K)).astype(dtype)
    w = rng.standard_normal((K, N)).astype(dtype)
    want = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            for k in range(K):
                want[m, n] += float(x[m, k]) * float(w[k, n])
    np.testing.assert_array_equal(ref.linear(x, w), want.astype(dtype))
    np.testing.assert_array_equal(ref.linear(x, np.ascontiguousarray(w.T), w_is_nk=True), want.astype(dtype))


def _interleave(D):
    """ours[2i] = theirs[i], ours[2i+1] = theirs[i + D/2]"""
    perm = np.empty(D, np.int64)
    perm[0::2] = np.arange(D // 2)
    perm[1::2] = np.arange(D // 2) + D // 2
    return perm


@pytest.mark.parametrize("Hq,Hkv,D,I,L,T", [(4, 2, 8, 12, 2, 5), (6, 2, 16, 40, 3, 9), (4, 4, 8, 16, 1, 1)])
def test_decoder_step_against_library_llama(ref, Hq, Hkv, D, I, L, T):
    torch = pytest.importorskip("torch")
    transformers = pytest.importorskip("transformers")
    torch.manual_seed(Hq * 100 + T)
    hidden, B, S, eps = Hq * D, 2, 16, 1e-5
    cfg = transformers.LlamaConfig(hidden_size=hidden, intermediate_size=I, num_hidden_layers=L, num_attention_heads=Hq,
                                   num_key_value_heads=Hkv, head_dim=D, vocab_size=8, rms_norm_eps=eps, attention_bias=True,
                                   mlp_bias=False, max_position_embeddings=64, rope_theta=10000.0,
                                   attn_implementation="eager")
    model = transformers.LlamaModel(cfg).eval().float()
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn_like(p) * (0.3 if p.ndim == 2 else 1.0))
        for name, p in model.named_parameters():
            if name.endswith("layernorm.weight") or name == "norm.weight":
                p.copy_(torch.rand_like(p) + 0.5)
        embeds = torch.randn(B, T, hidden)
        full = model(inputs_embeds=embeds, use_cache=True)
        want = full.last_hidden_state[:, T - 1].numpy()
        full_k = [full.past_key_values.layers[l].keys.numpy() for l in range(L)]       # [B, Hkv, T, D], rotated
        full_v = [full.past_key_values.layers[l].values.numpy() for l in range(L)]

    perm = _interleave(D)
    sd = {k: v.detach().numpy() for k, v in model.state_dict().items()}

    def heads_perm(wT, nheads):          # wT [hidden, nheads*D] or bias [nheads*D]: permute inside every head
        shp = wT.shape
        return np.ascontiguousarray(wT.reshape(shp[:-1] + (nheads, D))[..., perm].reshape(shp))

    layers = []
    for l in range(L):
        pre = "layers.%d." % l
        wq, wk, wv = (sd[pre + "self_attn.%s_proj.weight" % n].T for n in "qkv")
        bq, bk, bv = (sd[pre + "self_attn.%s_proj.bias" % n] for n in "qkv")
        layers.append({
            "attn_norm": sd[pre + "input_layernorm.weight"], "ffn_norm": sd[pre + "post_attention_layernorm.weight"],
            "wqkv": np.ascontiguousarray(np.concatenate([heads_perm(wq, Hq), heads_perm(wk, Hkv), wv], axis=1)),
            "bqkv": np.ascontiguousarray(np.concatenate([heads_perm(bq, Hq), heads_perm(bk, Hkv), bv])),
            "wo": np.ascontiguousarray(sd[pre + "self_attn.o_proj.weight"].T), "bo": sd[pre + "self_attn.o_proj.bias"],
            "wgate": np.ascontiguousarray(sd[pre + "mlp.gate_proj.weight"].T),
            "wup": np.ascontiguousarray(sd[pre + "mlp.up_proj.weight"].T),
            "wdown": np.ascontiguousarray(sd[pre + "mlp.down_proj.weight"].T), "bdown": None,
        })
    kc = np.zeros((L, B, Hkv, S, D), np.float32)
    vc = np.zeros((L, B, Hkv, S, D), np.float32)
    for l in range(L):
        kc[l, :, :, :T - 1] = full_k[l][:, :, :T - 1][..., perm]
        vc[l, :, :, :T - 1] = full_v[l][:, :, :T - 1]
    x = np.ascontiguousarray(embeds[:, T - 1].numpy())
    got = ref.self_decoder_step(x, layers, sd["norm.weight"], kc, vc, Hq, T, D, 10000.0, eps)

    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-5)
    for l in range(L):                   # the step appended this token's rotated K and plain V to every layer
        np.testing.assert_allclose(kc[l, :, :, T - 1], full_k[l][:, :, T - 1][..., perm], rtol=2e-4, atol=2e-5)
        np.testing.assert_allclose(vc[l, :, :, T - 1], full_v[l][:, :, T - 1], rtol=2e-4, atol=2e-5)
    assert not kc[:, :, :, T:].any() and not vc[:, :, :, T:].any()
