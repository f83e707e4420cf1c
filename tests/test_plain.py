"""Pins of the plain implementation (CPU): special cases that reduce to a library routine and
invariants, each chosen so that a plausible misreading of the reference fails it.

The reference's own vectors for this architecture (tests/golden/lfm25_dense.json,
tests/ref_lfm25_dense_128.txt) need its quantised checkpoint and tokenizer and cannot be used
here: parity with those is unpinned; what pins the formulas is below.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import util
from plain import lfm2_plain as plain
from plain.sampler_plain import PlainSampler, XorShift128Plus

torch.manual_seed(0)


def r(*shape):
    return torch.randn(*shape, dtype=torch.float64)


# ------------------------------------------------------------------------------ norm
def test_rms_norm():
    x, w = r(5, 48), r(48)
    ref = x / np.sqrt((x.numpy() ** 2).mean(-1, keepdims=True) + 1e-5) * w
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), ref)
    # scale invariance for x >> sqrt(eps); a constant row with unit weight gives +-1
    assert torch.allclose(plain.rms_norm(1000 * x, w, 1e-5), plain.rms_norm(x, w, 1e-5), atol=1e-9)
    ones = plain.rms_norm(torch.full((1, 7), -3.0, dtype=torch.float64), torch.ones(7, dtype=torch.float64), 0.0)
    assert torch.allclose(ones, -torch.ones(1, 7, dtype=torch.float64))
    # eps is added to the mean inside the root, not to the root: a zero row stays zero, finite
    z = plain.rms_norm(torch.zeros(1, 4, dtype=torch.float64), torch.ones(4, dtype=torch.float64), 1e-6)
    assert torch.equal(z, torch.zeros(1, 4, dtype=torch.float64))
    big_eps = plain.rms_norm(torch.ones(1, 4, dtype=torch.float64), torch.ones(4, dtype=torch.float64), 3.0)
    assert torch.allclose(big_eps, torch.full((1, 4), 0.5, dtype=torch.float64))         # 1/sqrt(1+3), not 1/(1+3)
    # mean, not sum, over the last axis only
    assert not torch.allclose(plain.rms_norm(x, w, 1e-5), x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-5) * w)


# ------------------------------------------------------------------------------ rope
def test_rope_properties():
    T, H, hd, base = 9, 3, 16, 10000.0
    x = r(T, H, hd)
    pos = torch.arange(T)
    y = plain.rope_neox(x, pos, base)
    assert torch.allclose(y[0], x[0])                                               # position 0: identity
    half = hd // 2
    # each pair (j, j + hd/2) keeps its length; the interleaved pairing (2j, 2j+1) would not
    assert torch.allclose(y[..., :half] ** 2 + y[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2)
    pair_il = y[..., 0::2] ** 2 + y[..., 1::2] ** 2
    assert not torch.allclose(pair_il, x[..., 0::2] ** 2 + x[..., 1::2] ** 2)
    # angle of pair j at position p is p * base^(-2j/hd): check pair 3 at position 5 by hand
    j, p = 3, 5
    a = p * base ** (-2 * j / hd)
    x0, x1 = x[p, 1, j], x[p, 1, j + half]
    assert math.isclose(float(y[p, 1, j]), float(x0 * math.cos(a) - x1 * math.sin(a)), rel_tol=1e-12)
    assert math.isclose(float(y[p, 1, j + half]), float(x0 * math.sin(a) + x1 * math.cos(a)), rel_tol=1e-12)
    # <rope(q, m), rope(k, n)> depends on m - n only
    q, k = r(1, 1, hd), r(1, 1, hd)
    d1 = (plain.rope_neox(q, torch.tensor([7]), base) * plain.rope_neox(k, torch.tensor([3]), base)).sum()
    d2 = (plain.rope_neox(q, torch.tensor([107]), base) * plain.rope_neox(k, torch.tensor([103]), base)).sum()
    assert math.isclose(float(d1), float(d2), rel_tol=1e-9)


# ------------------------------------------------------------------------- short conv
def test_short_conv_is_a_causal_depthwise_convolution():
    T, d, K = 11, 6, 4
    h, w_in, w_conv, w_out = r(T, d), r(3 * d, d), r(d, K), r(d, d)
    got = plain.short_conv(h, w_in, w_conv, w_out)
    bcx = h @ w_in.T
    b, c, x = bcx[:, :d], bcx[:, d:2 * d], bcx[:, 2 * d:]
    u = (b * x).T[None]                                                             # [1, d, T]
    y = F.conv1d(F.pad(u, (K - 1, 0)), w_conv[:, None, :], groups=d)[0].T           # left pad K-1, no bias
    assert torch.allclose(got, (c * y) @ w_out.T)
    # the last tap multiplies the current token: taps [0, .., 0, 1] give y = u
    last = torch.zeros(d, K, dtype=torch.float64)
    last[:, K - 1] = 1
    assert torch.allclose(plain.short_conv(h, w_in, last, torch.eye(d, dtype=torch.float64)), c * (b * x))
    # taps [1, 0, .., 0] give u delayed by K-1 tokens, zero before
    first = torch.zeros(d, K, dtype=torch.float64)
    first[:, 0] = 1
    delayed = torch.cat([torch.zeros(K - 1, d, dtype=torch.float64), (b * x)[:T - K + 1]])
    assert torch.allclose(plain.short_conv(h, w_in, first, torch.eye(d, dtype=torch.float64)), c * delayed)
    # which third is the output gate: zero the middle third of in_proj -> output zero
    w0 = w_in.clone()
    w0[d:2 * d] = 0
    assert torch.equal(plain.short_conv(h, w0, w_conv, w_out), torch.zeros(T, d, dtype=torch.float64))
    # causal: changing token 7 leaves outputs 0..6 as they were
    h2 = h.clone()
    h2[7] += 1
    assert torch.allclose(plain.short_conv(h2, w_in, w_conv, w_out)[:7], got[:7])


# -------------------------------------------------------------------------- attention
def test_attention_reduces_to_library_attention():
    T, d, H, Hkv = 10, 32, 4, 2
    hd = d // H
    h = r(T, d)
    wq, wk, wv, wo = r(H * hd, d), r(Hkv * hd, d), r(Hkv * hd, d), r(d, H * hd)
    ones = torch.ones(hd, dtype=torch.float64)
    got = plain.attention(h, wq, wk, wv, wo, ones, ones, n_head=H, n_kv=Hkv, eps=1e-6, base=1e4)
    # by hand with the library: norm, rope, heads repeated, causal sdpa
    pos = torch.arange(T)
    q = plain.rope_neox(plain.rms_norm((h @ wq.T).reshape(T, H, hd), ones, 1e-6), pos, 1e4)
    k = plain.rope_neox(plain.rms_norm((h @ wk.T).reshape(T, Hkv, hd), ones, 1e-6), pos, 1e4)
    v = (h @ wv.T).reshape(T, Hkv, hd)
    k, v = k.repeat_interleave(H // Hkv, 1), v.repeat_interleave(H // Hkv, 1)
    o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    assert torch.allclose(got, o.transpose(0, 1).reshape(T, d) @ wo.T)
    # head i reads kv head i // (H / Hkv), not i % Hkv: with H=4, Hkv=2, heads 0,1 -> kv 0
    wv2 = wv.clone()
    wv2[hd:] = 0                                            # kv head 1 carries nothing
    got2 = plain.attention(h, wq, wk, wv2, torch.eye(d, dtype=torch.float64), ones, ones, n_head=H, n_kv=Hkv,
                           eps=1e-6, base=1e4)
    assert got2[:, :2 * hd].abs().sum() > 0 and got2[:, 2 * hd:].abs().sum() == 0
    # a single token attends to itself only: output = W_o v
    one = plain.attention(h[:1], wq, wk, wv, wo, ones, ones, n_head=H, n_kv=Hkv, eps=1e-6, base=1e4)
    assert torch.allclose(one, (h[:1] @ wv.T).reshape(1, Hkv, hd).repeat_interleave(2, 1).reshape(1, d) @ wo.T)
    # shifting all positions changes nothing: only distances count
    shifted = plain.attention(h, wq, wk, wv, wo, ones, ones, n_head=H, n_kv=Hkv, eps=1e-6, base=1e4, pos0=500)
    assert torch.allclose(shifted, got, atol=1e-9)
    # the per-head norm uses a weight over the head, and comes before the rotation
    wn = r(hd).abs() + 0.5
    normed = plain.attention(h, wq, wk, wv, wo, wn, ones, n_head=H, n_kv=Hkv, eps=1e-6, base=1e4)
    q2 = plain.rope_neox(plain.rms_norm((h @ wq.T).reshape(T, H, hd), wn, 1e-6), pos, 1e4)
    o2 = F.scaled_dot_product_attention(q2.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    assert torch.allclose(normed, o2.transpose(0, 1).reshape(T, d) @ wo.T)


def test_the_per_head_norm_of_q_and_k_uses_the_models_eps():
    """src/lfm25_engine.c:395 hands the model's one eps to the kernel that norms q and k per head
    (src/lfm25_gpu.cu:420-452: rsqrtf(total_sq / head_dim + eps)), and tools/lfm25_fp64_ref.py:131-132 uses the same
    rms() closure as for the layers' norms.  Configuration G has norm_eps = 0.5, far above a head's mean square, so
    another eps for the heads (1e-5, 1e-6, none) changes the scores many times over.  By hand, without the plain
    implementation's functions: one normed element of q, and the whole first layer's attention for two tokens."""
    cfg, w = util.plain_model("G")
    eps, H, base = cfg["norm_eps"], cfg["num_attention_heads"], cfg["rope_theta"]
    assert eps == 0.5 and cfg["layer_types"][0] == "full_attention" and cfg["num_key_value_heads"] == H
    hd = cfg["hidden_size"] // H
    toks = [3, 77]
    x = w["model.embed_tokens.weight"][toks]                                         # [2, d]
    nw = w["model.layers.0.operator_norm.weight"]
    h = torch.stack([x[t] / math.sqrt(float((x[t] ** 2).sum()) / x.shape[1] + eps) * nw for t in range(2)])
    p = "model.layers.0.self_attn."
    q, k, v = h @ w[p + "q_proj.weight"].T, h @ w[p + "k_proj.weight"].T, h @ w[p + "v_proj.weight"].T
    qn, kn = w[p + "q_layernorm.weight"], w[p + "k_layernorm.weight"]
    head, j = 2, 5
    qh = q[1, head * hd:(head + 1) * hd]
    ms = float((qh ** 2).sum()) / hd
    assert ms < eps / 5                                                              # eps decides the size
    want_q = float(qh[j]) / math.sqrt(ms + eps) * float(qn[j])
    got_q = plain.rms_norm(q.reshape(2, H, hd), qn, eps)[1, head, j]
    assert math.isclose(float(got_q), want_q, rel_tol=1e-12)
    # token 1's attention output in every head, by hand: norm with eps, rotate the halves, two scores, softmax
    def normed_rotated(vec, weight, pos):
        out = torch.empty_like(vec)
        for a in range(H):
            hv = vec[a * hd:(a + 1) * hd]
            hv = hv / math.sqrt(float((hv ** 2).sum()) / hd + eps) * weight
            for i in range(hd // 2):
                ang = pos * base ** (-2.0 * i / hd)
                out[a * hd + i] = hv[i] * math.cos(ang) - hv[i + hd // 2] * math.sin(ang)
                out[a * hd + i + hd // 2] = hv[i] * math.sin(ang) + hv[i + hd // 2] * math.cos(ang)
        return out
    q1, k0, k1 = normed_rotated(q[1], qn, 1), normed_rotated(k[0], kn, 0), normed_rotated(k[1], kn, 1)
    o = torch.empty(H * hd, dtype=torch.float64)
    for a in range(H):
        sl = slice(a * hd, (a + 1) * hd)
        s0, s1 = float(q1[sl] @ k0[sl]) / math.sqrt(hd), float(q1[sl] @ k1[sl]) / math.sqrt(hd)
        p0 = 1.0 / (1.0 + math.exp(s1 - s0))
        o[sl] = p0 * v[0, sl] + (1 - p0) * v[1, sl]
    want = o @ w[p + "out_proj.weight"].T
    got = plain.attention(h, w[p + "q_proj.weight"], w[p + "k_proj.weight"], w[p + "v_proj.weight"], w[p + "out_proj.weight"],
                          qn, kn, n_head=H, n_kv=H, eps=eps, base=base)[1]
    assert torch.allclose(got, want, rtol=1e-10, atol=1e-14)
    # ... and the whole model hands that eps on: with the layers' outputs after the first mixer zeroed, the logits
    # of token 1 are head(norm(x + attention)) with the attention computed above
    w0 = dict(w)
    for name in w:
        if name.endswith("feed_forward.w2.weight") or (name.endswith("out_proj.weight") and ".layers.0." not in name):
            w0[name] = torch.zeros_like(w[name])
    x1 = x[1] + want
    fin = x1 / math.sqrt(float((x1 ** 2).sum()) / x1.shape[0] + eps) * w["model.embedding_norm.weight"]
    assert torch.allclose(plain.forward_logits(cfg, w0, toks)[1], fin @ w["lm_head.weight"].T, rtol=1e-10, atol=1e-14)
    # the pin bites: the same with the heads normed by another eps is far off
    other = plain.attention(h, w[p + "q_proj.weight"], w[p + "k_proj.weight"], w[p + "v_proj.weight"], w[p + "out_proj.weight"],
                            qn, kn, n_head=H, n_kv=H, eps=1e-5, base=base)[1]
    assert (other - want).abs().max() > 0.02 * want.abs().max()


def test_attention_scale_is_one_over_root_of_the_head_size():
    # one head, no rotation effect at position 0 for the key: two tokens, scores by hand
    d = hd = 4
    eye = torch.eye(d, dtype=torch.float64)
    ones = torch.ones(hd, dtype=torch.float64)
    h = torch.tensor([[1.0, 0, 0, 0], [1.0, 0, 0, 0]], dtype=torch.float64)
    wv = torch.zeros(d, d, dtype=torch.float64)
    out = plain.attention(h, eye, eye, eye, eye, ones, ones, n_head=1, n_kv=1, eps=0.0, base=1e4)
    # token 1 sees keys 0 and 1; after the norm q = k = [2, 0, 0, 0]; channel 0 pairs with channel 2
    a = 1.0                                                                          # angle of pair 0 at position 1
    s0 = (2 * math.cos(a)) * 2 / math.sqrt(hd)
    s1 = 4 / math.sqrt(hd)
    p0 = math.exp(s0) / (math.exp(s0) + math.exp(s1))
    assert math.isclose(float(out[1, 0]), 1.0, rel_tol=1e-12)                        # both values are h itself
    q = plain.rope_neox(plain.rms_norm(h.reshape(2, 1, hd), ones, 0.0), torch.arange(2), 1e4)
    s = (q[1, 0] * q[0, 0]).sum() / math.sqrt(hd)
    assert math.isclose(float(s), s0, rel_tol=1e-12)
    assert 0 < p0 < 0.5


# ---------------------------------------------------------------------------- swiglu
def test_swiglu():
    h, wg, wu, wd = r(5, 8), r(12, 8), r(12, 8), r(8, 12)
    assert torch.allclose(plain.swiglu(h, wg, wu, wd), (F.silu(h @ wg.T) * (h @ wu.T)) @ wd.T)
    assert torch.equal(plain.swiglu(h, torch.zeros_like(wg), wu, wd), torch.zeros(5, 8, dtype=torch.float64))
    # the gate is the first matrix: swapping gate and up changes the result
    assert not torch.allclose(plain.swiglu(h, wg, wu, wd), plain.swiglu(h, wu, wg, wd))


# ----------------------------------------------------------------------------- model
def test_model_structure():
    cfg, w = util.plain_model("A")
    toks = util.rand_tokens(12, cfg["vocab_size"], 4)
    base = plain.forward_logits(cfg, w, toks)
    assert base.shape == (12, cfg["vocab_size"])
    # with every output projection zeroed the layers add nothing: logits = head(norm(embedding))
    w0 = dict(w)
    for k in w:
        if k.endswith("out_proj.weight") or k.endswith("feed_forward.w2.weight"):
            w0[k] = torch.zeros_like(w[k])
    emb = w["model.embed_tokens.weight"]
    want = plain.rms_norm(emb[toks], w["model.embedding_norm.weight"], cfg["norm_eps"]) @ emb.T
    assert torch.allclose(plain.forward_logits(cfg, w0, toks), want)
    # causal: logits at position 5 do not depend on later tokens
    other = toks[:6] + util.rand_tokens(6, cfg["vocab_size"], 5)
    assert torch.allclose(plain.forward_logits(cfg, w, other)[:6], base[:6])
    # each layer's kind follows layer_types
    assert [plain.layer_is_conv(cfg, i) for i in range(4)] == [True, True, False, True]
    # an untied head is used instead of the embedding
    cfg_b, w_b = util.plain_model("B")
    toks_b = util.rand_tokens(5, cfg_b["vocab_size"], 6)
    lb = plain.forward_logits(cfg_b, w_b, toks_b)
    w_b2 = dict(w_b)
    w_b2["lm_head.weight"] = w_b["lm_head.weight"] * 2
    assert torch.allclose(plain.forward_logits(cfg_b, w_b2, toks_b), 2 * lb)


def test_float32_run_of_the_plain_model_is_close_to_float64():
    cfg, w = util.plain_model("B")
    toks = util.rand_tokens(40, cfg["vocab_size"], 8)
    w32 = {k: v.float() for k, v in w.items()}
    a = plain.forward_logits(cfg, w, toks)
    b = plain.forward_logits(cfg, w32, toks, dtype=torch.float32)
    assert (a - b.double()).abs().max() < 1e-5


# --------------------------------------------------------------------------- sampler
def test_generator_matches_the_product_generator_and_its_own_definition():
    from tuff_amd.sampling.params import XorShift128Plus as Product
    for seed in (1, 42, 2 ** 63 + 5):
        a, b = XorShift128Plus(seed), Product(seed)
        assert [a.next() for _ in range(5)] == [b.next_u64() for _ in range(5)]
        assert [float(a.uniform()) for _ in range(5)] == [b.uniform() for _ in range(5)]
    g = XorShift128Plus(7)
    us = [float(g.uniform()) for _ in range(2000)]
    assert 0.0 <= min(us) and max(us) <= 1.0 and 0.45 < sum(us) / len(us) < 0.55
    # one step by hand from the seeding rule (src/sampler.c:20-45)
    s0 = 7 ^ 0x8A5CD789635D2DFF
    s1 = ((7 + 0x9E3779B97F4A7C15) & (2 ** 64 - 1)) ^ 0x123456789ABCDEF0
    h = XorShift128Plus.__new__(XorShift128Plus)
    h.s = [s0, s1]
    x, y = s0, s1
    x ^= (x << 23) & (2 ** 64 - 1)
    new1 = x ^ y ^ (x >> 17) ^ (y >> 26)
    assert h.next() == (new1 + y) & (2 ** 64 - 1) and h.s == [s1, new1]


def test_plain_sampler_semantics():
    logits = np.array([1.0, 3.0, 3.0, -2.0, 0.5], dtype=np.float32)
    assert PlainSampler(temp=0.0).sample(logits) == 1                          # first maximum
    # temperature -> 0+ converges to greedy; top_k = 1 is greedy whatever the draw
    assert PlainSampler(temp=1e-4, seed=3).sample(np.array([1.0, 3.0, 2.9, -2.0], dtype=np.float32)) == 1
    assert PlainSampler(temp=5.0, top_k=1, seed=9).sample(logits) == 1
    # min_p keeps tokens with p >= min_p * p_max: with T = 1, ln(0.2) = -1.6: 3.0 and 3.0 only (1.0 is -2)
    seen = {PlainSampler(temp=1.0, min_p=0.2, seed=s).sample(logits) for s in range(1, 60)}
    assert seen == {1, 2}
    # top_p: smallest prefix reaching p; 0.4 -> first token alone is 0.43 of the mass
    seen = {PlainSampler(temp=1.0, top_p=0.4, seed=s).sample(logits) for s in range(1, 60)}
    assert seen == {1}
    # same seed, same stream; the frequencies follow softmax(l / T)
    s1, s2 = PlainSampler(temp=0.8, seed=5), PlainSampler(temp=0.8, seed=5)
    assert [s1.sample(logits) for _ in range(20)] == [s2.sample(logits) for _ in range(20)]
    s = PlainSampler(temp=1.0, seed=17)
    n = 4000
    counts = np.bincount([s.sample(logits) for _ in range(n)], minlength=5) / n
    p = np.exp(logits - logits.max())
    p /= p.sum()
    assert np.abs(counts - p).max() < 0.03
    # repetition penalty: positive logits are divided, negative multiplied, once per ring entry
    s = PlainSampler(temp=1.0, repeat_penalty=2.0, top_k=1, seed=1)
    s.accept(1)
    s.accept(1)
    assert s.sample(np.array([1.0, 3.5, 0.5], dtype=np.float32)) == 0           # 3.5 / 4 < 1.0
    s = PlainSampler(temp=1.0, repeat_penalty=2.0, top_k=1, seed=1)
    s.accept(0)
    assert s.sample(np.array([-1.0, -1.5, -5.0], dtype=np.float32)) == 1        # -1.0 * 2 < -1.5
