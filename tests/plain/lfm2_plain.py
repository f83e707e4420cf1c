"""Plain LFM2 dense decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference (paths relative to the reference
tree).  It reads a model folder with the `safetensors` library and `json`, so it
shares neither loader, nor layers, nor cache with the engine under test.

Everything runs on the CPU in the dtype of the tensors handed in (float64 by
default).

`rnd`: where given, a function applied to every activation that an engine with
bfloat16 activations holds in bfloat16 between two of its operations: the normed
operand of every projection, a projection's output (q, k, v; B, C, X), the normed
and rotated q and k (the cache holds such keys) and v, the softmax weights as the
second product takes them, the attention's output, the gated conv output and the
SwiGLU product.  The residual stream, the sums inside every product, the norms'
statistics, the softmax and the conv's own sums stay as they are.  With
rnd = "round to bfloat16 and back" in float64 arithmetic this is a model of the
rounding noise that any such engine has, however it orders its sums: the
tests' yardstick for an engine's bfloat16 error, in the manner of the reference's
tolerance gate, which measures its engine against another runtime's error
(tools/lfm25_gate.py:117-144).
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------- parts
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w, eps inside the root, weight multiplies.

    tools/lfm25_fp64_ref.py:81-82; src/lfm25_gpu.cu:235,244.
    """
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rope_neox(x: torch.Tensor, pos: torch.Tensor, base: float) -> torch.Tensor:
    """Rotate the pairs (j, j + hd/2) of the last axis by pos * base^(-2j/hd).

    x: [T, heads, hd], pos: [T].  tools/lfm25_fp64_ref.py:90-100;
    src/lfm25_gpu.cu:459-474 (half-split pairs, theta = base^(-2j/hd)).
    """
    hd = x.shape[-1]
    half = hd // 2
    j = torch.arange(half, dtype=torch.float64)
    inv_freq = (torch.tensor(base, dtype=torch.float64) ** (-j * 2.0 / hd)).to(x.dtype)
    a = pos.to(x.dtype)[:, None] * inv_freq[None, :]          # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    x0, x1 = x[..., :half], x[..., half:]
    return torch.cat([x0 * c - x1 * s, x0 * s + x1 * c], dim=-1)


def _same(t):
    return t


def to_bfloat16_and_back(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def short_conv(h: torch.Tensor, w_in: torch.Tensor, w_conv: torch.Tensor,
               w_out: torch.Tensor, rnd=_same) -> torch.Tensor:
    """Gated short convolution over a whole sequence that starts with empty history.

    bcx = W_in h; B, C, X = thirds of bcx; u = B*X;
    y_t = sum_k w[:, k] * u_{t-(K-1)+k} (tap K-1 multiplies the current token,
    missing history is zero); out = W_out (C*y).
    tools/lfm25_fp64_ref.py:118-126; src/lfm25_gpu.cu:378-397.
    h: [T, d]; w_in: [3d, d]; w_conv: [d, K]; w_out: [d, d].
    """
    T, d = h.shape
    K = w_conv.shape[1]
    bcx = rnd(h @ w_in.T)
    b, c, xx = bcx[:, :d], bcx[:, d:2 * d], bcx[:, 2 * d:]
    u = b * xx
    hist = torch.cat([torch.zeros(K - 1, d, dtype=h.dtype), u], dim=0)   # row i = time i-(K-1)
    y = torch.zeros_like(u)
    for k in range(K):
        y = y + hist[k:k + T] * w_conv[:, k]
    return rnd(c * y) @ w_out.T


def attention(h: torch.Tensor, wq, wk, wv, wo, q_norm_w, k_norm_w, *, n_head: int,
              n_kv: int, eps: float, base: float, pos0: int = 0, rnd=_same) -> torch.Tensor:
    """Causal GQA attention with per-head RMSNorm on q and k, then rotation.

    q head i reads kv head i // (n_head // n_kv); scores scaled by 1/sqrt(hd);
    token t sees tokens <= t.  tools/lfm25_fp64_ref.py:128-143;
    src/lfm25_gpu.cu:420-485 (norm then rotation, K cached after both), :506-558.
    """
    T, _ = h.shape
    hd = wq.shape[0] // n_head
    pos = torch.arange(pos0, pos0 + T)
    q = rnd(h @ wq.T).reshape(T, n_head, hd)
    k = rnd(h @ wk.T).reshape(T, n_kv, hd)
    v = rnd(h @ wv.T).reshape(T, n_kv, hd)
    q = rnd(rope_neox(rms_norm(q, q_norm_w, eps), pos, base))
    k = rnd(rope_neox(rms_norm(k, k_norm_w, eps), pos, base))
    g = n_head // n_kv
    k = k.repeat_interleave(g, dim=1)
    v = v.repeat_interleave(g, dim=1)
    s = torch.einsum("thd,shd->hts", q, k) / math.sqrt(hd)
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, float("-inf"))
    s = torch.exp(s - s.max(-1, keepdim=True).values)
    total = s.sum(-1, keepdim=True)
    o = torch.einsum("hts,shd->thd", rnd(s), v) / total.permute(1, 0, 2)
    return rnd(o.reshape(T, n_head * hd)) @ wo.T


def swiglu(h: torch.Tensor, w_gate, w_up, w_down, rnd=_same) -> torch.Tensor:
    """W_down (g / (1 + exp(-g)) * u) with g = W_gate h, u = W_up h.

    tools/lfm25_fp64_ref.py:159-161; src/lfm25_gpu.cu:614-617.
    """
    g = h @ w_gate.T
    u = h @ w_up.T
    return rnd(g / (1.0 + torch.exp(-g)) * u) @ w_down.T


# --------------------------------------------------------------------------- model
def ff_dim(cfg: dict) -> int:
    """Width of the feed-forward from the block_* keys.

    The reference reads the adjusted value from its file (src/lfm25_model.c:99-100);
    the rule here is fixed by the vectors 384 -> 256 (multiple_of 64) and
    12288 -> 8192, 16128 -> 10752, 10368 -> 6912 (multiple_of 256).
    """
    f = int(cfg["block_ff_dim"])
    if cfg.get("block_auto_adjust_ff_dim", False):
        f = int(2 * f / 3)
        mult = cfg.get("block_ffn_dim_multiplier")
        if mult is not None:
            f = int(mult * f)
        m = int(cfg.get("block_multiple_of", 256))
        f = m * ((f + m - 1) // m)
    return f


def read_model(model_dir: str, dtype=torch.float64):
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return cfg, tensors


def layer_is_conv(cfg: dict, i: int) -> bool:
    return cfg["layer_types"][i] == "conv"


def forward_logits(cfg: dict, w: dict, tokens, dtype=torch.float64, rnd=_same) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence starting at position 0.

    Pre-norm decoder, two residual sub-blocks a layer: x += mixer(norm(x));
    x += ffn(norm(x)); logits = head(norm(x)); the head is the embedding when tied.
    src/lfm25_engine.c:370-430; tools/lfm25_fp64_ref.py:113-163.
    """
    eps = float(cfg["norm_eps"])
    base = float(cfg["rope_theta"])
    n_head = int(cfg["num_attention_heads"])
    n_kv = int(cfg["num_key_value_heads"])
    tok = torch.as_tensor(tokens, dtype=torch.long)
    x = w["model.embed_tokens.weight"][tok].to(dtype)
    for i in range(int(cfg["num_hidden_layers"])):
        p = f"model.layers.{i}."
        h = rnd(rms_norm(x, w[p + "operator_norm.weight"], eps))
        if layer_is_conv(cfg, i):
            conv_w = w[p + "conv.conv.weight"]
            conv_w = conv_w.reshape(conv_w.shape[0], conv_w.shape[-1])
            o = short_conv(h, w[p + "conv.in_proj.weight"], conv_w, w[p + "conv.out_proj.weight"], rnd=rnd)
        else:
            o = attention(h, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.k_proj.weight"],
                          w[p + "self_attn.v_proj.weight"], w[p + "self_attn.out_proj.weight"],
                          w[p + "self_attn.q_layernorm.weight"], w[p + "self_attn.k_layernorm.weight"],
                          n_head=n_head, n_kv=n_kv, eps=eps, base=base, rnd=rnd)
        x = x + o
        h = rnd(rms_norm(x, w[p + "ffn_norm.weight"], eps))
        x = x + swiglu(h, w[p + "feed_forward.w1.weight"], w[p + "feed_forward.w3.weight"],
                       w[p + "feed_forward.w2.weight"], rnd=rnd)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return rnd(rms_norm(x, w["model.embedding_norm.weight"], eps)) @ head.T


def greedy_generate(cfg: dict, w: dict, prompt, n_new: int, dtype=torch.float64):
    """Greedy continuation by re-running the whole sequence for every new token.

    Exact ties go to the lowest id (src/lfm25_gpu.cu:691-692; src/sampler.c:103-113).
    Returns (ids, margins) where margin = top1 - top2 logit at each step.
    """
    ids = list(prompt)
    out, margins = [], []
    for _ in range(n_new):
        row = forward_logits(cfg, w, ids, dtype)[-1]
        top = torch.topk(row, 2).values
        best = int(torch.nonzero(row == row.max())[0])
        out.append(best)
        margins.append(float(top[0] - top[1]))
        ids.append(best)
    return out, margins
