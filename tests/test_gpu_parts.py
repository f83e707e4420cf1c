"""Each part alone on the GPU against its plain counterpart, at sizes of its own, and a toy
mixer with state of its own that is registered, built and stepped from this file."""
import dataclasses
import math
from typing import ClassVar

import pytest
import torch

import util
from plain import lfm2_plain as plain

pytestmark = pytest.mark.gpu


def _r(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


class Harness:
    """Runs one mixer (or any callable taking h, ctx, cache, residual) over requests cut into steps."""

    def __init__(self, gpu, dtype, cache_spec, page_size=16, pages=64):
        from tuff_amd.cache.manager import CacheLayout, CacheManager
        from tuff_amd.cache.storage import CacheStorage
        from tuff_amd.parts.base import Runtime
        self.gpu, self.dtype = gpu, dtype
        self.rt = Runtime(gpu, dtype)
        self.mgr = CacheManager(CacheLayout.from_specs({0: cache_spec}), page_size, pages, 4)
        self.storage = CacheStorage(self.mgr, dtype, gpu, poison=True)

    def run(self, forward, inputs: dict, cuts: dict, d_out: int):
        """inputs: {rid: [n, d] float tensor}; cuts: {rid: [portion sizes]}; all requests advance together."""
        from tuff_amd.engine.batch import StepEntry, build_context
        done = {rid: 0 for rid in inputs}
        outs = {rid: [] for rid in inputs}
        for rid in inputs:
            slot = self.mgr.admit(rid)
            self.storage.zero_slot(slot)
        step = 0
        while any(done[r] < inputs[r].shape[0] for r in inputs):
            entries, rows = [], []
            for rid, x in inputs.items():
                if step < len(cuts[rid]):
                    n = cuts[rid][step]
                    self.mgr.extend(rid, n)
                    entries.append(StepEntry(rid, [0] * n, []))
                    rows.append(x[done[rid]:done[rid] + n])
            ctx = build_context(entries, self.mgr, self.gpu, 1)
            h = torch.cat(rows).to(self.gpu, self.dtype).contiguous()
            residual = torch.zeros(h.shape[0], d_out, device=self.gpu)
            forward(h, ctx, self.storage.views.get(0), residual)
            t = 0
            for e in entries:
                outs[e.req_id].append(residual[t:t + len(e.tokens)].cpu())
                done[e.req_id] += len(e.tokens)
                t += len(e.tokens)
            step += 1
        return {rid: torch.cat(v).double() for rid, v in outs.items()}


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 3e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d,H,Hkv,hd,window,theta", [(48, 3, 1, 16, None, 1e4), (80, 2, 2, 40, 21, 1e6), (64, 8, 2, 8, None, 50.0)])
def test_attention_mixer_alone(gpu, dtype, d, H, Hkv, hd, window, theta):
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.rope import Rotary
    names = {k: k for k in ("q", "k", "v", "o", "q_norm", "k_norm")}
    mixer = AttentionMixer(d, H, Hkv, hd, names=names, qk_norm_eps=1e-6, position=Rotary(hd, theta), window=window)
    w = {"q": _r(H * hd, d, seed=1, scale=0.3), "k": _r(Hkv * hd, d, seed=2, scale=0.3), "v": _r(Hkv * hd, d, seed=3, scale=0.3),
         "o": _r(d, H * hd, seed=4, scale=0.3), "q_norm": 1 + _r(hd, seed=5, scale=0.1), "k_norm": 1 + _r(hd, seed=6, scale=0.1)}
    w = {k: v.to(dtype) for k, v in w.items()}
    hs = Harness(gpu, dtype, mixer.cache_spec())
    mixer.bind({k: v.to(gpu) for k, v in w.items()}, hs.rt)
    inputs = {"a": _r(70, d, seed=7).to(dtype).float(), "b": _r(37, d, seed=8).to(dtype).float()}
    got = hs.run(mixer.forward, inputs, {"a": [33, 1, 1, 30, 5], "b": [2, 20, 15]}, d)
    wd = {k: v.double() for k, v in w.items()}
    for rid, x in inputs.items():
        want = plain.attention(x.double(), wd["q"], wd["k"], wd["v"], wd["o"], wd["q_norm"], wd["k_norm"],
                               n_head=H, n_kv=Hkv, eps=1e-6, base=theta)
        if window:                       # the plain function is full attention: redo it with the window
            T = x.shape[0]
            pos = torch.arange(T)
            q = plain.rope_neox(plain.rms_norm((x.double() @ wd["q"].T).reshape(T, H, hd), wd["q_norm"], 1e-6), pos, theta)
            k = plain.rope_neox(plain.rms_norm((x.double() @ wd["k"].T).reshape(T, Hkv, hd), wd["k_norm"], 1e-6), pos, theta)
            v = (x.double() @ wd["v"].T).reshape(T, Hkv, hd)
            k, v = k.repeat_interleave(H // Hkv, 1), v.repeat_interleave(H // Hkv, 1)
            s = torch.einsum("thd,shd->hts", q, k) / math.sqrt(hd)
            i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
            s = s.masked_fill(~((j <= i) & (j > i - window)), float("-inf"))
            want = torch.einsum("hts,shd->thd", torch.softmax(s, -1), v).reshape(T, H * hd) @ wd["o"].T
        assert (got[rid] - want).abs().max() <= tol(dtype) * float(want.abs().max()), rid


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_mixer_without_norm_or_position_is_plain_attention(gpu, dtype):
    """No rotation, no norm, one head: the library's causal attention."""
    from tuff_amd.parts.attention import AttentionMixer
    d = hd = 32
    mixer = AttentionMixer(d, 1, 1, hd, names={k: k for k in "qkvo"})
    w = {k: _r(d, d, seed=i, scale=0.2).to(dtype) for i, k in enumerate("qkvo")}
    hs = Harness(gpu, dtype, mixer.cache_spec())
    mixer.bind({k: v.to(gpu) for k, v in w.items()}, hs.rt)
    x = _r(50, d, seed=9).to(dtype).float()
    got = hs.run(mixer.forward, {"a": x}, {"a": [17, 33]}, d)["a"]
    xd = x.double()
    q, k, v = (xd @ w[n].double().T for n in "qkv")
    o = torch.nn.functional.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    want = o @ w["o"].double().T
    assert (got - want).abs().max() <= tol(dtype) * float(want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d,K", [(40, 3), (72, 5)])
def test_shortconv_mixer_alone(gpu, dtype, d, K):
    from tuff_amd.parts.shortconv import ShortConvMixer
    mixer = ShortConvMixer(d, K, names={"in_proj": "i", "conv": "c", "out_proj": "o"})
    w = {"i": _r(3 * d, d, seed=1, scale=0.3).to(dtype), "c": _r(d, K, seed=2, scale=0.5).to(dtype),
         "o": _r(d, d, seed=3, scale=0.3).to(dtype)}
    hs = Harness(gpu, dtype, mixer.cache_spec())
    mixer.bind({k: v.to(gpu) for k, v in w.items()}, hs.rt)
    inputs = {"a": _r(30, d, seed=4).to(dtype).float(), "b": _r(9, d, seed=5).to(dtype).float()}
    got = hs.run(mixer.forward, inputs, {"a": [1, 1, 20, 2, 6], "b": [5, 1, 3]}, d)
    for rid, x in inputs.items():
        want = plain.short_conv(x.double(), w["i"].double(), w["c"].double(), w["o"].double())
        assert (got[rid] - want).abs().max() <= tol(dtype) * float(want.abs().max()), rid


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_norm_and_block_alone(gpu, dtype):
    from tuff_amd.parts.base import Runtime
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.ffn import SwiGLU
    from tuff_amd.parts.norm import RMSNorm
    from tuff_amd.parts.shortconv import ShortConvMixer
    d, F, K, eps = 56, 104, 3, 1e-4
    rt = Runtime(gpu, dtype)
    w = {"g": _r(F, d, seed=1, scale=0.3), "u": _r(F, d, seed=2, scale=0.3), "dn": _r(d, F, seed=3, scale=0.3),
         "n1": 1 + _r(d, seed=4, scale=0.1), "n2": 1 + _r(d, seed=5, scale=0.1),
         "i": _r(3 * d, d, seed=6, scale=0.3), "c": _r(d, K, seed=7, scale=0.5), "o": _r(d, d, seed=8, scale=0.3)}
    w = {k: v.to(dtype) for k, v in w.items()}
    wg = {k: v.to(gpu) for k, v in w.items()}
    wd = {k: v.double() for k, v in w.items()}
    x = _r(13, d, seed=9)
    # norm
    norm = RMSNorm(d, eps, "n1")
    norm.bind(wg, rt)
    h = norm.forward(x.to(gpu))
    want_h = plain.rms_norm(x.double(), wd["n1"], eps)
    assert h.dtype == dtype and (h.cpu().double() - want_h).abs().max() <= tol(dtype) * float(want_h.abs().max())
    # feed-forward
    ffn = SwiGLU(d, F, names={"gate": "g", "up": "u", "down": "dn"})
    ffn.bind(wg, rt)
    res = x.to(gpu).clone()
    ffn.forward(h, None, res)
    want = x.double() + plain.swiglu(h.cpu().double(), wd["g"], wd["u"], wd["dn"])
    assert (res.cpu().double() - want).abs().max() <= tol(dtype) * float(want.abs().max())
    # the block: x += mixer(norm1 x); x += ffn(norm2 x)
    block = PreNormBlock(RMSNorm(d, eps, "n1"), ShortConvMixer(d, K, names={"in_proj": "i", "conv": "c", "out_proj": "o"}),
                         RMSNorm(d, eps, "n2"), SwiGLU(d, F, names={"gate": "g", "up": "u", "down": "dn"}))
    assert sorted(dd.name for dd in block.weight_decls()) == sorted(w)
    hs = Harness(gpu, dtype, block.mixer.cache_spec())
    block.bind(wg, hs.rt)

    def fwd(h_in, ctx, cache, residual):
        residual.copy_(h_in.float())
        block.forward(residual, ctx, cache)
    got = hs.run(fwd, {"a": x.to(dtype).float()}, {"a": [4, 9]}, d)["a"]
    xd = x.to(dtype).double()
    y = xd + plain.short_conv(plain.rms_norm(xd, wd["n1"], eps), wd["i"], wd["c"], wd["o"])
    y = y + plain.swiglu(plain.rms_norm(y, wd["n2"], eps), wd["g"], wd["u"], wd["dn"])
    assert (got - y).abs().max() <= tol(dtype) * float(y.abs().max())


def test_position_encoding_of_its_own_goes_through_apply(gpu):
    """A position encoding that is not rotary: the mixer norms, calls apply(), then writes the cache."""
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.base import PositionEncoding

    class SignFlip(PositionEncoding):
        """Negates q and k at odd positions (q.k of two odd or two even positions is unchanged)."""
        calls = 0

        def apply(self, q, k, positions):
            SignFlip.calls += 1
            sign = (1 - 2 * (positions % 2)).to(q.dtype)[:, None]
            q.mul_(sign)
            k.mul_(sign)
    d = hd = 16
    w = {k: _r(d, d, seed=i, scale=0.4) for i, k in enumerate("qkvo")}
    x = _r(12, d, seed=5)
    outs = []
    for pos in (SignFlip(), None):
        mixer = AttentionMixer(d, 1, 1, hd, names={k: k for k in "qkvo"}, position=pos)
        hs = Harness(gpu, torch.float32, mixer.cache_spec())
        mixer.bind({k: v.to(gpu) for k, v in w.items()}, hs.rt)
        outs.append(hs.run(mixer.forward, {"a": x}, {"a": [5, 7]}, d)["a"])
    assert SignFlip.calls == 2
    xd = x.double()
    q, k, v = (xd @ w[n].double().T for n in "qkv")
    sign = (1 - 2 * (torch.arange(12) % 2)).double()[:, None]
    o = torch.nn.functional.scaled_dot_product_attention((q * sign)[None], (k * sign)[None], v[None], is_causal=True)[0]
    assert (outs[0] - o @ w["o"].double().T).abs().max() < 1e-5
    assert (outs[0] - outs[1]).abs().max() > 1e-3


# ---------------------------------------------------------------------- a toy mixer
def test_toy_mixer_with_state_is_registered_built_and_stepped(gpu):
    """A leaky running sum s_t = a * s_{t-1} + h_t (state [d] per request), out = W s_t, defined
    here, put into an architecture of its own, run through Engine.step in different cuttings."""
    from tuff_amd.config.base import ModelConfig
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models import registry
    from tuff_amd.models.decoder import DecoderModel
    from tuff_amd.parts.base import MIXERS, FixedState, Mixer, WeightDecl
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.ffn import SwiGLU
    from tuff_amd.parts.norm import RMSNorm

    class LeakySum(Mixer):
        def __init__(self, d, decay, name):
            self.d, self.decay, self.name = d, decay, name

        def weight_decls(self):
            return [WeightDecl(self.name, (self.d, self.d))]

        def cache_spec(self):
            return FixedState((self.d,))

        def bind(self, weights, rt):
            self.rt, self.w = rt, weights[self.name].float()

        def forward(self, h, ctx, cache, residual, write_cache=True):
            hf = h.float()
            slots = ctx.state_slot.tolist()
            t = 0
            for r, n in enumerate(ctx.host["q_len"].tolist()):
                s = cache.state[slots[r]].clone()
                for i in range(n):
                    s = self.decay * s + hf[t + i]
                    residual[t + i] += s @ self.w.T
                if write_cache:
                    cache.state[slots[r]] = s
                t += n

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyLeakyForCausalLM"
        vocab_size: int
        hidden_size: int
        num_hidden_layers: int
        decay: float
        ffn: int

    def build(cfg):
        blocks = [PreNormBlock(RMSNorm(cfg.hidden_size, 1e-5, f"l{i}.n1"),
                               MIXERS.get("leaky_sum")(cfg.hidden_size, cfg.decay, f"l{i}.mix"),
                               RMSNorm(cfg.hidden_size, 1e-5, f"l{i}.n2"),
                               SwiGLU(cfg.hidden_size, cfg.ffn, names={"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}))
                  for i in range(cfg.num_hidden_layers)]
        return DecoderModel(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                            embedding=WeightDecl("emb", (cfg.vocab_size, cfg.hidden_size)), blocks=blocks,
                            final_norm=RMSNorm(cfg.hidden_size, 1e-5, "fn"))

    MIXERS.register("leaky_sum", LeakySum)
    registry.register_architecture("ToyLeakyForCausalLM", ToyConfig, build)
    try:
        cfg = registry.config_from_dict({"architectures": ["ToyLeakyForCausalLM"], "vocab_size": 97, "hidden_size": 24,
                                         "num_hidden_layers": 2, "decay": 0.7, "ffn": 40})
        from tuff_amd.weights.random_init import random_weights
        model = registry.build_model(cfg)
        w32 = random_weights(model.weight_decls(), 3, torch.float32, "cpu")
        eng = Engine(model, {k: v.to(gpu) for k, v in w32.items()}, dtype="float32", max_tokens=256)
        assert eng.layout.states and not eng.layout.paged
        reqs = {"a": util.rand_tokens(19, 97, 1), "b": util.rand_tokens(8, 97, 2)}
        whole = util.run_plan(eng, util.plan_whole(reqs))
        single = util.run_plan(eng, util.plan_tail(reqs, 100))
        mixed = util.run_plan(eng, util.plan_mixed(reqs, seed=1, decode_tail=3))
        for rid in reqs:
            assert (whole[rid] - single[rid]).abs().max() < 1e-5
            assert (whole[rid] - mixed[rid]).abs().max() < 1e-5
        # against a plain loop over the same weights
        w = {k: v.double() for k, v in w32.items()}
        for rid, toks in reqs.items():
            x = w["emb"][toks]
            for i in range(2):
                h = plain.rms_norm(x, w[f"l{i}.n1"], 1e-5)
                s = torch.zeros(24, dtype=torch.float64)
                rows = []
                for t in range(h.shape[0]):
                    s = 0.7 * s + h[t]
                    rows.append(s @ w[f"l{i}.mix"].T)
                x = x + torch.stack(rows)
                x = x + plain.swiglu(plain.rms_norm(x, w[f"l{i}.n2"], 1e-5), w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])
            want = plain.rms_norm(x, w["fn"], 1e-5) @ w["emb"].T
            util.assert_close_f32(whole[rid], want, rid)
    finally:
        MIXERS.unregister("leaky_sum")
        registry.unregister_architecture("ToyLeakyForCausalLM")


def test_toy_mixer_with_several_cache_entries(gpu):
    """A mixer that keeps three things per request: the last input row (a convolution's tail), a
    decaying matrix of outer products (a recurrent state) and a count of the tokens seen, in int32.
    cache_spec() returns a tuple and forward() is handed a tuple of views.  Beside it in the same
    model an attention layer with paged keys and values.  Whole, token by token and mixed, against a
    plain loop; the counter must hold the request's length after every step."""
    from tuff_amd.config.base import ModelConfig
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models import registry
    from tuff_amd.models.decoder import DecoderModel
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.base import MIXERS, FixedState, Mixer, PagedKV, WeightDecl
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.ffn import SwiGLU
    from tuff_amd.parts.norm import RMSNorm
    from tuff_amd.weights.random_init import random_weights
    d, dk, V, gamma, eps = 24, 8, 89, 0.8, 1e-5
    seen_counts = {}

    class TailAndMatrix(Mixer):
        def __init__(self, d, dk, gamma, name):
            self.d, self.dk, self.gamma, self.name = d, dk, gamma, name

        def weight_decls(self):
            return [WeightDecl(self.name, (self.d, self.d))]

        def cache_spec(self):
            return (FixedState((self.d,)), FixedState((self.dk, self.d)), FixedState((1,), "int32"))

        def bind(self, weights, rt):
            self.rt, self.w = rt, weights[self.name].float()

        def forward(self, h, ctx, cache, residual, write_cache=True):
            tail, matrix, count = cache                           # views in the order of the declarations
            assert count.state.dtype == torch.int32 and matrix.state.shape[1:] == (self.dk, self.d)
            hf = h.float()
            slots = ctx.state_slot.tolist()
            t = 0
            for r, n in enumerate(ctx.host["q_len"].tolist()):
                prev, S = tail.state[slots[r]].clone(), matrix.state[slots[r]].clone()
                for i in range(n):
                    x = hf[t + i]
                    S = self.gamma * S + torch.outer(x[:self.dk], x + prev)
                    residual[t + i] += (x[:self.dk] @ S) @ self.w.T
                    prev = x
                if write_cache:
                    tail.state[slots[r]], matrix.state[slots[r]] = prev, S
                    count.state[slots[r]] += n
                    # zeroed when the slot was taken, then every token counted once, however the request was cut
                    assert int(count.state[slots[r], 0]) == int(ctx.host["ctx_len"][r])
                    seen_counts[slots[r]] = seen_counts.get(slots[r], 0) + 1
                t += n

    @dataclasses.dataclass
    class Cfg(ModelConfig):
        architecture: ClassVar[str] = "ToySeveralForCausalLM"
        vocab_size: int

    def build(cfg):
        def ffn(i):
            return SwiGLU(d, 40, names={"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"})
        blocks = [PreNormBlock(RMSNorm(d, eps, "l0.n1"), MIXERS.get("tail_and_matrix")(d, dk, gamma, "l0.mix"),
                               RMSNorm(d, eps, "l0.n2"), ffn(0)),
                  PreNormBlock(RMSNorm(d, eps, "l1.n1"), AttentionMixer(d, 3, 1, 8, names={k: f"l1.{k}" for k in "qkvo"}),
                               RMSNorm(d, eps, "l1.n2"), ffn(1))]
        return DecoderModel(vocab_size=cfg.vocab_size, hidden_size=d, embedding=WeightDecl("emb", (cfg.vocab_size, d)),
                            blocks=blocks, final_norm=RMSNorm(d, eps, "fn"))

    MIXERS.register("tail_and_matrix", TailAndMatrix)
    registry.register_architecture("ToySeveralForCausalLM", Cfg, build)
    try:
        model = registry.build_model(registry.config_from_dict({"architectures": ["ToySeveralForCausalLM"], "vocab_size": V}))
        assert model.cache_specs == {(0, 0): FixedState((d,)), (0, 1): FixedState((dk, d)), (0, 2): FixedState((1,), "int32"),
                                     1: PagedKV(1, 8, None)}
        w32 = random_weights(model.weight_decls(), 5, torch.float32, "cpu")
        eng = Engine(model, {k: v.to(gpu) for k, v in w32.items()}, dtype="float32", max_tokens=256, poison_cache=True)
        assert len(eng.layout.states) == 3 and len(eng.layout.paged) == 1
        assert eng.layout.state_bytes_per_request() == 4 * (d + dk * d + 1)
        reqs = {"a": util.rand_tokens(21, V, 1), "b": util.rand_tokens(9, V, 2), "c": util.rand_tokens(14, V, 3)}
        whole = util.run_plan(eng, util.plan_whole(reqs))
        assert seen_counts
        single = util.run_plan(eng, util.plan_tail(reqs, 100))
        mixed = util.run_plan(eng, util.plan_mixed(reqs, seed=4, decode_tail=4))
        w = {k: v.double() for k, v in w32.items()}
        for rid, toks in reqs.items():
            x = w["emb"][toks]
            h = plain.rms_norm(x, w["l0.n1"], eps)
            S, prev, rows = torch.zeros(dk, d, dtype=torch.float64), torch.zeros(d, dtype=torch.float64), []
            for t in range(h.shape[0]):
                S = gamma * S + torch.outer(h[t, :dk], h[t] + prev)
                rows.append((h[t, :dk] @ S) @ w["l0.mix"].T)
                prev = h[t]
            x = x + torch.stack(rows)
            x = x + plain.swiglu(plain.rms_norm(x, w["l0.n2"], eps), w["l0.g"], w["l0.u"], w["l0.d"])
            h = plain.rms_norm(x, w["l1.n1"], eps)
            q, k, v = (h @ w[f"l1.{n}"].T for n in "qkv")
            o = torch.nn.functional.scaled_dot_product_attention(q.reshape(-1, 3, 8).transpose(0, 1)[None],
                                                                 k.reshape(-1, 1, 8).transpose(0, 1)[None].expand(1, 3, -1, -1),
                                                                 v.reshape(-1, 1, 8).transpose(0, 1)[None].expand(1, 3, -1, -1),
                                                                 is_causal=True)[0].transpose(0, 1).reshape(-1, 24)
            x = x + o @ w["l1.o"].T
            x = x + plain.swiglu(plain.rms_norm(x, w["l1.n2"], eps), w["l1.g"], w["l1.u"], w["l1.d"])
            want = plain.rms_norm(x, w["fn"], eps) @ w["emb"].T
            for got in (whole, single, mixed):
                util.assert_close_f32(got[rid], want, rid)
    finally:
        MIXERS.unregister("tail_and_matrix")
        registry.unregister_architecture("ToySeveralForCausalLM")


@pytest.mark.parametrize("value_rows", [False, True])
def test_toy_mixer_with_keys_narrower_than_values(gpu, value_rows):
    """A mixer whose keys are 8 wide and whose values are the model's width, in one PagedKV entry with
    a window: the pool is laid out by the declaration ([pages, heads, page, 8] and [pages, heads, 24,
    page], or with value_rows [pages, heads, page, 24]: values a row a position, as a mixer with kernels of
    its own may want them), pages behind the window go back, and the framework's own attention refuses
    such a cache by its shape.  Whole, token by token and mixed with few pages, against a plain loop."""
    from tuff_amd.config.base import ModelConfig
    from tuff_amd.csrc import ops
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models import registry
    from tuff_amd.models.decoder import DecoderModel
    from tuff_amd.parts.base import MIXERS, Mixer, PagedKV, WeightDecl
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.ffn import SwiGLU
    from tuff_amd.parts.norm import RMSNorm
    from tuff_amd.weights.random_init import random_weights
    d, dk, V, eps, window = 24, 8, 83, 1e-5, 20
    shapes = {}

    class NarrowKeys(Mixer):
        def __init__(self, d, dk, window, name):
            self.d, self.dk, self.window, self.name = d, dk, window, name

        def weight_decls(self):
            return [WeightDecl(self.name + ".q", (self.dk, self.d)), WeightDecl(self.name + ".k", (self.dk, self.d))]

        def cache_spec(self):
            return PagedKV(1, self.dk, self.window, value_dim=self.d, value_rows=value_rows)

        def bind(self, weights, rt):
            self.rt, self.wq, self.wk = rt, weights[self.name + ".q"].float(), weights[self.name + ".k"].float()

        def forward(self, h, ctx, cache, residual, write_cache=True):
            shapes["k"], shapes["v"] = tuple(cache.k.shape[1:]), tuple(cache.v.shape[1:])
            ps, g = cache.page_size, ctx.groups[cache.group]
            hf = h.float()
            q, k = hf @ self.wq.T, hf @ self.wk.T
            assert write_cache
            slot = g.slot_mapping.long()
            cache.k[slot // ps, 0, slot % ps] = k.to(cache.k.dtype)
            if value_rows:
                cache.v[slot // ps, 0, slot % ps] = hf.to(cache.v.dtype)
            else:
                cache.v[slot // ps, 0, :, slot % ps] = hf.to(cache.v.dtype)
            pos, req = ctx.positions.tolist(), ctx.req_of_token.tolist()
            for t in range(ctx.T):
                lo = max(0, pos[t] - self.window + 1)
                at = torch.arange(lo, pos[t] + 1, device=h.device)
                page = g.block_table[req[t]].long()[at // ps]
                assert int(page.min()) >= 0                        # no page of the window was given back
                keys = cache.k[page, 0, at % ps].float()
                vals = (cache.v[page, 0, at % ps] if value_rows else cache.v[page, 0, :, at % ps]).float()
                p = torch.softmax(keys @ q[t] / self.dk ** 0.5, 0)
                residual[t] += p @ vals

    @dataclasses.dataclass
    class Cfg(ModelConfig):
        architecture: ClassVar[str] = "ToyNarrowKeysForCausalLM"
        vocab_size: int

    def build(cfg):
        blocks = [PreNormBlock(RMSNorm(d, eps, "n1"), MIXERS.get("narrow_keys")(d, dk, window, "mix"), RMSNorm(d, eps, "n2"),
                               SwiGLU(d, 40, names={"gate": "g", "up": "u", "down": "d"}))]
        return DecoderModel(vocab_size=cfg.vocab_size, hidden_size=d, embedding=WeightDecl("emb", (cfg.vocab_size, d)),
                            blocks=blocks, final_norm=RMSNorm(d, eps, "fn"))

    MIXERS.register("narrow_keys", NarrowKeys)
    registry.register_architecture("ToyNarrowKeysForCausalLM", Cfg, build)
    try:
        model = registry.build_model(registry.config_from_dict({"architectures": ["ToyNarrowKeysForCausalLM"], "vocab_size": V}))
        assert model.cache_specs == {0: PagedKV(1, dk, window, d, value_rows)}
        w32 = random_weights(model.weight_decls(), 6, torch.float32, "cpu")
        eng = Engine(model, {k: v.to(gpu) for k, v in w32.items()}, dtype="float32", max_tokens=192, poison_cache=True)
        assert eng.layout.bytes_per_token(4) == 4 * (dk + d)
        reqs = {"a": util.rand_tokens(70, V, 1), "b": util.rand_tokens(45, V, 2), "c": util.rand_tokens(52, V, 3)}
        whole = util.run_plan(eng, util.plan_whole(reqs))
        ps = eng.manager.page_size
        assert shapes == {"k": (1, ps, dk), "v": (1, ps, d) if value_rows else (1, d, ps)}
        single = util.run_plan(eng, util.plan_tail(reqs, 100))
        mixed = util.run_plan(eng, util.plan_mixed(reqs, seed=7, decode_tail=6))
        view = eng.storage.views[0]
        with pytest.raises(ops.KernelError, match="v_cache"):
            ops.attention_general(torch.zeros(1, dk, device=gpu), view.k, view.v, torch.zeros(1, dk, device=gpu),
                                  block_table=torch.zeros(1, 1, dtype=torch.int32, device=gpu),
                                  req_of_token=torch.zeros(1, dtype=torch.int32, device=gpu),
                                  positions=torch.zeros(1, dtype=torch.int32, device=gpu), H=1, Hkv=1, hd=dk, page_size=ps)
        w = {k: v.double() for k, v in w32.items()}
        for rid, toks in reqs.items():
            x = w["emb"][toks]
            h = plain.rms_norm(x, w["n1"], eps)
            q, k = h @ w["mix.q"].T, h @ w["mix.k"].T
            n = h.shape[0]
            i = torch.arange(n)
            seen = (i[None, :] <= i[:, None]) & (i[None, :] > i[:, None] - window)
            score = (q @ k.T / dk ** 0.5).masked_fill(~seen, float("-inf"))
            x = x + torch.softmax(score, -1) @ h
            x = x + plain.swiglu(plain.rms_norm(x, w["n2"], eps), w["g"], w["u"], w["d"])
            want = plain.rms_norm(x, w["fn"], eps) @ w["emb"].T
            for got in (whole, single, mixed):
                util.assert_close_f32(got[rid], want, rid)
    finally:
        MIXERS.unregister("narrow_keys")
        registry.unregister_architecture("ToyNarrowKeysForCausalLM")


# ------------------------------------------------------- run order and cache groups as data
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_run_twice_a_shared_cache_and_a_window_group(gpu, dtype):
    """A toy architecture whose run order names block 0 twice (two cache entries of its own) and
    lets block 2 read the keys and values block 1 writes; block 0 has a window of 24, so its
    entries form a page group of their own whose pages are given back as the window moves on.
    Whole, in portions and mixed with few pages, against a plain loop."""
    from tuff_amd.config.base import ModelConfig
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models import registry
    from tuff_amd.models.decoder import DecoderModel, LayerRun
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.base import WeightDecl
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.ffn import SwiGLU
    from tuff_amd.parts.norm import RMSNorm
    from tuff_amd.parts.rope import Rotary
    from tuff_amd.weights.random_init import random_weights
    d, H, Hkv, hd, ffn, V, W, theta, eps = 64, 4, 2, 16, 96, 211, 24, 1e4, 1e-5

    @dataclasses.dataclass
    class OrderConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyOrderForCausalLM"
        vocab_size: int

    def names(i):
        return {k: f"l{i}.{k}" for k in ("q", "k", "v", "o", "q_norm", "k_norm")}

    def build(cfg):
        def block(i, window):
            return PreNormBlock(RMSNorm(d, eps, f"l{i}.n1"),
                                AttentionMixer(d, H, Hkv, hd, names=names(i), qk_norm_eps=eps, position=Rotary(hd, theta),
                                               window=window),
                                RMSNorm(d, eps, f"l{i}.n2"),
                                SwiGLU(d, ffn, names={"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}))
        return DecoderModel(vocab_size=cfg.vocab_size, hidden_size=d, embedding=WeightDecl("emb", (cfg.vocab_size, d)),
                            blocks=[block(0, W), block(1, None), block(2, None)], final_norm=RMSNorm(d, eps, "fn"),
                            schedule=[LayerRun(0), LayerRun(1, cache=7), LayerRun(0), LayerRun(2, cache=7, writes=False)])

    registry.register_architecture("ToyOrderForCausalLM", OrderConfig, build)
    try:
        cfg = registry.config_from_dict({"architectures": ["ToyOrderForCausalLM"], "vocab_size": V})
        model = registry.build_model(cfg)
        stored = torch.float32 if dtype == "float32" else torch.bfloat16
        weights = random_weights(model.weight_decls(), 4, stored, "cpu", stored_dtype=stored)
        reqs = {f"r{i}": util.rand_tokens(n, V, 30 + i) for i, n in enumerate([90, 61, 75, 40, 52])}
        plan = util.plan_mixed(reqs, seed=3, decode_tail=20)
        eng = Engine(model, {k: v.to(gpu) for k, v in weights.items()}, dtype=dtype, page_size=16,
                     max_tokens=util.live_tokens_peak(plan))
        assert sorted(w is None for w in eng.layout.group_windows) == [False, True]      # two page groups
        whole = util.run_plan(eng, util.plan_whole(reqs))
        allocated = [g.pool.allocations for g in eng.manager.groups]
        mixed = util.run_plan(eng, plan)
        chunks = util.run_plan(eng, util.plan_chunks(reqs))
        eng.manager.check()
        assert not eng.manager.live()
        # the window group handed its pages out again and again
        win = [i for i, g in enumerate(eng.manager.groups) if g.window is not None][0]
        assert eng.manager.groups[win].pool.allocations - allocated[win] > eng.manager.groups[win].pool.num_pages

        # ---- the plain loop
        w = {k: v.double() for k, v in weights.items()}

        def keys_values(i, h):
            T = h.shape[0]
            pos = torch.arange(T)
            k = plain.rope_neox(plain.rms_norm((h @ w[f"l{i}.k"].T).reshape(T, Hkv, hd), w[f"l{i}.k_norm"], eps), pos, theta)
            return k, (h @ w[f"l{i}.v"].T).reshape(T, Hkv, hd)

        def attend(i, h, k, v, window):
            T = h.shape[0]
            pos = torch.arange(T)
            q = plain.rope_neox(plain.rms_norm((h @ w[f"l{i}.q"].T).reshape(T, H, hd), w[f"l{i}.q_norm"], eps), pos, theta)
            k, v = k.repeat_interleave(H // Hkv, 1), v.repeat_interleave(H // Hkv, 1)
            s = torch.einsum("thd,shd->hts", q, k) / math.sqrt(hd)
            a, b = torch.arange(T)[:, None], torch.arange(T)[None, :]
            seen = (b <= a) if window is None else ((b <= a) & (b > a - window))
            s = s.masked_fill(~seen, float("-inf"))
            return torch.einsum("hts,shd->thd", torch.softmax(s, -1), v).reshape(T, H * hd) @ w[f"l{i}.o"].T

        def ffn_of(i, x):
            return plain.swiglu(plain.rms_norm(x, w[f"l{i}.n2"], eps), w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])

        for rid, toks in reqs.items():
            x = w["emb"][toks]
            shared = None
            for i, reads in ((0, False), (1, False), (0, False), (2, True)):
                h = plain.rms_norm(x, w[f"l{i}.n1"], eps)
                if reads:
                    k, v = shared                                # block 1's keys and values, block 2's queries
                else:
                    k, v = keys_values(i, h)
                    if i == 1:
                        shared = (k, v)
                x = x + attend(i, h, k, v, W if i == 0 else None)
                x = x + ffn_of(i, x)
            want = plain.rms_norm(x, w["fn"], eps) @ w["emb"].T
            for got in (whole, mixed, chunks):
                util.assert_close(dtype, got[rid], want, rid)
    finally:
        registry.unregister_architecture("ToyOrderForCausalLM")


# ------------------------------------------- a position encoding that reads more than positions
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_encoding_over_two_axes_reads_what_comes_with_the_tokens(gpu, dtype):
    """A rotary encoding defined here whose angle comes from two numbers a token (a row and a column, as of the
    patches of an image), not from the token's place in the sequence: half of every head turns with the row, half
    with the column.  It declares the input it reads (TokenInput), steps bring it in StepEntry.inputs, the step's
    context hands it on; requests of a scheduler bring it as a function of the place.  Nothing in the framework's
    files knows of it.  Whole, in portions and mixed against a plain loop; greedy generation through LLM.generate
    (the generated tokens go on along a row) against the plain loop run again for every token."""
    from tuff_amd.config.base import ModelConfig
    from tuff_amd.engine.engine import Engine
    from tuff_amd.engine.llm import LLM
    from tuff_amd.models import registry
    from tuff_amd.models.decoder import DecoderModel
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.base import PositionEncoding, TokenInput, WeightDecl
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.ffn import SwiGLU
    from tuff_amd.parts.norm import RMSNorm
    from tuff_amd.sampling.params import SamplingParams
    from tuff_amd.weights.random_init import random_weights
    d, H, Hkv, hd, ffn, V, theta, eps, width = 48, 3, 1, 16, 80, 131, 100.0, 1e-5, 7

    def turn(x, pos, half):
        """x [T, heads, hd] with channels half*hd/2 .. of every head rotated by pos (half-split pairs), the rest as it is."""
        lo = half * hd // 2
        out = x.clone()
        out[..., lo:lo + hd // 2] = plain.rope_neox(x[..., lo:lo + hd // 2], pos, theta)
        return out

    class GridRotary(PositionEncoding):
        def token_inputs(self):
            return [TokenInput("grid", cols=2)]

        def apply_step(self, q, k, ctx):
            grid = ctx.inputs["grid"].long()
            for t, heads in ((q, H), (k, Hkv)):
                x = t.view(t.shape[0], heads, hd)
                for half in (0, 1):
                    lo = half * hd // 2
                    inv = theta ** (-2.0 * torch.arange(hd // 4, device=t.device, dtype=torch.float32) / (hd // 2))
                    ang = grid[:, half].float()[:, None] * inv
                    c, s_ = ang.cos()[:, None, :].to(t.dtype), ang.sin()[:, None, :].to(t.dtype)
                    a, b = x[..., lo:lo + hd // 4].clone(), x[..., lo + hd // 4:lo + hd // 2].clone()
                    x[..., lo:lo + hd // 4] = a * c - b * s_
                    x[..., lo + hd // 4:lo + hd // 2] = b * c + a * s_

    @dataclasses.dataclass
    class GridConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyGridForCausalLM"
        vocab_size: int

    def build(cfg):
        def block(i):
            names = {k: f"l{i}.{k}" for k in ("q", "k", "v", "o", "q_norm", "k_norm")}
            return PreNormBlock(RMSNorm(d, eps, f"l{i}.n1"),
                                AttentionMixer(d, H, Hkv, hd, names=names, qk_norm_eps=eps, position=GridRotary()),
                                RMSNorm(d, eps, f"l{i}.n2"),
                                SwiGLU(d, ffn, names={"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}))
        return DecoderModel(vocab_size=cfg.vocab_size, hidden_size=d, embedding=WeightDecl("emb", (cfg.vocab_size, d)),
                            blocks=[block(0), block(1)], final_norm=RMSNorm(d, eps, "fn"))

    def grid_of(rid, start, n):
        """Request rid's tokens lie row by row on a grid `width` wide that starts at row = its number."""
        first = int(rid[1:])
        place = torch.arange(start, start + n)
        return {"grid": torch.stack([first + place // width, place % width], 1).numpy()}

    registry.register_architecture("ToyGridForCausalLM", GridConfig, build)
    try:
        cfg = registry.config_from_dict({"architectures": ["ToyGridForCausalLM"], "vocab_size": V})
        model = registry.build_model(cfg)
        assert [t.name for t in model.token_inputs()] == ["grid"]
        stored = torch.float32 if dtype == "float32" else torch.bfloat16
        weights = random_weights(model.weight_decls(), 6, stored, "cpu", stored_dtype=stored)
        w = {k: v.double() for k, v in weights.items()}

        def logits_of(rid, toks):
            T = len(toks)
            g = torch.from_numpy(grid_of(rid, 0, T)["grid"])
            x = w["emb"][toks]
            for i in range(2):
                h = plain.rms_norm(x, w[f"l{i}.n1"], eps)
                q = plain.rms_norm((h @ w[f"l{i}.q"].T).reshape(T, H, hd), w[f"l{i}.q_norm"], eps)
                k = plain.rms_norm((h @ w[f"l{i}.k"].T).reshape(T, Hkv, hd), w[f"l{i}.k_norm"], eps)
                q, k = turn(turn(q, g[:, 0], 0), g[:, 1], 1), turn(turn(k, g[:, 0], 0), g[:, 1], 1)
                v = (h @ w[f"l{i}.v"].T).reshape(T, Hkv, hd)
                k, v = k.repeat_interleave(H // Hkv, 1), v.repeat_interleave(H // Hkv, 1)
                s_ = torch.einsum("thd,shd->hts", q, k) / math.sqrt(hd)
                s_ = s_.masked_fill(~torch.ones(T, T, dtype=torch.bool).tril(), float("-inf"))
                x = x + torch.einsum("hts,shd->thd", torch.softmax(s_, -1), v).reshape(T, H * hd) @ w[f"l{i}.o"].T
                x = x + plain.swiglu(plain.rms_norm(x, w[f"l{i}.n2"], eps), w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])
            return plain.rms_norm(x, w["fn"], eps) @ w["emb"].T

        reqs = {f"r{i}": util.rand_tokens(n, V, 50 + i) for i, n in enumerate([60, 33, 47, 20])}
        plan = util.plan_mixed(reqs, seed=5, decode_tail=10)
        eng = Engine(model, {k: v.to(gpu) for k, v in weights.items()}, dtype=dtype, page_size=16,
                     max_tokens=util.live_tokens_peak(plan))
        runs = [util.run_plan(eng, p, grid_of) for p in (util.plan_whole(reqs), plan, util.plan_chunks(reqs))]
        eng.manager.check()
        for rid, toks in reqs.items():
            want = logits_of(rid, toks)
            for got in runs:
                util.assert_close(dtype, got[rid], want, rid)
        # the coordinates matter: the same tokens along one long row give other logits
        flat = util.run_plan(eng, util.plan_whole({"r0": reqs["r0"]}),
                             lambda rid, start, n: {"grid": [[0, c] for c in range(start, start + n)]})["r0"]
        assert (flat.double() - logits_of("r0", reqs["r0"])).abs().max() > 1e-2
        # a step that leaves them out is refused by name, and the engine goes on
        eng.begin("x")
        with pytest.raises(ValueError, match="reads the input 'grid'"):
            eng.step([("x", [1, 2, 3], [2])])
        eng.end("x")
        if dtype == "float32":
            # through the scheduler: prompts in portions of 16 beside decoding requests, the inputs as a function of the place
            llm = LLM(engine=eng, max_num_seqs=3, max_batched_tokens=16, ctx_size=96)
            prompts = {f"r{i}": util.rand_tokens(n, V, 70 + i) for i, n in enumerate([21, 9, 30])}
            gens = llm.generate(list(prompts.values()), SamplingParams(temp=0.0, max_new_tokens=6),
                                inputs=[lambda start, n, rid=rid: grid_of(rid, start, n) for rid in prompts])
            for (rid, prompt), gen in zip(prompts.items(), gens):
                ids = list(prompt)
                for tok in gen.token_ids:
                    row = logits_of(rid, ids)[-1]
                    top = torch.topk(row, 2).values
                    if float(top[0] - top[1]) > 1e-3:
                        assert tok == int(row.argmax()), rid
                    ids.append(tok)
    finally:
        registry.unregister_architecture("ToyGridForCausalLM")


# --------------------------------------------------------------- a toy routed feed-forward
def test_toy_feed_forward_with_routing_beside_the_frameworks_parts(gpu):
    """A feed-forward defined here: a float32 router picks one of three small SwiGLU experts per
    token (the experts are the framework's own SwiGLU parts; the routing is a few torch calls).
    Layer 0 uses it, layer 1 the dense SwiGLU: feed-forwards differ layer by layer.  Because the
    choice is per token, cutting and batching change nothing."""
    from tuff_amd.config.base import ModelConfig
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models import registry
    from tuff_amd.models.decoder import DecoderModel
    from tuff_amd.parts.base import FEED_FORWARDS, FeedForward, WeightDecl
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.ffn import SwiGLU
    from tuff_amd.parts.norm import RMSNorm
    from tuff_amd.parts.shortconv import ShortConvMixer
    from tuff_amd.weights.random_init import random_weights
    d, F, E, V, K, eps = 48, 40, 3, 131, 3, 1e-5

    class RoutedSwiGLU(FeedForward):
        def __init__(self, d, F, n_experts, prefix):
            self.router = f"{prefix}.router"
            self.experts = [SwiGLU(d, F, names={k: f"{prefix}.e{e}.{k}" for k in ("gate", "up", "down")})
                            for e in range(n_experts)]
            self.d, self.E = d, n_experts

        def weight_decls(self):
            return [WeightDecl(self.router, (self.E, self.d))] + [x for e in self.experts for x in e.weight_decls()]

        def kernel_modules(self):
            return [m for e in self.experts for m in e.kernel_modules()]

        def bind(self, weights, rt):
            self.rt, self.w_router = rt, weights[self.router].float()
            for e in self.experts:
                e.bind(weights, rt)

        def forward(self, h, ctx, residual):
            choice = (h.float() @ self.w_router.T).argmax(-1)                 # router logits in float32
            for e, expert in enumerate(self.experts):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel():
                    part = torch.zeros(rows.numel(), self.d, dtype=torch.float32, device=h.device)
                    expert.forward(h[rows].contiguous(), ctx, part)
                    residual[rows] += part

    @dataclasses.dataclass
    class RoutedConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyRoutedForCausalLM"
        vocab_size: int

    def build(cfg):
        def mixer(i):
            return ShortConvMixer(d, K, names={"in_proj": f"l{i}.in", "conv": f"l{i}.conv", "out_proj": f"l{i}.out"})
        ffs = [FEED_FORWARDS.get("toy_routed")(d, F, E, "l0.moe"),
               SwiGLU(d, 2 * F, names={"gate": "l1.g", "up": "l1.u", "down": "l1.d"})]
        blocks = [PreNormBlock(RMSNorm(d, eps, f"l{i}.n1"), mixer(i), RMSNorm(d, eps, f"l{i}.n2"), ffs[i]) for i in range(2)]
        return DecoderModel(vocab_size=cfg.vocab_size, hidden_size=d, embedding=WeightDecl("emb", (cfg.vocab_size, d)),
                            blocks=blocks, final_norm=RMSNorm(d, eps, "fn"))

    FEED_FORWARDS.register("toy_routed", RoutedSwiGLU)
    registry.register_architecture("ToyRoutedForCausalLM", RoutedConfig, build)
    try:
        cfg = registry.config_from_dict({"architectures": ["ToyRoutedForCausalLM"], "vocab_size": V})
        model = registry.build_model(cfg)
        weights = random_weights(model.weight_decls(), 6, torch.float32, "cpu", stored_dtype=torch.float32)
        weights["l0.moe.router"] = weights["l0.moe.router"] * 40          # clear choices: no ties to argue about
        eng = Engine(model, {k: v.to(gpu) for k, v in weights.items()}, dtype="float32", max_tokens=256)
        reqs = {"a": util.rand_tokens(33, V, 1), "b": util.rand_tokens(20, V, 2), "c": util.rand_tokens(9, V, 3)}
        whole = util.run_plan(eng, util.plan_whole(reqs))
        mixed = util.run_plan(eng, util.plan_mixed(reqs, seed=2, decode_tail=5))
        w = {k: v.double() for k, v in weights.items()}
        used = set()
        for rid, toks in reqs.items():
            x = w["emb"][toks]
            for i in range(2):
                x = x + plain.short_conv(plain.rms_norm(x, w[f"l{i}.n1"], eps), w[f"l{i}.in"], w[f"l{i}.conv"], w[f"l{i}.out"])
                h = plain.rms_norm(x, w[f"l{i}.n2"], eps)
                if i == 0:
                    choice = (h @ w["l0.moe.router"].T).argmax(-1)
                    used |= set(choice.tolist())
                    y = torch.stack([plain.swiglu(h[t:t + 1], w[f"l0.moe.e{int(c)}.gate"], w[f"l0.moe.e{int(c)}.up"],
                                                  w[f"l0.moe.e{int(c)}.down"])[0] for t, c in enumerate(choice)])
                else:
                    y = plain.swiglu(h, w["l1.g"], w["l1.u"], w["l1.d"])
                x = x + y
            want = plain.rms_norm(x, w["fn"], eps) @ w["emb"].T
            util.assert_close_f32(whole[rid], want, rid)
            util.assert_close_f32(mixed[rid], want, rid)
        assert len(used) == E                                             # every expert was chosen by some token
    finally:
        registry.unregister_architecture("ToyRoutedForCausalLM")
        FEED_FORWARDS.unregister("toy_routed")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_biases_a_scaled_embedding_and_capped_logits(gpu, dtype):
    """What the reference's architecture has none of, declared by a toy one without a change to the
    framework: projections with a bias (a gated feed-forward defined here from two `Linear`s), embedding
    rows times sqrt(d), logits times a factor under a soft cap.  Whole and mixed plans against the
    formulas written out here."""
    from tuff_amd.config.base import ModelConfig
    from tuff_amd.engine.engine import Engine
    from tuff_amd.models import registry
    from tuff_amd.models.decoder import DecoderModel
    from tuff_amd.parts.base import FEED_FORWARDS, FeedForward, WeightDecl
    from tuff_amd.parts.block import PreNormBlock
    from tuff_amd.parts.linear import Linear
    from tuff_amd.parts.norm import RMSNorm
    from tuff_amd.parts.shortconv import ShortConvMixer
    from tuff_amd.weights.random_init import random_weights
    from tuff_amd.csrc import ops
    d, F, V, K, eps = 48, 40, 131, 3, 1e-5
    emb_scale, logit_scale, cap = math.sqrt(d), 0.5, 3.0

    class BiasedGatedFF(FeedForward):
        graph_safe = True

        def __init__(self, d, F, prefix):
            self.gate_up = Linear([f"{prefix}.g", f"{prefix}.u"], d, [F, F], swiglu_pair=True,
                                  bias=[f"{prefix}.gb", f"{prefix}.ub"])
            self.down = Linear(f"{prefix}.d", F, d, bias=f"{prefix}.db")
            self.F = F

        def weight_decls(self):
            return self.gate_up.weight_decls() + self.down.weight_decls()

        def kernel_modules(self):
            return ["elementwise"]

        def bind(self, weights, rt):
            self.rt = rt
            self.gate_up.bind(weights, rt)
            self.down.bind(weights, rt)

        def forward(self, h, ctx, residual):
            gu = self.gate_up.forward(h)
            act = self.rt.empty(h.shape[0], self.F, dtype=gu.dtype)
            ops.swiglu(gu, act)
            self.down.forward(act, accumulate_into=residual)

    @dataclasses.dataclass
    class BiasedConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyBiasedForCausalLM"
        vocab_size: int

    def build(cfg):
        blocks = [PreNormBlock(RMSNorm(d, eps, f"l{i}.n1"),
                               ShortConvMixer(d, K, names={"in_proj": f"l{i}.in", "conv": f"l{i}.conv", "out_proj": f"l{i}.out"}),
                               RMSNorm(d, eps, f"l{i}.n2"), FEED_FORWARDS.get("toy_biased")(d, F, f"l{i}.ff")) for i in range(2)]
        return DecoderModel(vocab_size=cfg.vocab_size, hidden_size=d, embedding=WeightDecl("emb", (cfg.vocab_size, d)),
                            blocks=blocks, final_norm=RMSNorm(d, eps, "fn"), embedding_scale=emb_scale,
                            logit_scale=logit_scale, logit_softcap=cap)

    FEED_FORWARDS.register("toy_biased", BiasedGatedFF)
    registry.register_architecture("ToyBiasedForCausalLM", BiasedConfig, build)
    try:
        cfg = registry.config_from_dict({"architectures": ["ToyBiasedForCausalLM"], "vocab_size": V})
        model = registry.build_model(cfg)
        stored = torch.float32 if dtype == "float32" else torch.bfloat16
        weights = random_weights(model.weight_decls(), 8, stored, "cpu", stored_dtype=stored)
        for k in list(weights):
            if k.endswith("b"):                                           # biases large enough to matter
                weights[k] = (weights[k].float() * 20).to(stored)
            elif ".ff." in k or k == "emb":
                weights[k] = (weights[k].float() * 6).to(stored)          # logits wide enough to reach the cap
        eng = Engine(model, {k: v.to(gpu) for k, v in weights.items()}, dtype=dtype, max_tokens=256)
        reqs = {"a": util.rand_tokens(33, V, 1), "b": util.rand_tokens(20, V, 2), "c": util.rand_tokens(9, V, 3)}
        whole = util.run_plan(eng, util.plan_whole(reqs))
        mixed = util.run_plan(eng, util.plan_mixed(reqs, seed=2, decode_tail=5))
        w = {k: v.double() for k, v in weights.items()}
        capped = 0
        for rid, toks in reqs.items():
            x = w["emb"][toks] * emb_scale
            for i in range(2):
                x = x + plain.short_conv(plain.rms_norm(x, w[f"l{i}.n1"], eps), w[f"l{i}.in"], w[f"l{i}.conv"], w[f"l{i}.out"])
                h = plain.rms_norm(x, w[f"l{i}.n2"], eps)
                g = h @ w[f"l{i}.ff.g"].T + w[f"l{i}.ff.gb"]
                u = h @ w[f"l{i}.ff.u"].T + w[f"l{i}.ff.ub"]
                x = x + (g / (1 + torch.exp(-g)) * u) @ w[f"l{i}.ff.d"].T + w[f"l{i}.ff.db"]
            raw = plain.rms_norm(x, w["fn"], eps) @ w["emb"].T * logit_scale
            want = cap * torch.tanh(raw / cap)
            capped += int((raw.abs() > cap).sum())
            for got in (whole[rid], mixed[rid]):
                if dtype == "float32":
                    util.assert_close_f32(got, want, rid)
                else:
                    util.assert_close_bf16(got, want, rid)
        assert capped > 50                                                # the cap does something here
    finally:
        registry.unregister_architecture("ToyBiasedForCausalLM")
        FEED_FORWARDS.unregister("toy_biased")
