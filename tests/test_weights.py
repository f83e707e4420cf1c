"""Weights: the safetensors container, loading by name, errors, the random-weights folder (CPU)."""
import json
import os

import pytest
import torch

import util
from tuff_amd.models import registry
from tuff_amd.weights import loader, random_init
from tuff_amd.weights.safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors


def model_and_decls(name):
    cfg = registry.config_from_dict(util.CONFIGS[name][0])
    model = registry.build_model(cfg)
    return cfg, model, model.weight_decls()


def test_container_agrees_with_the_safetensors_library(tmp_path):
    from safetensors import safe_open
    from safetensors.torch import save_file
    tensors = {"a": torch.randn(3, 5).to(torch.bfloat16), "b.c": torch.arange(7, dtype=torch.int32),
               "d": torch.randn(2, 1, 4), "e": torch.zeros(0, 3)}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()], lambda n: tensors[n])
    with safe_open(ours, framework="pt") as f:
        assert sorted(f.keys()) == sorted(tensors)
        for k, v in tensors.items():
            assert torch.equal(f.get_tensor(k), v)
    theirs = str(tmp_path / "theirs.safetensors")
    save_file(tensors, theirs)
    st = SafetensorsFile(theirs)
    for k, v in tensors.items():
        assert st.shape(k) == tuple(v.shape) and st.dtype(k) == v.dtype
        assert torch.equal(st.read(k), v)


def test_broken_files_are_refused(tmp_path):
    p = tmp_path / "x.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(p))
    p.write_bytes((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="does not match"):
        SafetensorsFile(str(p))


def test_random_folder_loads_back_and_is_reproducible(tmp_path):
    cfg, model, decls = model_and_decls("B")
    a = random_init.write_random_model(cfg, str(tmp_path / "a"), seed=1)
    b = random_init.write_random_model(cfg, str(tmp_path / "b"), seed=1)
    c = random_init.write_random_model(cfg, str(tmp_path / "c"), seed=2)
    assert registry.load_config(a) == cfg
    wa = loader.load_weights(a, decls, torch.bfloat16, "cpu")
    wb = loader.load_weights(b, decls, torch.bfloat16, "cpu")
    wc = loader.load_weights(c, decls, torch.bfloat16, "cpu")
    assert set(wa) == {d.name for d in decls}
    for d in decls:
        assert wa[d.name].dtype == torch.bfloat16 and tuple(wa[d.name].shape) == tuple(d.shape)
        assert torch.equal(wa[d.name], wb[d.name])
    assert not torch.equal(wa["lm_head.weight"], wc["lm_head.weight"])
    # matrices N(0, 0.02), norm weights 1 + N(0, 0.01)
    big = wa["model.embed_tokens.weight"].float()
    assert abs(float(big.std()) - 0.02) < 0.001 and abs(float(big.mean())) < 0.001
    nw = torch.cat([wa[d.name].float() for d in decls if d.init == "norm"])
    assert abs(float(nw.mean()) - 1.0) < 0.005 and 0.005 < float(nw.std()) < 0.015
    # a tensor's values do not depend on the other tensors: same name, same seed, other model
    cfg2, _, decls2 = model_and_decls("A")
    d_b = next(d for d in decls if d.name == "model.layers.1.ffn_norm.weight")
    t1 = random_init.random_tensor(d_b, 1, torch.float32)
    t2 = random_init.random_tensor(d_b, 1, torch.float32)
    assert torch.equal(t1, t2)


def test_the_generator_is_the_specified_one(monkeypatch):
    """Every element against the numpy restatement of the generator's text (tests/plain/random_plain.py, which
    shares no code with it): the float64 deviates bit for bit, the float32 values, the bfloat16 bits; the same
    whether a tensor is made whole or in pieces; and against the library's ln, cos and root to 1e-14."""
    import math
    import numpy as np
    from plain import random_plain
    from tuff_amd.parts.base import WeightDecl
    name, seed, n = "model.layers.3.feed_forward.w1.weight", 5, 70001
    z = random_init.normal_deviates(random_init.tensor_key(seed, name), 0, n).numpy()
    zp = random_plain.deviates(seed, name, n)
    assert np.array_equal(z.view(np.uint64), zp.view(np.uint64))
    # against the formula with the library's functions, from the text's integers
    key, G = random_init.tensor_key(seed, name), random_init.GOLDEN
    for i in (0, 1, 2, 999, 70000):
        a, b = random_init._mix_int(key + (2 * i + 1) * G), random_init._mix_int(key + (2 * i + 2) * G)
        u1, u2 = ((a >> 11) + 1) * 2.0 ** -53, (b >> 11) * 2.0 ** -53
        assert abs(z[i] - math.sqrt(-2 * math.log(u1)) * math.cos(2 * math.pi * u2)) < 1e-14
    # the extremes of the uniform draws: nothing non-finite, the root of zero is harmless
    assert abs(z.mean()) < 0.02 and abs(z.std() - 1) < 0.01 and abs((z ** 4).mean() - 3) < 0.15 and np.abs(z).max() > 3.5
    for init, shape in (("normal", (37, 53)), ("norm", (97,))):
        d = WeightDecl("some.weight", shape, init)
        want32 = random_plain.tensor_f32(9, "some.weight", shape, init)
        assert np.array_equal(random_init.random_tensor(d, 9, torch.float32).numpy().view(np.uint32), want32.view(np.uint32))
        got16 = random_init.random_tensor(d, 9, torch.bfloat16)
        assert np.array_equal(got16.view(torch.int16).numpy().view(np.uint16), random_plain.to_bfloat16_bits(want32))
        monkeypatch.setitem(random_init.CHUNK, "cpu", 11)             # in pieces of 11 elements: the same tensor
        assert torch.equal(random_init.random_tensor(d, 9, torch.bfloat16), got16)
        monkeypatch.setitem(random_init.CHUNK, "cpu", 1 << 21)
    # another seed, another name: other values
    d1, d2 = WeightDecl("a.weight", (64,), "normal"), WeightDecl("b.weight", (64,), "normal")
    assert not torch.equal(random_init.random_tensor(d1, 1, torch.float32), random_init.random_tensor(d2, 1, torch.float32))
    assert not torch.equal(random_init.random_tensor(d1, 1, torch.float32), random_init.random_tensor(d1, 2, torch.float32))


@pytest.mark.parametrize("stored", [torch.bfloat16, torch.float32])
def test_a_seed_is_one_model_whichever_entry_point_makes_it(tmp_path, stored):
    """random_weights() (what Engine.from_config and `tuff --random` use) and write_random_model() read back
    (what the C interface's tuff_model_write_random and the tests' folders use): the same bits."""
    cfg, model, decls = model_and_decls("B")
    folder = random_init.write_random_model(cfg, str(tmp_path / "m"), seed=4, dtype=stored, device="cpu")
    for run in (torch.bfloat16, torch.float32):
        made = random_init.random_weights(decls, 4, run, "cpu", stored_dtype=stored)
        read = loader.load_weights(folder, decls, run, "cpu")
        assert set(made) == set(read)
        for k in made:
            assert made[k].dtype == read[k].dtype and torch.equal(made[k], read[k]), k


def test_a_checkpoint_in_several_files(tmp_path):
    """model.safetensors.index.json names the file of every tensor: the same weights as from one file."""
    cfg, model, decls = model_and_decls("A")
    folder = random_init.write_random_model(cfg, str(tmp_path / "m"), seed=0)
    whole = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    st = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    names = st.names()
    parts = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    for fn, ns in parts.items():
        write_safetensors(os.path.join(folder, fn), [(n, st.shape(n), st.dtype(n)) for n in ns], st.read)
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": {n: fn for fn, ns in parts.items() for n in ns}}, f)
    os.unlink(os.path.join(folder, "model.safetensors"))
    sharded = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    assert all(torch.equal(whole[k], sharded[k]) for k in whole)
    # an index that names a tensor its file does not hold, or a file outside the folder
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {n: "model-00001-of-00002.safetensors" for n in names}}, f)
    with pytest.raises(loader.WeightsError):
        loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {names[0]: "../x.safetensors"}}, f)
    with pytest.raises(loader.WeightsError):
        loader.load_weights(folder, decls, torch.bfloat16, "cpu")


def test_tensors_the_model_does_not_know_are_a_warning_listed_once(tmp_path):
    cfg, model, decls = model_and_decls("A")
    folder = random_init.write_random_model(cfg, str(tmp_path / "m"), seed=0)
    before = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    _rewrite(folder, lambda t: t.update({"model.layers.9.extra.weight": torch.zeros(2), "rotary.inv_freq": torch.zeros(8)}))
    with pytest.warns(loader.UnexpectedTensorsWarning) as rec:
        after = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    assert len(rec) == 1 and rec[0].message.names == ["model.layers.9.extra.weight", "rotary.inv_freq"]
    assert set(after) == set(before) and all(torch.equal(before[k], after[k]) for k in before)
    with pytest.raises(loader.WeightsError, match=r"unexpected tensors \(2\)"):
        loader.load_weights(folder, decls, torch.bfloat16, "cpu", strict=True)


def test_types_are_kept_as_stored(tmp_path):
    cfg, model, decls = model_and_decls("A")
    folder = random_init.write_random_model(cfg, str(tmp_path / "f32"), seed=0, dtype=torch.float32)
    w = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    assert all(t.dtype == torch.float32 for t in w.values())          # stored in 32-bit: stays so
    folder = random_init.write_random_model(cfg, str(tmp_path / "bf16"), seed=0)
    w16 = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    w32 = loader.load_weights(folder, decls, torch.float32, "cpu")
    assert all(t.dtype == torch.bfloat16 for t in w16.values())
    assert all(t.dtype == torch.float32 for t in w32.values())
    assert all(torch.equal(w16[k].float(), w32[k]) for k in w16)      # the up-cast is exact
    assert loader.target_dtype(torch.int64, torch.bfloat16) == torch.int32
    assert loader.target_dtype(torch.float16, torch.bfloat16) == torch.bfloat16


def _rewrite(folder, change):
    """Rewrites model.safetensors with `change(dict name -> tensor)` applied."""
    st = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {n: st.read(n) for n in st.names()}
    change(tensors)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()], lambda n: tensors[n])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg, model, decls = model_and_decls("A")
    folder = random_init.write_random_model(cfg, str(tmp_path / "m"), seed=0)

    def change(t):
        del t["model.layers.2.self_attn.q_layernorm.weight"]
        del t["model.layers.0.conv.conv.weight"]
        t["model.layers.9.extra.weight"] = torch.zeros(2)
        t["model.layers.1.feed_forward.w2.weight"] = torch.zeros(64, 100, dtype=torch.bfloat16)
        t["model.embedding_norm.weight"] = torch.zeros(63, dtype=torch.bfloat16)
    _rewrite(folder, change)
    with pytest.raises(loader.WeightsError) as e:
        loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    err = e.value
    assert sorted(err.missing) == ["model.layers.0.conv.conv.weight", "model.layers.2.self_attn.q_layernorm.weight"]
    assert err.unexpected == ["model.layers.9.extra.weight"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["model.embedding_norm.weight", "model.layers.1.feed_forward.w2.weight"]
    text = str(err)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "has shape [64, 100], expected [64, 192]",
                  "model.layers.2.self_attn.q_layernorm.weight"):
        assert piece in text


def test_tied_and_untied_heads(tmp_path):
    cfg, model, decls = model_and_decls("A")                                 # tied
    folder = random_init.write_random_model(cfg, str(tmp_path / "tied"), seed=0)
    _rewrite(folder, lambda t: t.update({"lm_head.weight": torch.zeros(512, 64, dtype=torch.bfloat16)}))
    with pytest.raises(loader.WeightsError, match="unexpected tensors"):
        loader.load_weights(folder, decls, torch.bfloat16, "cpu", strict=True)
    with pytest.warns(loader.UnexpectedTensorsWarning, match="lm_head.weight"):    # a tied model reads no head of its own
        w = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    assert "lm_head.weight" not in w
    cfg, model, decls = model_and_decls("B")                                 # untied
    folder = random_init.write_random_model(cfg, str(tmp_path / "untied"), seed=0)
    _rewrite(folder, lambda t: t.pop("lm_head.weight"))
    with pytest.raises(loader.WeightsError, match="missing tensors.*lm_head.weight"):
        loader.load_weights(folder, decls, torch.bfloat16, "cpu")


def test_reference_style_names_and_conv_shape_are_accepted(tmp_path):
    """The names the reference reads from GGUF (src/lfm25_model.c:120-216) load as aliases, and the
    conv taps may come as [d, 1, K]."""
    cfg, model, decls = model_and_decls("A")
    folder = random_init.write_random_model(cfg, str(tmp_path / "m"), seed=0)
    before = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    rename = {"model.embed_tokens.weight": "token_embd.weight", "model.embedding_norm.weight": "token_embd_norm.weight"}
    for i in range(4):
        p, g = f"model.layers.{i}.", f"blk.{i}."
        rename.update({p + "operator_norm.weight": g + "attn_norm.weight", p + "ffn_norm.weight": g + "ffn_norm.weight",
                       p + "feed_forward.w1.weight": g + "ffn_gate.weight", p + "feed_forward.w3.weight": g + "ffn_up.weight",
                       p + "feed_forward.w2.weight": g + "ffn_down.weight",
                       p + "conv.in_proj.weight": g + "shortconv.in_proj.weight", p + "conv.conv.weight": g + "shortconv.conv.weight",
                       p + "conv.out_proj.weight": g + "shortconv.out_proj.weight",
                       p + "self_attn.q_proj.weight": g + "attn_q.weight", p + "self_attn.k_proj.weight": g + "attn_k.weight",
                       p + "self_attn.v_proj.weight": g + "attn_v.weight", p + "self_attn.out_proj.weight": g + "attn_output.weight",
                       p + "self_attn.q_layernorm.weight": g + "attn_q_norm.weight", p + "self_attn.k_layernorm.weight": g + "attn_k_norm.weight"})

    def change(t):
        for old, new in rename.items():
            if old in t:
                t[new] = t.pop(old)
        t["blk.0.shortconv.conv.weight"] = t["blk.0.shortconv.conv.weight"].reshape(64, 1, 3)
    _rewrite(folder, change)
    after = loader.load_weights(folder, decls, torch.bfloat16, "cpu")
    assert all(torch.equal(before[k], after[k]) for k in before)


def test_missing_file():
    _, _, decls = model_and_decls("A")
    with pytest.raises(loader.WeightsError):
        loader.load_weights("/nonexistent/folder", decls, torch.bfloat16, "cpu")


def test_tile_major_weight_layout():
    """The order the matrix kernels stream a bfloat16 weight in: piece l of block (t, b) is row
    16 t + l % 16, k 32 b + 8 (l // 16) .. + 7; zero outside the matrix; rows() gives it back."""
    from tuff_amd.csrc import ops
    for N, K in ((50, 40), (16, 32), (33, 96)):
        w = torch.randn(N, K).to(torch.bfloat16)
        t = ops.tile_weight(w)
        assert t.shape == (N, K) and t.blocks.shape == (-(-N // 16), -(-K // 32), 64, 8)
        for tile, blk, piece in ((0, 0, 0), (t.blocks.shape[0] - 1, t.blocks.shape[1] - 1, 63), (1 % t.blocks.shape[0], 0, 37)):
            row, k = 16 * tile + piece % 16, 32 * blk + 8 * (piece // 16)
            want = torch.zeros(8, dtype=torch.bfloat16)
            if row < N:
                n = max(0, min(8, K - k))
                want[:n] = w[row, k:k + n]
            assert torch.equal(t.blocks[tile, blk, piece], want), (N, K, tile, blk, piece)
        assert torch.equal(t.rows(), w)
