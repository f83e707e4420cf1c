"""Configuration and registry (CPU)."""
import copy
import json
import os

import pytest

import util
from tuff_amd.config.base import ConfigError
from tuff_amd.config.lfm2 import Lfm2Config
from tuff_amd.models import registry


def cfg_of(raw):
    return registry.config_from_dict(raw)


def test_tiny_configs_parse_and_differ_in_every_size():
    a, b, c = (cfg_of(util.CONFIGS[k][0]) for k in "ABC")
    for name in ("num_hidden_layers", "hidden_size", "vocab_size", "conv_L_cache", "norm_eps", "rope_theta",
                 "head_dim", "ffn_dim", "num_key_value_heads", "max_position_embeddings"):
        vals = {getattr(x, name) for x in (a, b, c)}
        assert len(vals) == 3, name
    assert a.tie_word_embeddings and not b.tie_word_embeddings
    assert (a.head_dim, b.head_dim, c.head_dim) == (16, 24, 80)
    assert b.layer_types[0] == b.layer_types[-1] == "full_attention" and a.layer_types[0] == "conv"


@pytest.mark.parametrize("ff,mult_of,want", [(384, 64, 256), (12288, 256, 8192), (16128, 256, 10752), (10368, 256, 6912)])
def test_ffn_width_auto_adjust(ff, mult_of, want):
    raw = dict(util.TINY_B, block_ff_dim=ff, block_multiple_of=mult_of, block_auto_adjust_ff_dim=True)
    assert cfg_of(raw).ffn_dim == want
    raw["block_auto_adjust_ff_dim"] = False
    assert cfg_of(raw).ffn_dim == ff
    from plain.lfm2_plain import ff_dim
    raw["block_auto_adjust_ff_dim"] = True
    assert ff_dim(raw) == want


def test_ffn_multiplier():
    raw = dict(util.TINY_B, block_ff_dim=384, block_multiple_of=32, block_auto_adjust_ff_dim=True,
               block_ffn_dim_multiplier=1.5)
    assert cfg_of(raw).ffn_dim == 384                       # int(1.5 * 256) = 384


def test_full_attn_idxs_is_the_older_spelling_of_layer_types():
    raw = copy.deepcopy(util.TINY_A)
    del raw["layer_types"]
    raw["full_attn_idxs"] = [2]
    assert cfg_of(raw).layer_types == util.TINY_A["layer_types"]
    raw["full_attn_idxs"] = [4]
    with pytest.raises(ConfigError, match="full_attn_idxs"):
        cfg_of(raw)


def test_aliases_and_ignored_keys():
    raw = dict(util.TINY_A, tie_embedding=False, theta=123.0, model_type="lfm2", torch_dtype="bfloat16", some_new_key=1)
    del raw["tie_word_embeddings"], raw["rope_theta"]
    cfg = cfg_of(raw)
    assert cfg.tie_word_embeddings is False and cfg.rope_theta == 123.0
    assert cfg.unknown_keys == ["some_new_key"]


@pytest.mark.parametrize("change,msg", [
    ({"hidden_size": None}, "hidden_size"),
    ({"layer_types": ["conv"]}, "layer_types must list 4"),
    ({"layer_types": ["conv", "conv", "mamba", "conv"]}, "unknown kind"),
    ({"num_attention_heads": 5}, "not divisible"),
    ({"num_key_value_heads": 3}, "not a multiple"),
    ({"conv_bias": True}, "conv_bias"),
    ({"conv_L_cache": 1}, "conv_L_cache"),
    ({"norm_eps": 0}, "norm_eps"),
    ({"norm_eps": "1e-5"}, "norm_eps"),
    ({"vocab_size": 3.5}, "vocab_size"),
    ({"tie_word_embeddings": 1}, "tie_word_embeddings"),
    ({"block_use_swiglu": False}, "block_use_swiglu"),
    ({"conv_dim": 128}, "conv_dim"),
    ({"hidden_size": 68, "num_attention_heads": 4}, "must be even"),
])
def test_bad_configs_are_refused_with_the_key_named(change, msg):
    raw = dict(util.TINY_A)
    for k, v in change.items():
        if v is None:
            raw.pop(k)
        else:
            raw[k] = v
    with pytest.raises(ConfigError, match=msg):
        cfg_of(raw)


def test_missing_keys_are_listed_together():
    raw = dict(util.TINY_A)
    del raw["vocab_size"], raw["block_ff_dim"]
    with pytest.raises(ConfigError, match="block_ff_dim, vocab_size"):
        cfg_of(raw)


def test_registry():
    assert "Lfm2ForCausalLM" in registry.architectures()
    with pytest.raises(ConfigError, match="unknown architecture 'NopeForCausalLM'"):
        cfg_of({"architectures": ["NopeForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        cfg_of({"hidden_size": 4})
    with pytest.raises(ValueError, match="already registered"):
        registry.register_architecture("Lfm2ForCausalLM", Lfm2Config, lambda c: None)


def test_round_trip_through_a_folder(tmp_path):
    cfg = cfg_of(util.TINY_B)
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg.to_dict(), f)
    again = registry.load_config(str(tmp_path))
    assert again == cfg and type(again) is Lfm2Config
    with pytest.raises(ConfigError, match="no config.json"):
        registry.load_config(str(tmp_path / "nope"))
    (tmp_path / "bad").mkdir()
    (tmp_path / "bad" / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        registry.load_config(str(tmp_path / "bad"))


def test_model_is_built_layer_by_layer_from_the_configuration():
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.base import FixedState, PagedKV
    from tuff_amd.parts.shortconv import ShortConvMixer
    cfg = cfg_of(util.TINY_B)
    model = registry.build_model(cfg)
    kinds = [type(b.mixer) for b in model.blocks]
    assert kinds == [AttentionMixer, ShortConvMixer, ShortConvMixer, AttentionMixer, ShortConvMixer, AttentionMixer]
    assert model.cache_specs[0] == PagedKV(1, 24, None) and model.cache_specs[1] == FixedState((3, 96))
    assert model.head_decl is not None and registry.build_model(cfg_of(util.TINY_A)).head_decl is None
    # parameter count of the benchmark shape (10 conv + 6 attention layers, tied head)
    import bench
    big = registry.build_model(bench.shape_config(16))
    assert big.num_parameters() == 1170340608
    assert bench.matmul_params(big) == 10 * 16777216 + 6 * 10485760 + 16 * 50331648


def test_run_order_is_data():
    from tuff_amd.models.decoder import DecoderModel, LayerRun
    cfg = cfg_of(util.TINY_B)
    base = registry.build_model(cfg)
    kw = dict(vocab_size=base.vocab_size, hidden_size=base.hidden_size, embedding=base.embedding_decl,
              blocks=base.blocks, final_norm=base.final_norm, head=base.head_decl)
    twice = DecoderModel(schedule=[LayerRun(0), LayerRun(1), LayerRun(0), LayerRun(3)], **kw)
    assert [r.cache for r in twice.schedule] == [0, 1, 2, 3] and len(twice.cache_specs) == 4
    shared = DecoderModel(schedule=[LayerRun(0, cache=7), LayerRun(3, cache=7, writes=False)], **kw)
    assert list(shared.cache_specs) == [7]
    with pytest.raises(ValueError, match="before any run writes"):
        DecoderModel(schedule=[LayerRun(0, cache=1, writes=False)], **kw)
    with pytest.raises(ValueError, match="two writers"):
        DecoderModel(schedule=[LayerRun(0, cache=1), LayerRun(3, cache=1)], **kw)
    with pytest.raises(ValueError, match="cannot be shared"):
        DecoderModel(schedule=[LayerRun(1, cache=1), LayerRun(2, cache=1, writes=False)], **kw)


def test_a_mixer_may_declare_several_cache_entries():
    """cache_spec() returning a tuple: the run's entries are (cache, 0), (cache, 1), ...; sharing
    such a run's paged entries works like sharing one, a fixed-size state among them forbids it."""
    from tuff_amd.models.decoder import DecoderModel, LayerRun
    from tuff_amd.parts.base import FixedState, Mixer, PagedKV
    from tuff_amd.parts.block import PreNormBlock

    class Keeps(Mixer):
        def __init__(self, *specs):
            self.specs = specs

        def cache_spec(self):
            return self.specs

    base = registry.build_model(cfg_of(util.TINY_B))
    n1 = base.blocks[0].norm1
    kv_and_state = PreNormBlock(n1, Keeps(PagedKV(2, 8, 16), FixedState((5,), "bfloat16")))
    two_kv = PreNormBlock(n1, Keeps(PagedKV(2, 8), PagedKV(1, 4, 16)))
    nothing = PreNormBlock(n1, Keeps())
    kw = dict(vocab_size=base.vocab_size, hidden_size=base.hidden_size, embedding=base.embedding_decl,
              final_norm=base.final_norm, head=base.head_decl)
    m = DecoderModel(blocks=[kv_and_state, base.blocks[1], two_kv, nothing], **kw)
    assert m.cache_specs == {(0, 0): PagedKV(2, 8, 16), (0, 1): FixedState((5,), "bfloat16"), 1: FixedState((3, 96)),
                             (2, 0): PagedKV(2, 8), (2, 1): PagedKV(1, 4, 16)}
    views = {e: f"view of {e}" for e in m.cache_specs}
    assert m._views_of(0, views) == ("view of (0, 0)", "view of (0, 1)") and m._views_of(1, views) == "view of 1"
    assert m._views_of(3, views) == ()
    from tuff_amd.cache.manager import CacheLayout
    lay = CacheLayout.from_specs(m.cache_specs)
    assert lay.group_windows == [16, None] and lay.group_of_entry == {(0, 0): 0, (2, 0): 1, (2, 1): 0}
    assert lay.state_bytes_per_request() == 5 * 2 + 3 * 96 * 4
    shared = DecoderModel(blocks=[two_kv], schedule=[LayerRun(0, cache=4), LayerRun(0, cache=4, writes=False)], **kw)
    assert list(shared.cache_specs) == [(4, 0), (4, 1)]
    with pytest.raises(ValueError, match="cannot be shared"):
        DecoderModel(blocks=[kv_and_state], schedule=[LayerRun(0, cache=4), LayerRun(0, cache=4, writes=False)], **kw)
