"""Configuration of the LFM2 / LFM2.5 dense decoder (`Lfm2ForCausalLM`).

The reference reads the same quantities from GGUF keys (src/lfm25_model.c:73-117):
block_count, embedding_length, head_count, head_count_kv (per layer, 0 on conv
layers), shortconv.l_cache, layer_norm_rms_epsilon, rope.freq_base,
feed_forward_length (already adjusted), context_length.  Here they come from the
config.json keys of the architecture; the layer kinds come from `layer_types`
where the reference derives them from tensor presence (src/lfm25_model.c:153-186).
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Optional

from .base import ConfigError, ModelConfig

CONV = "conv"
FULL_ATTENTION = "full_attention"


@dataclasses.dataclass
class Lfm2Config(ModelConfig):
    architecture: ClassVar[str] = "Lfm2ForCausalLM"
    aliases: ClassVar[dict[str, str]] = {
        "tie_embedding": "tie_word_embeddings",
        "theta": "rope_theta",
        "num_heads": "num_attention_heads",
        "block_norm_eps": "norm_eps",
    }
    ignored: ClassVar[frozenset[str]] = ModelConfig.ignored | frozenset({
        "block_mlp_init_scale", "block_out_init_scale", "block_use_xavier_init",
        "conv_use_xavier_init",
    })

    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    block_ff_dim: int
    layer_types: Optional[list] = None          # "conv" | "full_attention" per layer
    full_attn_idxs: Optional[list] = None       # older spelling: indices of attention layers
    conv_L_cache: int = 3
    conv_bias: bool = False
    norm_eps: float = 1e-5
    rope_theta: float = 1000000.0
    max_position_embeddings: int = 128000
    tie_word_embeddings: bool = True
    block_auto_adjust_ff_dim: bool = False
    block_multiple_of: int = 256
    block_ffn_dim_multiplier: Optional[float] = None
    block_use_swiglu: bool = True
    block_dim: Optional[int] = None
    conv_dim: Optional[int] = None
    conv_dim_out: Optional[int] = None
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None
    pad_token_id: Optional[int] = None

    # ------------------------------------------------------------------ validation
    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "block_ff_dim", "block_multiple_of",
                     "max_position_embeddings"):
            self._int(name)
        self._int("conv_L_cache", minimum=2)
        for name in ("norm_eps", "rope_theta"):
            self._float(name)
        for name in ("conv_bias", "tie_word_embeddings", "block_auto_adjust_ff_dim",
                     "block_use_swiglu"):
            self._bool(name)
        if self.block_ffn_dim_multiplier is not None:
            self._float("block_ffn_dim_multiplier")
        L = self.num_hidden_layers
        if self.layer_types is None:
            if self.full_attn_idxs is None:
                raise ConfigError("Lfm2ForCausalLM: config.json lacks required key(s): layer_types")
            idx = list(self.full_attn_idxs)
            if any((not isinstance(i, int)) or i < 0 or i >= L for i in idx):
                raise ConfigError(f"full_attn_idxs {idx} must be layer indices in [0, {L})")
            self.layer_types = [FULL_ATTENTION if i in idx else CONV for i in range(L)]
        if not isinstance(self.layer_types, list) or len(self.layer_types) != L:
            raise ConfigError(f"layer_types must list {L} entries (num_hidden_layers), "
                              f"got {self.layer_types!r}")
        bad = sorted({t for t in self.layer_types if t not in (CONV, FULL_ATTENTION)})
        if bad:
            raise ConfigError(f"layer_types holds unknown kind(s) {bad}; "
                              f"known: '{CONV}', '{FULL_ATTENTION}'")
        self.full_attn_idxs = [i for i, t in enumerate(self.layer_types) if t == FULL_ATTENTION]
        d, H, Hkv = self.hidden_size, self.num_attention_heads, self.num_key_value_heads
        # src/lfm25_model.c:322-329: d divisible by heads, heads a multiple of kv heads
        if d % H != 0:
            raise ConfigError(f"hidden_size {d} is not divisible by num_attention_heads {H}")
        if H % Hkv != 0:
            raise ConfigError(f"num_attention_heads {H} is not a multiple of "
                              f"num_key_value_heads {Hkv}")
        if (d // H) % 2 != 0:
            raise ConfigError(f"head size {d // H} must be even for the half-split rotation")
        if self.conv_bias:
            # the reference binds no bias tensors for the short conv (src/lfm25_model.c:154-163)
            raise ConfigError("conv_bias=true is not supported: the short convolution has no bias")
        if not self.block_use_swiglu:
            raise ConfigError("block_use_swiglu=false is not supported: the feed-forward is SwiGLU")
        for name in ("block_dim", "conv_dim", "conv_dim_out"):
            v = getattr(self, name)
            if v is not None and v != d:
                raise ConfigError(f"{name} {v} differs from hidden_size {d}; not supported")
        for name in ("bos_token_id", "eos_token_id", "pad_token_id"):
            v = getattr(self, name)
            if v is not None and (isinstance(v, bool) or not isinstance(v, int)):
                raise ConfigError(f"{name} must be an integer or null, got {v!r}")

    # --------------------------------------------------------------------- derived
    @property
    def head_dim(self) -> int:
        # src/lfm25_model.c:90: head size is hidden / heads, not a free key
        return self.hidden_size // self.num_attention_heads

    @property
    def ffn_dim(self) -> int:
        """Feed-forward width.  With auto-adjust: two thirds, optional multiplier,
        rounded up to block_multiple_of (384 -> 256 at multiple 64; 12288 -> 8192)."""
        f = self.block_ff_dim
        if self.block_auto_adjust_ff_dim:
            f = int(2 * f / 3)
            if self.block_ffn_dim_multiplier is not None:
                f = int(self.block_ffn_dim_multiplier * f)
            m = self.block_multiple_of
            f = m * ((f + m - 1) // m)
        return f

    def is_conv(self, layer: int) -> bool:
        return self.layer_types[layer] == CONV

    def to_dict(self) -> dict[str, Any]:
        out = super().to_dict()
        out["model_type"] = "lfm2"
        for k in ("block_dim", "conv_dim", "conv_dim_out", "block_ffn_dim_multiplier",
                  "bos_token_id", "eos_token_id", "pad_token_id"):
            if out.get(k) is None:
                out.pop(k, None)
        return out
