"""LFM2 / LFM2.5 dense decoder put together from parts.

Every layer is a pre-norm block: operator_norm -> (short conv | attention) -> residual;
ffn_norm -> SwiGLU -> residual (src/lfm25_engine.c:365-419).  Attention layers norm q and k
per head with the model's eps and rotate them in the half-split form with theta = rope_theta
(src/lfm25_gpu.cu:420-485).  The final norm is `embedding_norm`; the head is the embedding when
tied (src/lfm25_model.c:123-131).

Checkpoint names follow the Hugging Face layout of the architecture; the names the reference
reads from GGUF (`blk.N.*`, src/lfm25_model.c:120-216) are accepted as aliases.
"""
from __future__ import annotations

from ..config.lfm2 import Lfm2Config
from ..parts.attention import AttentionMixer
from ..parts.base import WeightDecl
from ..parts.block import PreNormBlock
from ..parts.ffn import SwiGLU
from ..parts.norm import RMSNorm
from ..parts.rope import Rotary
from ..parts.shortconv import ShortConvMixer
from .decoder import DecoderModel


def build_lfm2(cfg: Lfm2Config) -> DecoderModel:
    d, eps = cfg.hidden_size, cfg.norm_eps
    blocks = []
    for i in range(cfg.num_hidden_layers):
        p, g = f"model.layers.{i}.", f"blk.{i}."
        norm1 = RMSNorm(d, eps, p + "operator_norm.weight", aliases=(g + "attn_norm.weight",))
        if cfg.is_conv(i):
            mixer = ShortConvMixer(
                d, cfg.conv_L_cache,
                names={"in_proj": p + "conv.in_proj.weight", "conv": p + "conv.conv.weight",
                       "out_proj": p + "conv.out_proj.weight"},
                aliases={"in_proj": (g + "shortconv.in_proj.weight",),
                         "conv": (g + "shortconv.conv.weight",),
                         "out_proj": (g + "shortconv.out_proj.weight",)})
        else:
            mixer = AttentionMixer(
                d, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                names={"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                       "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.out_proj.weight",
                       "q_norm": p + "self_attn.q_layernorm.weight",
                       "k_norm": p + "self_attn.k_layernorm.weight"},
                aliases={"q": (g + "attn_q.weight",), "k": (g + "attn_k.weight",),
                         "v": (g + "attn_v.weight",), "o": (g + "attn_output.weight",),
                         "q_norm": (g + "attn_q_norm.weight",), "k_norm": (g + "attn_k_norm.weight",)},
                qk_norm_eps=eps,
                position=Rotary(cfg.head_dim, cfg.rope_theta, table_positions=min(cfg.max_position_embeddings, 1 << 18)))
        norm2 = RMSNorm(d, eps, p + "ffn_norm.weight", aliases=(g + "ffn_norm.weight",))
        ffn = SwiGLU(d, cfg.ffn_dim,
                     names={"gate": p + "feed_forward.w1.weight", "up": p + "feed_forward.w3.weight",
                            "down": p + "feed_forward.w2.weight"},
                     aliases={"gate": (g + "ffn_gate.weight",), "up": (g + "ffn_up.weight",),
                              "down": (g + "ffn_down.weight",)})
        blocks.append(PreNormBlock(norm1, mixer, norm2, ffn))
    head = None if cfg.tie_word_embeddings else WeightDecl(
        "lm_head.weight", (cfg.vocab_size, d), "normal", aliases=("output.weight",))
    return DecoderModel(
        vocab_size=cfg.vocab_size, hidden_size=d,
        embedding=WeightDecl("model.embed_tokens.weight", (cfg.vocab_size, d), "normal",
                             aliases=("token_embd.weight",)),
        blocks=blocks,
        final_norm=RMSNorm(d, eps, "model.embedding_norm.weight",
                           aliases=("token_embd_norm.weight", "output_norm.weight")),
        head=head, max_positions=cfg.max_position_embeddings, eos_token_id=cfg.eos_token_id)
