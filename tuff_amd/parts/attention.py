"""Grouped-query attention mixer over the paged cache.

q = W_q h, k = W_k h, v = W_v h; optional per-head RMSNorm of q and k with a shared [hd]
weight; optional position encoding; k (normed, encoded) and v (as projected) go to the cache
at the token's slot; every token attends to the cached keys of its request up to its own
position (within `window` if given); query head i reads kv head i // (H / Hkv); scores are
scaled by 1/sqrt(hd); o = W_o concat(heads).
Reference: src/lfm25_engine.c:386-405, src/lfm25_gpu.cu:420-485, :506-558.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from ..csrc import ops
from .base import MIXERS, Mixer, PagedKV, PositionEncoding, Runtime, WeightDecl
from .linear import Linear


@MIXERS.register("attention")
class AttentionMixer(Mixer):
    accepts_pending_norm = True
    adds_once_through_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, *,
                 names: dict[str, str], qk_norm_eps: Optional[float] = None,
                 position: Optional[PositionEncoding] = None, window: Optional[int] = None,
                 scale: Optional[float] = None, aliases: Optional[dict[str, tuple]] = None):
        """names: checkpoint names of 'q', 'k', 'v', 'o' and, with qk_norm_eps, 'q_norm', 'k_norm'."""
        if num_heads % num_kv_heads:
            raise ValueError(f"heads {num_heads} must be a multiple of kv heads {num_kv_heads}")
        if head_dim > 256:
            raise ValueError(f"head size {head_dim} above 256 is not supported by the attention kernels")
        self.d, self.H, self.Hkv, self.hd = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.position, self.window = position, (int(window) if window else None)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.hd)
        self.names = dict(names)
        al = aliases or {}
        self.qkv = Linear([names["q"], names["k"], names["v"]], self.d,
                          [self.H * self.hd, self.Hkv * self.hd, self.Hkv * self.hd],
                          aliases=[al.get("q", ()), al.get("k", ()), al.get("v", ())])
        self.out = Linear(names["o"], self.H * self.hd, self.d, aliases=[al.get("o", ())])
        self._al = al
        self.q_norm_w = self.k_norm_w = None

    @property
    def graph_safe(self):
        return self.position is None or self.position.graph_safe

    @property
    def records_portions(self):
        return self.graph_safe

    def weight_decls(self):
        decls = self.qkv.weight_decls() + self.out.weight_decls()
        if self.eps is not None:
            decls += [WeightDecl(self.names["q_norm"], (self.hd,), "norm", aliases=self._al.get("q_norm", ())),
                      WeightDecl(self.names["k_norm"], (self.hd,), "norm", aliases=self._al.get("k_norm", ()))]
        if self.position is not None:
            decls += self.position.weight_decls()
        return decls

    def kernel_modules(self):
        mods = ["rope_kv", "attention", "attention_mfma", "attention_prefill"]
        if self.position is not None:
            mods += self.position.kernel_modules()
        return mods

    def token_inputs(self):
        return self.position.token_inputs() if self.position is not None else []

    def cache_spec(self):
        return PagedKV(self.Hkv, self.hd, self.window)

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.qkv.bind(weights, rt)
        self.out.bind(weights, rt)
        if self.eps is not None:
            self.q_norm_w = weights[self.names["q_norm"]]
            self.k_norm_w = weights[self.names["k_norm"]]
            if self.q_norm_w.dtype != self.k_norm_w.dtype:
                self.q_norm_w = self.q_norm_w.float()
                self.k_norm_w = self.k_norm_w.float()
        if self.position is not None:
            self.position.bind(weights, rt)

    def forward(self, h, ctx, cache, residual, write_cache: bool = True, next_norm=None) -> None:
        T = h.shape[0]
        H, Hkv, hd = self.H, self.Hkv, self.hd
        qkv = self.qkv.forward(h)
        q = self.rt.empty(T, H * hd)
        o = self.rt.empty(T, H * hd)
        norm = dict(eps=self.eps or 0.0, q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w)
        tables = self.position.rotary_tables() if self.position is not None else None
        fused = self.position is None or tables is not None
        # a position encoding of its own: norm, then its apply(), then the cache write
        k = None if fused else self.rt.empty(T, Hkv * hd)

        one_kernel = (fused and tables is not None and ctx.max_q_len == 1 and ops.attention_decode_fused_supported(
            qkv.dtype, H, Hkv, hd, cache.page_size, tables[1], tables[2]))

        def over_the_cache(ctx):
            """What depends on where the step's tokens lie: positions, cache slots, block tables."""
            g = ctx.groups[cache.group]
            if one_kernel:
                # single tokens, heads of 64: norm, rotation, cache write and attention in one kernel
                ops.attention_decode_fused(qkv, cache.k, cache.v, o, block_table=g.block_table, req_info=ctx.req_info,
                                           positions=ctx.positions, inv_freq=tables[0], H=H, Hkv=Hkv,
                                           page_size=cache.page_size, max_ctx_len=ctx.max_ctx_len,
                                           slot_mapping=g.slot_mapping if write_cache else None,
                                           q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, eps=self.eps or 0.0,
                                           window=self.window or 0, scale=self.scale,
                                           angles=getattr(self.position, "angle_table", lambda: None)())
                return
            if fused:
                rot = {}
                if tables is not None:
                    rot = dict(inv_freq=tables[0], rotary_dim=tables[1], interleaved=tables[2],
                               angles=getattr(self.position, "angle_table", lambda: None)())
                wr = dict(k_cache=cache.k, v_cache=cache.v, slot_mapping=g.slot_mapping) if write_cache else {}
                ops.qkv_post(qkv, q, H=H, Hkv=Hkv, hd=hd, positions=ctx.positions, page_size=cache.page_size,
                             **norm, **rot, **wr)
            else:
                ops.qkv_post(qkv, q, H=H, Hkv=Hkv, hd=hd, positions=ctx.positions, k_out=k, **norm)
                self.position.apply_step(q, k, ctx)
                if write_cache:
                    v = qkv[:, (H + Hkv) * hd:].contiguous()
                    ops.kv_write(k, v, cache.k, cache.v, g.slot_mapping, Hkv=Hkv, hd=hd, page_size=cache.page_size)
            self.attend(q, o, ctx, cache, g)

        ctx.run_eagerly(over_the_cache)
        self.out.forward(o, accumulate_into=residual, next_norm=next_norm)

    @staticmethod
    def _upload(array, device):
        """Through pinned memory, so that the host does not wait for the stream."""
        return torch.from_numpy(array).pin_memory().to(device, non_blocking=True)

    @classmethod
    def _blocks(cls, ctx, G, nb, device, skip_single: bool = False, longest_first: bool = False):
        key = ("query_blocks", G, nb, skip_single, longest_first)
        blocks = ctx.host.get(key)
        if blocks is None:
            q_len = ctx.host["q_len"]
            if skip_single:
                q_len = np.where(q_len == 1, 0, q_len)
            ctx_len = ctx.host["ctx_len"] if longest_first else None
            blocks = ctx.host[key] = cls._upload(ops.query_blocks(q_len, G, nb, ctx_len), device)
        return blocks

    @classmethod
    def _single_token_runs(cls, ctx, G, device):
        """Runs of neighbouring requests with one token each in a step that also holds portions:
        [(first token, tokens, block list, request records relative to the first token, longest
        context)], made once a step.  Only where a request's heads fit one block of 16 columns."""
        key = ("single_token_runs", G)
        runs = ctx.host.get(key)
        if runs is None:
            runs = []
            q_len, ctx_len = ctx.host["q_len"], ctx.host["ctx_len"]
            if G <= 16 and (q_len == 1).any():
                start = np.concatenate([[0], np.cumsum(q_len)[:-1]])
                single = np.concatenate([[False], q_len == 1, [False]])
                edges = np.flatnonzero(single[1:] != single[:-1])          # run r_lo .. r_hi - 1 for every pair
                for r_lo, r_hi in zip(edges[0::2], edges[1::2]):
                    tok_lo = int(start[r_lo])
                    info = np.stack([start - tok_lo, q_len, ctx_len - q_len, ctx_len], axis=1).astype(np.int32)
                    blocks = np.stack([np.arange(r_lo, r_hi), np.zeros(r_hi - r_lo, dtype=np.int64)], axis=1).astype(np.int32)
                    runs.append((tok_lo, int(r_hi - r_lo), cls._upload(blocks, device), cls._upload(info, device),
                                 int(ctx_len[r_lo:r_hi].max())))
            ctx.host[key] = runs
        return runs

    def attend(self, q, o, ctx, cache, g) -> None:
        G = self.H // self.Hkv
        if ops.attention_mfma_supported(q.dtype, self.hd, cache.page_size):
            common = dict(block_table=g.block_table, req_info=ctx.req_info, H=self.H, Hkv=self.Hkv, hd=self.hd,
                          page_size=cache.page_size, max_ctx_len=ctx.max_ctx_len, window=self.window or 0,
                          scale=self.scale)
            if ctx.max_q_len > 1:
                # prompt portions in the step: blocks of columns walk over their keys through LDS.
                # Requests with a single token beside them (runs of neighbours in the step's order) go
                # the way of a step of single tokens: one workgroup walking all keys of such a request
                # would be the longest of the step.
                nb = ops.attention_prefill_block_columns(self.hd) // 16
                runs = self._single_token_runs(ctx, G, q.device)
                # (first: with key segments it writes every row of o, the single tokens' rows come after)
                ops.attention_prefill(q, cache.k, cache.v, o, blocks=self._blocks(ctx, G, nb, q.device, skip_single=bool(runs), longest_first=True),
                                      positions=ctx.positions, **common)
                for tok_lo, n, blocks, info, ctx_len in runs:
                    ops.attention_mfma(q[tok_lo:tok_lo + n], cache.k, cache.v, o[tok_lo:tok_lo + n], blocks=blocks, nb=1,
                                       positions=ctx.positions[tok_lo:tok_lo + n], **dict(common, req_info=info, max_ctx_len=ctx_len))
                return
            # single tokens: the keys of a request are split over many waves, then merged
            nb = 1 if G <= 16 else (2 if G <= 32 else 4)
            blocks = self._blocks(ctx, G, nb, q.device) if G > 16 * nb else None
            ops.attention_mfma(q, cache.k, cache.v, o, blocks=blocks, nb=nb, positions=ctx.positions, **common)
            return
        ops.attention_general(q, cache.k, cache.v, o, block_table=g.block_table,
                              req_of_token=ctx.req_of_token, positions=ctx.positions,
                              H=self.H, Hkv=self.Hkv, hd=self.hd, page_size=cache.page_size,
                              window=self.window or 0, scale=self.scale)
