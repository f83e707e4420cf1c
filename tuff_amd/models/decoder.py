"""A decoder as data: an embedding, a set of blocks, the order in which they run, a final norm
and a head.  The run order is a list of LayerRun; it may name a block twice (each run then has
a cache of its own) or let a run read the cache that another run writes.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from ..csrc import ops
from ..parts.base import Block, FixedState, Norm, PagedKV, Runtime, WeightDecl, cache_specs_of


@dataclasses.dataclass(frozen=True)
class LayerRun:
    block: int                      # index into DecoderModel.blocks
    cache: Optional[int] = None     # cache entry this run uses (default: one of its own)
    writes: bool = True             # False: only reads the entry, which an earlier run writes


class _Head:
    """Stands for the head as the consumer of the final norm."""
    accepts_pending_norm = True


_HEAD = _Head()


class DecoderModel:
    def __init__(self, *, vocab_size: int, hidden_size: int, embedding: WeightDecl,
                 blocks: list[Block], final_norm: Norm, head: Optional[WeightDecl] = None,
                 schedule: Optional[list[LayerRun]] = None, max_positions: Optional[int] = None,
                 eos_token_id: Optional[int] = None, embedding_scale: float = 1.0,
                 logit_scale: float = 1.0, logit_softcap: Optional[float] = None):
        """head=None: the head is the embedding (tied), as the reference does when the file has
        no output matrix (src/lfm25_model.c:128-131).
        embedding_scale: the embedding rows are multiplied by it on their way into the residual stream.
        logit_scale, logit_softcap: logits = head(norm(x)) * logit_scale, then, with a cap c,
        c * tanh(logits / c).  The reference has none of the three (scale 1, no cap), which are the defaults."""
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.embedding_decl, self.head_decl = embedding, head
        self.blocks, self.final_norm = list(blocks), final_norm
        self.max_positions, self.eos_token_id = max_positions, eos_token_id
        self.embedding_scale, self.logit_scale = float(embedding_scale), float(logit_scale)
        self.logit_softcap = None if not logit_softcap else float(logit_softcap)
        runs = schedule if schedule is not None else [LayerRun(i) for i in range(len(self.blocks))]
        self.schedule: list[LayerRun] = []
        next_id = 0
        used = {r.cache for r in runs if r.cache is not None}
        for r in runs:
            if not 0 <= r.block < len(self.blocks):
                raise ValueError(f"run order names block {r.block}; there are {len(self.blocks)}")
            cache = r.cache
            if cache is None:
                while next_id in used:
                    next_id += 1
                cache = next_id
                used.add(cache)
            self.schedule.append(LayerRun(r.block, cache, r.writes))
        # Every cache entry has exactly one writer, which comes before its readers.  A run's entry is named
        # by LayerRun.cache; a mixer that declares several things to keep has the entries (cache, 0),
        # (cache, 1), ... in the order of its declarations.
        self.cache_specs: dict = {}
        self._run_entries: list = []             # per run: (the mixer declares a tuple, its entry ids)
        written: dict = {}
        for r in self.schedule:
            specs, several = cache_specs_of(self.blocks[r.block].mixer)
            ids = tuple((r.cache, j) for j in range(len(specs))) if several else (r.cache,) * len(specs)
            if r.writes:
                if r.cache in written:
                    raise ValueError(f"cache entry {r.cache} has two writers")
                written[r.cache] = specs
                self.cache_specs.update(zip(ids, specs))
            else:
                if r.cache not in written:
                    raise ValueError(f"a run reads cache entry {r.cache} before any run writes it")
                if written[r.cache] != specs:
                    raise ValueError(f"a run reads cache entry {r.cache} of another shape: "
                                     f"{written[r.cache]} vs {specs}")
                if any(isinstance(s_, FixedState) for s_ in specs):
                    raise ValueError("a fixed-size state cannot be shared between runs")
            self._run_entries.append((several, ids))
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None

    # ------------------------------------------------------------------ description
    def weight_decls(self) -> list[WeightDecl]:
        decls = [self.embedding_decl]
        for b in self.blocks:
            decls += b.weight_decls()
        decls += self.final_norm.weight_decls()
        if self.head_decl is not None:
            decls.append(self.head_decl)
        seen, out = set(), []
        for d in decls:
            if d.name in seen:
                raise ValueError(f"two parts declare the tensor '{d.name}'")
            seen.add(d.name)
            out.append(d)
        return out

    def kernel_modules(self) -> list[str]:
        mods = ["elementwise"]
        for b in self.blocks:
            mods += b.kernel_modules()
        mods += self.final_norm.kernel_modules()
        return sorted(set(mods))

    def token_inputs(self) -> tuple:
        """What the parts read of a step's tokens beside ids and positions (parts.base.TokenInput), a name once."""
        from ..engine.batch import merge_token_inputs
        return merge_token_inputs([t for b in self.blocks for t in b.token_inputs()])

    def graph_safe(self) -> bool:
        return all(b.graph_safe for b in self.blocks) and self.final_norm.graph_safe

    def records_portions(self) -> bool:
        return self.graph_safe() and all(getattr(b, "records_portions", False) for b in self.blocks)

    def num_parameters(self) -> int:
        n = 0
        for d in self.weight_decls():
            k = 1
            for s in d.shape:
                k *= s
            n += k
        return n

    # ------------------------------------------------------------------------ bind
    def bind(self, weights: dict[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        self.embedding = weights[self.embedding_decl.name]
        self.head = weights[self.head_decl.name] if self.head_decl is not None else self.embedding
        for b in self.blocks:
            b.bind(weights, rt)
        self.final_norm.bind(weights, rt)
        self._head_cast: Optional[torch.Tensor] = None
        if self.head.dtype != rt.dtype and self.head.dtype != torch.float32:
            raise TypeError(f"head weight of type {self.head.dtype} in a {rt.dtype} run")
        if self.head.dtype == torch.bfloat16:
            # the matrix kernels stream a tile-major copy; a tied embedding keeps its rows for the lookup
            if self.hidden_size % 8 != 0:
                raise ValueError(f"the bfloat16 matrix kernels need a hidden size that is a multiple of 8, "
                                 f"got {self.hidden_size}")
            self.head = ops.tile_weight(self.head)

    # --------------------------------------------------------------------- forward
    def forward(self, ctx, cache_views: dict[int, object]) -> Optional[torch.Tensor]:
        """Runs the step's tokens through all layers.  Returns float32 logits
        [len(ctx.logit_rows), vocab], or None when no logits are wanted."""
        rt = self.rt
        x = torch.empty(ctx.T, self.hidden_size, dtype=torch.float32, device=rt.device)
        ops.embed_rows(self.embedding, ctx.tokens, x, self.embedding_scale)
        head_fused, all_rows = self._head_fused(ctx)
        for i, run in enumerate(self.schedule):
            block = self.blocks[run.block]
            if getattr(block, "takes_next_norm", False):
                if i + 1 < len(self.schedule):
                    nb = self.blocks[self.schedule[i + 1].block]
                    nxt = nb.first_norm_consumer() if hasattr(nb, "first_norm_consumer") else None
                else:
                    nxt = (self.final_norm, _HEAD) if head_fused and all_rows else None
                block.forward(x, ctx, self._views_of(i, cache_views), run.writes, next_norm=nxt)
            else:
                block.forward(x, ctx, self._views_of(i, cache_views), run.writes)
        # which rows are wanted is a fact of the step, not of its shape: the head runs outside of what is recorded
        # (a recorder keeps the function and hands back what it returns at each replay)
        # What the last block left for the final norm is taken here, where the step's kernels are issued (or
        # recorded: the tensors are then the recording's own, and every replay's head finds them as the eager
        # step's head does), not inside the function that runs later.
        pre = None
        if head_fused and all_rows and hasattr(self.final_norm, "take_announced"):
            pre = self.final_norm.take_announced(x)
        out: list = []

        def head(c):
            out[:] = [self._head(x, c, pre)]
            return out[0]

        ctx.run_eagerly(head)
        for part in self.blocks + [self.final_norm]:
            if hasattr(part, "forget"):                # what a product left for a norm that never asked for it
                part.forget()
        return out[0] if out else None

    def recording_key(self, ctx) -> tuple:
        """What forward() reads of a step outside of ctx.run_eagerly and bakes into its launches: a
        recording of a step in sections is valid for steps with the same key."""
        head_fused, all_rows = self._head_fused(ctx)
        return (ctx.T, bool(head_fused and all_rows))

    def _views_of(self, i: int, cache_views: dict):
        """What run i's mixer is handed as `cache`: None, a view, or a tuple of views."""
        several, ids = self._run_entries[i]
        if several:
            return tuple(cache_views[e] for e in ids)
        return cache_views[ids[0]] if ids else None

    def _head_fused(self, ctx) -> tuple:
        all_rows = ctx.n_logits == ctx.T and bool(ctx.host.get("logit_rows_identity", False))
        # the final norm inside the head's product (at most 16 rows), or, when every row is wanted,
        # from the row scales the last block leaves (at most 64)
        fused = (hasattr(self.final_norm, "pending") and self.head.dtype == torch.bfloat16
                 and self.hidden_size % 8 == 0 and ctx.n_logits > 0
                 and (ctx.n_logits <= ops.NORMED_MAX_ROWS and self.hidden_size <= ops.NORMED_MAX_K
                      or all_rows and ctx.n_logits <= ops.EMIT_MAX_ROWS))
        return fused, all_rows

    def _head(self, x, ctx, pre=None) -> Optional[torch.Tensor]:
        logits = self._head_product(x, ctx, pre)
        if logits is not None and (self.logit_scale != 1.0 or self.logit_softcap is not None):
            ops.scale_cap(logits, self.logit_scale, self.logit_softcap or 0.0)
        return logits

    def _head_product(self, x, ctx, pre=None) -> Optional[torch.Tensor]:
        """pre: (xw, ss), the final norm's operand and row sums as the last block's product left them, or None."""
        if ctx.n_logits == 0:
            return None
        rt = self.rt
        head_fused, all_rows = self._head_fused(ctx)
        logits = torch.empty(ctx.n_logits, self.vocab_size, dtype=torch.float32, device=rt.device)
        if head_fused:
            fn = self.final_norm
            if pre is not None and all_rows:
                ops.gemm_scaled(pre[0], pre[1], fn.eps, self.head, logits)
                return logits
            if ctx.n_logits <= ops.NORMED_MAX_ROWS and self.hidden_size <= ops.NORMED_MAX_K:
                ops.gemm_normed(x, fn.weight_f32, fn.eps, self.head, logits, rows=ctx.logit_rows)
                return logits
        h = self.final_norm.forward(x, rows=ctx.logit_rows)
        if h.dtype != self.head.dtype:
            h32 = torch.empty(h.shape, dtype=torch.float32, device=rt.device)
            ops.cast(h, h32)
            h = h32
        ops.gemm(h, self.head, logits)
        return logits
