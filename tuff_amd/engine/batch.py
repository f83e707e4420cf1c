"""The description of one step as the kernels read it: a flat list of tokens with, per token,
its position and request, and, per request, where its tokens start, its state slot and its
block tables.  Everything goes to the device in one copy.
"""
from __future__ import annotations

import dataclasses
from typing import Hashable, Sequence

import numpy as np
import torch


@dataclasses.dataclass
class StepEntry:
    """The next tokens of one request, and the places among them whose logits are wanted."""
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclasses.dataclass
class GroupContext:
    block_table: torch.Tensor      # int32 [R, max_blocks]; -1 where a window freed the page
    slot_mapping: torch.Tensor     # int32 [T]: page * page_size + offset of each token


@dataclasses.dataclass
class StepContext:
    T: int                         # tokens in this step
    R: int                         # requests in this step
    n_logits: int
    tokens: torch.Tensor           # int32 [T]
    positions: torch.Tensor        # int32 [T] absolute position of each token in its request
    req_of_token: torch.Tensor     # int32 [T] index into the per-request arrays below
    q_start: torch.Tensor          # int32 [R] first token of the request in this step
    q_len: torch.Tensor            # int32 [R] number of its tokens in this step
    ctx_len: torch.Tensor          # int32 [R] length of the request after this step
    state_slot: torch.Tensor       # int32 [R]
    logit_rows: torch.Tensor       # int32 [n_logits] indices into the step's tokens
    groups: list[GroupContext]
    # host-side facts kernels may be chosen by
    max_q_len: int = 1
    max_ctx_len: int = 1
    host: dict = dataclasses.field(default_factory=dict)


def build_context(entries: Sequence[StepEntry], manager, device, vocab_size: int) -> StepContext:
    """`manager` has already been extended by every entry's tokens."""
    R = len(entries)
    T = sum(len(e.tokens) for e in entries)
    n_groups = len(manager.groups)
    max_blocks = max(1, max(len(manager.block_table(e.req_id, g)) for e in entries for g in range(n_groups))
                     if n_groups else 1)
    n_logits = sum(len(e.want) for e in entries)
    ps = manager.page_size
    # one int32 buffer: [tokens | positions | req_of_token | q_start | q_len | ctx_len | slot |
    #                    logit_rows | per group: slot_mapping, block_table]
    sizes = [T, T, T, R, R, R, R, n_logits] + [T, R * max_blocks] * n_groups
    offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    buf = np.zeros(int(offs[-1]), dtype=np.int32)
    tokens, positions, req_of = (buf[offs[i]:offs[i + 1]] for i in range(3))
    q_start, q_len, ctx_len, slot, rows = (buf[offs[i]:offs[i + 1]] for i in range(3, 8))
    t = 0
    li = 0
    max_q = max_ctx = 1
    for r, e in enumerate(entries):
        n = len(e.tokens)
        total = manager.length(e.req_id)
        past = total - n
        toks = np.asarray(e.tokens, dtype=np.int64)
        if n and (toks.min() < 0 or toks.max() >= vocab_size):
            raise ValueError(f"request {e.req_id!r}: token id outside [0, {vocab_size})")
        tokens[t:t + n] = toks
        positions[t:t + n] = np.arange(past, total)
        req_of[t:t + n] = r
        q_start[r], q_len[r], ctx_len[r], slot[r] = t, n, total, manager.slot(e.req_id)
        for w in e.want:
            if not 0 <= w < n:
                raise ValueError(f"request {e.req_id!r}: wanted place {w} is outside its {n} tokens")
            rows[li] = t + w
            li += 1
        for g in range(n_groups):
            table = manager.block_table(e.req_id, g)
            sm = buf[offs[8 + 2 * g]:offs[9 + 2 * g]]
            bt = buf[offs[9 + 2 * g]:offs[10 + 2 * g]].reshape(R, max_blocks)
            bt[r, :len(table)] = table
            bt[r, len(table):] = -1
            pos = np.arange(past, total)
            pages = np.asarray(table, dtype=np.int64)[pos // ps] if n else np.zeros(0, dtype=np.int64)
            if n and pages.min() < 0:
                raise RuntimeError(f"request {e.req_id!r}: a token would be written to a freed page")
            sm[t:t + n] = pages * ps + pos % ps
        t += n
        max_q, max_ctx = max(max_q, n), max(max_ctx, total)
    host = torch.from_numpy(buf)
    dev = host.pin_memory().to(device, non_blocking=True) if buf.size else host.to(device)
    sl = lambda i: dev[int(offs[i]):int(offs[i + 1])]
    groups = [GroupContext(block_table=sl(9 + 2 * g).view(R, max_blocks), slot_mapping=sl(8 + 2 * g))
              for g in range(n_groups)]
    return StepContext(T=T, R=R, n_logits=n_logits, tokens=sl(0), positions=sl(1), req_of_token=sl(2),
                       q_start=sl(3), q_len=sl(4), ctx_len=sl(5), state_slot=sl(6), logit_rows=sl(7),
                       groups=groups, max_q_len=max_q, max_ctx_len=max_ctx,
                       host={"q_len": q_len.copy(), "ctx_len": ctx_len.copy()})
