"""The description of one step as the kernels read it: a flat list of tokens with, per token,
its position and request, and, per request, where its tokens start, its state slot and its
block tables.  Everything is packed into one int32 buffer and goes to the device in one copy;
the device tensors are views into that buffer, so a recorded graph can be replayed after the
buffer alone was refreshed.
"""
from __future__ import annotations

import dataclasses
from typing import Hashable, Mapping, Optional, Sequence

import numpy as np
import torch


@dataclasses.dataclass
class StepEntry:
    """The next tokens of one request, and the places among them whose logits are wanted."""
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()
    inputs: Optional[Mapping[str, Sequence]] = None    # name -> integers [n tokens] or [n tokens, cols], for what the model's parts declare (parts.base.TokenInput)


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
    req_info: torch.Tensor         # int32 [R, 4]: (q_start, q_len, position of the first token, ctx_len)
    groups: list[GroupContext]
    # host-side facts kernels may be chosen by
    max_q_len: int = 1
    max_ctx_len: int = 1           # an upper bound of every position + 1 of the step
    host: dict = dataclasses.field(default_factory=dict)     # 'q_len', 'ctx_len' (numpy) and what parts cache
    recorder: object = None        # set while a step is recorded in sections
    inputs: dict = dataclasses.field(default_factory=dict)   # name -> int32 [T, cols]: what parts declared as TokenInput

    def run_eagerly(self, fn) -> None:
        """fn(ctx) now; where the step is being recorded in sections, fn is kept instead and runs at
        every replay, between the graphs of what came before and after it, with that step's ctx."""
        if self.recorder is None:
            fn(self)
        else:
            self.recorder.eager(fn)


@dataclasses.dataclass
class PackedStep:
    """A step on the host: the int32 buffer and where its pieces lie."""
    buf: np.ndarray
    offs: np.ndarray
    T: int
    R: int
    n_logits: int
    n_groups: int
    max_blocks: int
    max_q_len: int
    max_ctx_len: int
    q_len: np.ndarray
    ctx_len: np.ndarray
    logit_rows_identity: bool = False     # logits are wanted of every token of the step, in order
    token_inputs: tuple = ()              # the TokenInput declarations whose values lie behind the last piece, in this order

    def shape_key(self):
        return (self.T, self.R, self.n_logits, self.n_groups, self.max_blocks, self.logit_rows_identity)


def merge_token_inputs(decls) -> tuple:
    """The declarations of all parts of a model as one tuple, a name once; two parts that name the same input
    must mean the same."""
    out: dict = {}
    for d in decls:
        if d.name in out and out[d.name] != d:
            raise ValueError(f"two parts declare the token input '{d.name}' differently: {out[d.name]} and {d}")
        if d.cols < 1:
            raise ValueError(f"token input '{d.name}': {d.cols} columns")
        out[d.name] = d
    return tuple(out.values())


def check_token_inputs(entries, token_inputs) -> None:
    """Raises ValueError, by request and name, where an entry's inputs are not what the model's parts declared:
    one that is missing and has no default, a wrong shape or type, one that no part reads."""
    if not token_inputs and not any(e.inputs for e in entries):
        return
    for e in entries:
        n = len(e.tokens)
        for d in token_inputs:
            given = None if e.inputs is None else e.inputs.get(d.name)
            if given is None:
                if d.default is None:
                    raise ValueError(f"request {e.req_id!r}: the model reads the input '{d.name}' of every token, and this "
                                     f"entry brings none")
                continue
            a = np.asarray(given)
            if a.dtype.kind not in "iu" or a.shape not in ((n, d.cols),) + (((n,),) if d.cols == 1 else ()):
                raise ValueError(f"request {e.req_id!r}: input '{d.name}' must be integers of shape [{n}, {d.cols}], "
                                 f"got {a.dtype} {list(a.shape)}")
        for name in (e.inputs or ()):
            if all(name != d.name for d in token_inputs):
                raise ValueError(f"request {e.req_id!r}: no part of the model reads an input '{name}'")


def _fill_token_inputs(buf, offs, first, token_inputs, entries, manager) -> None:
    for i, d in enumerate(token_inputs):
        dst = buf[offs[first + i]:offs[first + i + 1]].reshape(-1, d.cols)
        t = 0
        for e in entries:
            n = len(e.tokens)
            given = None if e.inputs is None else e.inputs.get(d.name)
            if given is not None:
                dst[t:t + n] = np.asarray(given).reshape(n, d.cols)
            elif isinstance(d.default, str) and d.default == "position":
                total = manager.length(e.req_id)
                dst[t:t + n] = np.arange(total - n, total)[:, None]
            else:
                dst[t:t + n] = int(d.default)
            t += n


def pack_step(entries: Sequence[StepEntry], manager, vocab_size: int,
              max_blocks: Optional[int] = None, token_inputs: tuple = ()) -> PackedStep:
    """`manager` has already been extended by every entry's tokens.  max_blocks: width of the
    block tables (default: the longest table of the step).  token_inputs: the model's TokenInput
    declarations; their values go behind everything else, [T, cols] each."""
    R = len(entries)
    T = sum(len(e.tokens) for e in entries)
    n_groups = len(manager.groups)
    tables = [[manager.block_table_array(e.req_id, g) for g in range(n_groups)] for e in entries]
    longest = max([len(t) for ts in tables for t in ts] + [1])
    if max_blocks is None:
        max_blocks = longest
    elif max_blocks < longest:
        raise ValueError(f"block tables need {longest} entries, {max_blocks} given")
    n_logits = sum(len(e.want) for e in entries)
    ps = manager.page_size
    # [tokens | positions | req_of_token | q_start | q_len | ctx_len | slot | logit_rows |
    #  per group: slot_mapping, block_table]
    sizes = [T, T, T, R, R, R, R, n_logits] + [T, R * max_blocks] * n_groups + [4 * R] + [T * d.cols for d in token_inputs]
    offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    buf = np.zeros(int(offs[-1]), dtype=np.int32)
    tokens, positions, req_of = (buf[offs[i]:offs[i + 1]] for i in range(3))
    q_start, q_len, ctx_len, slot, rows = (buf[offs[i]:offs[i + 1]] for i in range(3, 8))
    info = buf[offs[8 + 2 * n_groups]:offs[9 + 2 * n_groups]].reshape(R, 4)
    t = li = 0
    max_q = max_ctx = 1
    slot_maps = [buf[offs[8 + 2 * g]:offs[9 + 2 * g]] for g in range(n_groups)]
    block_tables = [buf[offs[9 + 2 * g]:offs[10 + 2 * g]].reshape(R, max_blocks) for g in range(n_groups)]
    for bt in block_tables:
        bt.fill(-1)
    for r, e in enumerate(entries):
        n = len(e.tokens)
        total = manager.length(e.req_id)
        past = total - n
        if n == 1:                        # the common entry of a serving step, without array detours
            tok = int(e.tokens[0])
            if tok < 0 or tok >= vocab_size:
                raise ValueError(f"request {e.req_id!r}: token id outside [0, {vocab_size})")
            tokens[t], positions[t], req_of[t] = tok, past, r
        else:
            toks = np.asarray(e.tokens, dtype=np.int64)
            if n and (toks.min() < 0 or toks.max() >= vocab_size):
                raise ValueError(f"request {e.req_id!r}: token id outside [0, {vocab_size})")
            tokens[t:t + n] = toks
            positions[t:t + n] = np.arange(past, total)
            req_of[t:t + n] = r
        q_start[r], q_len[r], ctx_len[r], slot[r] = t, n, total, manager.slot(e.req_id)
        info[r] = (t, n, past, total)
        for w in e.want:
            if not 0 <= w < n:
                raise ValueError(f"request {e.req_id!r}: wanted place {w} is outside its {n} tokens")
            rows[li] = t + w
            li += 1
        for g in range(n_groups):
            table = tables[r][g]
            block_tables[g][r, :len(table)] = table
            if n == 1:
                page = int(table[past // ps])
                if page < 0:
                    raise RuntimeError(f"request {e.req_id!r}: a token would be written to a freed page")
                slot_maps[g][t] = page * ps + past % ps
            elif n:
                pos = np.arange(past, total)
                pages = table[pos // ps].astype(np.int64)
                if pages.min() < 0:
                    raise RuntimeError(f"request {e.req_id!r}: a token would be written to a freed page")
                slot_maps[g][t:t + n] = pages * ps + pos % ps
        t += n
        max_q, max_ctx = max(max_q, n), max(max_ctx, total)
    identity = n_logits == T and bool((rows == np.arange(T)).all())
    check_token_inputs(entries, token_inputs)
    _fill_token_inputs(buf, offs, 9 + 2 * n_groups, token_inputs, entries, manager)
    return PackedStep(buf, offs, T, R, n_logits, n_groups, max_blocks, max_q, max_ctx, q_len.copy(), ctx_len.copy(),
                      identity, tuple(token_inputs))


def context_on(dev: torch.Tensor, p: PackedStep, max_ctx_len: Optional[int] = None) -> StepContext:
    """Views of the device buffer `dev` (same layout as p.buf) as a StepContext."""
    offs = p.offs
    sl = lambda i: dev[int(offs[i]):int(offs[i + 1])]
    groups = [GroupContext(block_table=sl(9 + 2 * g).view(p.R, p.max_blocks), slot_mapping=sl(8 + 2 * g))
              for g in range(p.n_groups)]
    return StepContext(T=p.T, R=p.R, n_logits=p.n_logits, tokens=sl(0), positions=sl(1), req_of_token=sl(2),
                       q_start=sl(3), q_len=sl(4), ctx_len=sl(5), state_slot=sl(6), logit_rows=sl(7),
                       req_info=sl(8 + 2 * p.n_groups).view(p.R, 4), groups=groups, max_q_len=p.max_q_len,
                       max_ctx_len=max_ctx_len if max_ctx_len is not None else p.max_ctx_len,
                       host={"q_len": p.q_len, "ctx_len": p.ctx_len, "logit_rows_identity": p.logit_rows_identity,
                             "packed": {name: p.buf[int(offs[i]):int(offs[i + 1])] for i, name in
                                        ((0, "tokens"), (2, "req_of_token"), (3, "q_start"), (4, "q_len"), (6, "state_slot"))}},
                       inputs={d.name: sl(9 + 2 * p.n_groups + i).view(p.T, d.cols) for i, d in enumerate(p.token_inputs)})


def build_context(entries: Sequence[StepEntry], manager, device, vocab_size: int, token_inputs: tuple = ()) -> StepContext:
    p = pack_step(entries, manager, vocab_size, token_inputs=token_inputs)
    host = torch.from_numpy(p.buf)
    dev = host.pin_memory().to(device, non_blocking=True) if p.buf.size else host.to(device)
    return context_on(dev, p)
