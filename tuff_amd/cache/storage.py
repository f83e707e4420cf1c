"""The tensors behind the cache manager's book-keeping.

Per PagedKV entry: K as [num_pages, kv_heads, page_size, head_dim] and V transposed within the
page, [num_pages, kv_heads, head_dim, page_size] (the matrix cores read both with the summed
index contiguous), in the compute dtype
(bfloat16 in serving, float32 in the 32-bit path; the reference keeps float32 rows
[layer][kv_head][pos][hd], src/lfm25_gpu.cu:480-483).  Per FixedState entry: one float32
tensor [num_slots, *shape].  Pages are not cleared when they are handed out again: nothing
reads a position before it is written.  A state slot is zeroed when a request takes it
(the reference zeroes its conv state at start, src/lfm25_engine.c:46-51).
"""
from __future__ import annotations

import dataclasses

import torch

from ..csrc import ops
from .manager import CacheLayout, CacheManager


@dataclasses.dataclass
class PagedKVView:
    k: torch.Tensor
    v: torch.Tensor
    group: int
    page_size: int
    window: object


@dataclasses.dataclass
class StateView:
    state: torch.Tensor


class CacheStorage:
    def __init__(self, manager: CacheManager, dtype: torch.dtype, device, poison: bool = False):
        self.manager = manager
        layout: CacheLayout = manager.layout
        self.views: dict[int, object] = {}
        ps = manager.page_size
        for e, spec in layout.paged.items():
            gi = layout.group_of_entry[e]
            n = manager.groups[gi].pool.num_pages
            shape = (n, spec.num_kv_heads, ps, spec.head_dim)
            vshape = (n, spec.num_kv_heads, spec.head_dim, ps)
            if poison:
                # stale reads show up as NaN in the logits
                k = torch.full(shape, float("nan"), dtype=dtype, device=device)
                v = torch.full(vshape, float("nan"), dtype=dtype, device=device)
            else:
                k = torch.empty(shape, dtype=dtype, device=device)
                v = torch.empty(vshape, dtype=dtype, device=device)
            self.views[e] = PagedKVView(k, v, gi, ps, spec.window)
        for e, spec in layout.states.items():
            st = torch.zeros((manager.num_slots,) + tuple(spec.shape), dtype=torch.float32, device=device)
            self.views[e] = StateView(st)

    def zero_slot(self, slot: int) -> None:
        for v in self.views.values():
            if isinstance(v, StateView):
                ops.fill_u32(v.state[slot], 0)

    def nbytes(self) -> int:
        n = 0
        for v in self.views.values():
            if isinstance(v, PagedKVView):
                n += v.k.numel() * v.k.element_size() * 2
            else:
                n += v.state.numel() * 4
        return n
