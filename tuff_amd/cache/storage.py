"""The tensors behind the cache manager's book-keeping.

Per PagedKV entry: K as [num_pages, kv_heads, page_size, head_dim] and V transposed within the
page, [num_pages, kv_heads, value_dim, page_size] (the matrix cores read both with the summed
index contiguous; value_dim is head_dim unless the part declares another; a part that declares
`value_rows` gets [num_pages, kv_heads, page_size, value_dim] instead), in the compute dtype
(bfloat16 in serving, float32 in the 32-bit path; the reference keeps float32 rows
[layer][kv_head][pos][hd], src/lfm25_gpu.cu:480-483).  Per FixedState entry: one
tensor [num_slots, *shape] of the declared type (float32 unless the part says otherwise).  Pages are not cleared when they are handed out again: nothing
reads a position before it is written (with poison=True the pool starts as NaN and pages are
filled with NaN again when they are given back, which shows any such read).  A state slot is zeroed when a request takes it
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
    state: torch.Tensor              # [num_slots, *shape] in the declared type
    raw: torch.Tensor                # the same memory as int32 words [num_slots, words]


_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= d
    return n


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
            vshape = (n, spec.num_kv_heads, ps, spec.v_dim) if spec.value_rows else (n, spec.num_kv_heads, spec.v_dim, ps)
            if poison:
                # stale reads show up as NaN in the logits
                k = torch.full(shape, float("nan"), dtype=dtype, device=device)
                v = torch.full(vshape, float("nan"), dtype=dtype, device=device)
            else:
                k = torch.empty(shape, dtype=dtype, device=device)
                v = torch.empty(vshape, dtype=dtype, device=device)
            self.views[e] = PagedKVView(k, v, gi, ps, spec.window)
        for e, spec in layout.states.items():
            # a slot is a whole number of 32-bit words, so that one fill kernel clears any type
            words = -(-spec.nbytes() // 4)
            raw = torch.zeros(manager.num_slots, words, dtype=torch.int32, device=device)
            typed = raw.view(_STATE_DTYPES[spec.dtype])[:, :_numel(spec.shape)]
            self.views[e] = StateView(typed.view((manager.num_slots,) + tuple(spec.shape)), raw)

        if poison:
            manager.on_free = self.poison_pages

    def poison_pages(self, group: int, pages) -> None:
        """Debugging aid (poison=True): pages that go back to the pool are filled with NaN, on the
        stream, so that a later read of a position nobody has written since shows in the logits."""
        idx = None
        for v in self.views.values():
            if isinstance(v, PagedKVView) and v.group == group:
                if idx is None:
                    idx = torch.tensor(list(pages), dtype=torch.long, device=v.k.device)
                v.k[idx] = float("nan")
                v.v[idx] = float("nan")

    def zero_slot(self, slot: int) -> None:
        for v in self.views.values():
            if isinstance(v, StateView):
                ops.fill_u32(v.raw[slot], 0)

    def nbytes(self) -> int:
        n = 0
        for v in self.views.values():
            if isinstance(v, PagedKVView):
                n += (v.k.numel() + v.v.numel()) * v.k.element_size()
            else:
                n += v.raw.numel() * 4
        return n
