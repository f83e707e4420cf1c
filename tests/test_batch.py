"""The packed description of a step (engine/batch.py) on the CPU: what lies where in the one int32 buffer,
and the integers that come with tokens beside their ids (parts.base.TokenInput)."""
import numpy as np
import pytest
import torch

from tuff_amd.cache.manager import CacheLayout, CacheManager
from tuff_amd.engine.batch import StepEntry, context_on, merge_token_inputs, pack_step
from tuff_amd.parts.base import FixedState, PagedKV, TokenInput


def manager(page_size=4, pages=32, slots=4):
    layout = CacheLayout.from_specs({0: PagedKV(1, 8), 1: FixedState((3,))})
    return CacheManager(layout, page_size=page_size, num_pages=pages, num_slots=slots)


def begin(mgr, lengths: dict):
    for rid, n in lengths.items():
        mgr.admit(rid)
        mgr.extend(rid, n)


def test_a_step_is_packed_token_by_token_and_request_by_request():
    mgr = manager()
    begin(mgr, {"a": 5, "b": 1})
    p = pack_step([StepEntry("a", [7, 8, 9, 1, 2], [4]), StepEntry("b", [3], [0])], mgr, vocab_size=10)
    ctx = context_on(torch.from_numpy(p.buf), p)
    assert ctx.T == 6 and ctx.R == 2 and ctx.n_logits == 2
    assert ctx.tokens.tolist() == [7, 8, 9, 1, 2, 3]
    assert ctx.positions.tolist() == [0, 1, 2, 3, 4, 0]
    assert ctx.req_of_token.tolist() == [0, 0, 0, 0, 0, 1]
    assert ctx.q_start.tolist() == [0, 5] and ctx.q_len.tolist() == [5, 1] and ctx.ctx_len.tolist() == [5, 1]
    assert ctx.logit_rows.tolist() == [4, 5]
    assert ctx.req_info.tolist() == [[0, 5, 0, 5], [5, 1, 0, 1]]
    table = ctx.groups[0].block_table
    assert ctx.groups[0].slot_mapping.tolist() == [int(table[0, i // 4]) * 4 + i % 4 for i in range(5)] + [int(table[1, 0]) * 4]
    assert ctx.inputs == {}
    # the next portion goes on where the request stands
    mgr.extend("a", 2)
    p = pack_step([StepEntry("a", [4, 4], [])], mgr, vocab_size=10)
    assert context_on(torch.from_numpy(p.buf), p).positions.tolist() == [5, 6]


def test_what_a_step_refuses():
    mgr = manager()
    begin(mgr, {"a": 2})
    with pytest.raises(ValueError, match="token id outside"):
        pack_step([StepEntry("a", [1, 10], [])], mgr, vocab_size=10)
    with pytest.raises(ValueError, match="wanted place 2"):
        pack_step([StepEntry("a", [1, 2], [2])], mgr, vocab_size=10)
    with pytest.raises(ValueError, match="block tables need"):
        pack_step([StepEntry("a", [1, 2], [])], mgr, vocab_size=10, max_blocks=0)


GRID = TokenInput("grid", cols=2)
SEGMENT = TokenInput("segment", default=0)
PLACE = TokenInput("place", cols=3, default="position")


def test_integers_beside_the_tokens_lie_behind_everything_else():
    mgr = manager()
    begin(mgr, {"a": 3, "b": 2})
    decls = (GRID, SEGMENT, PLACE)
    plain = pack_step([StepEntry("a", [1, 2, 3], [2]), StepEntry("b", [4, 5], [])], mgr, vocab_size=10)
    p = pack_step([StepEntry("a", [1, 2, 3], [2], {"grid": [[0, 0], [0, 1], [1, 0]], "segment": [7, 7, 8]}),
                   StepEntry("b", [4, 5], [], {"grid": np.array([[5, 6], [5, 7]])})], mgr, vocab_size=10, token_inputs=decls)
    # nothing before them has moved
    assert np.array_equal(p.buf[:len(plain.buf)], plain.buf) and len(p.buf) == len(plain.buf) + 5 * (2 + 1 + 3)
    assert p.shape_key() == plain.shape_key()
    ctx = context_on(torch.from_numpy(p.buf), p)
    assert ctx.inputs["grid"].tolist() == [[0, 0], [0, 1], [1, 0], [5, 6], [5, 7]]
    assert ctx.inputs["segment"].tolist() == [[7], [7], [8], [0], [0]]               # b brings none: the default
    assert ctx.inputs["place"].tolist() == [[0] * 3, [1] * 3, [2] * 3, [0] * 3, [1] * 3]   # the position in every column
    # a later portion: the default "position" goes on counting
    mgr.extend("b", 2)
    p = pack_step([StepEntry("b", [1, 1], [], {"grid": [[0, 0], [0, 0]]})], mgr, vocab_size=10, token_inputs=decls)
    assert context_on(torch.from_numpy(p.buf), p).inputs["place"][:, 0].tolist() == [2, 3]


def test_inputs_that_do_not_fit_are_refused_by_name():
    mgr = manager()
    begin(mgr, {"a": 2})
    with pytest.raises(ValueError, match="'a'.*reads the input 'grid' of every token"):
        pack_step([StepEntry("a", [1, 2], [])], mgr, vocab_size=10, token_inputs=(GRID,))
    with pytest.raises(ValueError, match=r"input 'grid' must be integers of shape \[2, 2\], got int64 \[2\]"):
        pack_step([StepEntry("a", [1, 2], [], {"grid": [1, 2]})], mgr, vocab_size=10, token_inputs=(GRID,))
    with pytest.raises(ValueError, match="must be integers"):
        pack_step([StepEntry("a", [1, 2], [], {"grid": [[0.5, 1], [2, 3]]})], mgr, vocab_size=10, token_inputs=(GRID,))
    with pytest.raises(ValueError, match="no part of the model reads an input 'colour'"):
        pack_step([StepEntry("a", [1, 2], [], {"colour": [1, 2]})], mgr, vocab_size=10)
    # one column may come as a plain list
    p = pack_step([StepEntry("a", [1, 2], [], {"segment": [4, 5]})], mgr, vocab_size=10, token_inputs=(SEGMENT,))
    assert context_on(torch.from_numpy(p.buf), p).inputs["segment"].tolist() == [[4], [5]]


def test_parts_that_name_the_same_input_must_mean_the_same():
    assert merge_token_inputs([GRID, SEGMENT, GRID]) == (GRID, SEGMENT)
    with pytest.raises(ValueError, match="'grid' differently"):
        merge_token_inputs([GRID, TokenInput("grid", cols=3)])
    with pytest.raises(ValueError, match="0 columns"):
        merge_token_inputs([TokenInput("x", cols=0)])


def test_the_lfm2_model_reads_nothing_beside_ids_and_positions():
    from tuff_amd.models.registry import build_model, config_from_dict
    import util
    model = build_model(config_from_dict(util.CONFIGS["A"][0]))
    assert model.token_inputs() == ()
