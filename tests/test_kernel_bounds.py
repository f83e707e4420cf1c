"""Host arithmetic that the kernels' memory accesses rest on, checked without a GPU: the functions
are the kernels' own (compiled for host and device from one definition) and are called through
the built library."""
import ctypes

import pytest


@pytest.fixture(scope="module")
def mfma_lib():
    from tuff_amd.csrc import ops
    lib = ops.load("attention_mfma")
    lib.tuff_attention_partition_pages.argtypes = [ctypes.c_int, ctypes.c_int]
    lib.tuff_attention_partition_pages.restype = ctypes.c_int
    return lib


def test_single_token_attention_fetches_every_page_a_partition_touches(mfma_lib):
    """A partition of 256 keys that starts inside a page (page sizes that do not divide 256: 96, 112,
    144, ...) touches one page more than 256 / page size rounded up.  For every page size the kernel
    takes and every partition: lanes that fetch a page number == pages touched, and a wave has enough
    lanes.  (With 256 / page size rounded up, pages of 96 positions left the partition at key 256
    one page short: page number -1 from a lane that fetched nothing, keys read from before the pool.)"""
    from tuff_amd.csrc import ops
    part_keys = ops.ATTN_PARTITION
    short = set()
    for ps in range(16, 513, 16):
        for part in range(0, 2048 if ps <= 128 else 300):
            first = part * part_keys
            touched = (first + part_keys - 1) // ps - first // ps + 1
            assert touched == len({k // ps for k in range(first, first + part_keys, 16)})
            lanes = mfma_lib.tuff_attention_partition_pages(part, ps)
            assert lanes == touched, (ps, part, lanes, touched)
            assert lanes <= 64
            if touched > -(-part_keys // ps):
                short.add(ps)
    assert {96, 112, 144} <= short          # the sizes the old bound was wrong for are among those walked


def test_partition_pages_refuses_nonsense(mfma_lib):
    assert mfma_lib.tuff_attention_partition_pages(-1, 16) < 0
    assert mfma_lib.tuff_attention_partition_pages(0, 0) < 0
    assert mfma_lib.tuff_attention_partition_pages(2 ** 31 // 256, 16) < 0
