"""The attention entry point that allocates nothing (tuff_attention_mfma_static), called through
ctypes as a C caller would, against tuff_attention_mfma with a work space of the caller's: two calls
in a row, the second on a smaller step, so that what the first left in the library's array lies
under the second."""
import ctypes
import math

import pytest
import torch

from test_gpu_kernels import _check_step, _mixed_step_case

pytestmark = pytest.mark.gpu

_i, _f, _p, _ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong


def _library():
    from tuff_amd.csrc import build
    lib = ctypes.CDLL(build.ensure_built("attention_mfma"))
    lib.tuff_attention_static_setup.argtypes = []
    lib.tuff_attention_static_setup.restype = _i
    lib.tuff_attention_static_floats.argtypes = [_i, _i, _i, _i, ctypes.POINTER(_ll)]
    lib.tuff_attention_static_floats.restype = _ll
    lib.tuff_attention_mfma_static.argtypes = [_p, _p, _p, _p, _p, _i, _p, _i, _i, _p, _p,
                                               _i, _i, _i, _i, _i, _i, _f, _i, _p]
    lib.tuff_attention_mfma_static.restype = _i
    lib.tuff_attention_mfma.argtypes = [_p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _p, _p,
                                        _i, _i, _i, _i, _i, _i, _f, _i, _p]
    lib.tuff_attention_mfma.restype = _i
    return lib


def _step(gpu, reqs, H, Hkv, hd, ps, nb):
    from tuff_amd.csrc import ops
    case = _mixed_step_case(gpu, reqs, H, Hkv, hd, ps)
    case["q_gpu"] = case["q"].to(gpu)
    case["blocks"] = torch.from_numpy(ops.query_blocks(case["q_len"], H // Hkv, nb)).to(gpu)
    case["n_parts"] = -(-case["max_ctx_len"] // 256)
    return case


def _run(lib, case, H, Hkv, hd, ps, nb, window, static):
    T = case["q_gpu"].shape[0]
    out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=case["q_gpu"].device)
    n_parts = case["n_parts"]
    stream = torch.cuda.current_stream().cuda_stream
    common = (case["table"].data_ptr(), case["table"].shape[1], case["blocks"].data_ptr(), case["blocks"].shape[0], nb,
              case["req_info"].data_ptr(), case["positions"].data_ptr(), T, H, Hkv, hd, ps, window,
              1 / math.sqrt(hd), n_parts, stream)
    head = (case["q_gpu"].data_ptr(), case["kc"].data_ptr(), case["vc"].data_ptr(), out.data_ptr())
    if static:
        rc = lib.tuff_attention_mfma_static(*head, *common)
    else:
        ws_o = torch.empty(T * H * n_parts * hd, dtype=torch.float32, device=out.device)
        ws_ml = torch.empty(T * H * n_parts * 2, dtype=torch.float32, device=out.device)
        rc = lib.tuff_attention_mfma(*head, ws_o.data_ptr(), ws_ml.data_ptr(), *common)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("H,Hkv,hd,ps,nb", [(32, 8, 64, 16, 1), (6, 2, 128, 64, 2)])
@pytest.mark.parametrize("window", [0, 300])
def test_static_attention_equals_the_one_with_a_work_space(gpu, H, Hkv, hd, ps, nb, window):
    lib = _library()
    assert lib.tuff_attention_static_setup() == 0
    large = [(1499, 1), (230, 50), (0, 33), (700, 1), (255, 3), (1023, 2)]
    small = [(300, 1), (0, 5)]
    for tag, reqs in (("first call", large), ("second, smaller call", small)):
        case = _step(gpu, reqs, H, Hkv, hd, ps, nb)
        want = _run(lib, case, H, Hkv, hd, ps, nb, window, static=False)
        got = _run(lib, case, H, Hkv, hd, ps, nb, window, static=True)
        assert torch.isfinite(got.float()).all(), tag
        assert torch.equal(got, want), tag
        _check_step(case, reqs, got.cpu().double().reshape(-1, H, hd), H, hd, window, tag)


def test_static_attention_refuses_what_does_not_fit(gpu):
    lib = _library()
    cap = _ll(0)
    need = lib.tuff_attention_static_floats(64, 32, 64, 128, ctypes.byref(cap))
    assert cap.value == 4 << 20 and need > cap.value
    # refused before anything is read: the pointers are never touched
    rc = lib.tuff_attention_mfma_static(None, None, None, None, None, 2048, None, 64, 1, None, None,
                                        64, 32, 8, 64, 16, 0, 0.125, 128, None)
    assert rc == -7
    assert lib.tuff_attention_static_floats(8, 32, 64, 32, None) <= cap.value
