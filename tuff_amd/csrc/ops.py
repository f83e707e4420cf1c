"""Python face of the HIP kernels: loads the compiled libraries with ctypes, checks every
operand on the host (device, dtype, contiguity, shape) and launches on torch's current stream.

There is no other implementation behind these functions: a missing library is compiled, a
library that cannot be compiled or a tensor that is not on the GPU is an error.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional

import torch

from . import build

DT_F32, DT_BF16 = 0, 1
OUT_BF16, OUT_F32, OUT_F32_ACCUM, OUT_SWIGLU = 0, 1, 2, 3

_c_int, _c_float, _c_void_p, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong


class KernelError(RuntimeError):
    pass


_SIGNATURES = {
    "elementwise": {
        "tuff_embed_rows": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
        "tuff_add_bias": [_c_void_p, _c_int, _c_void_p, _c_ll, _c_int, _c_void_p],
        "tuff_scale_cap": [_c_void_p, _c_ll, _c_float, _c_float, _c_void_p],
        "tuff_rmsnorm": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_int, _c_float, _c_void_p],
        "tuff_swiglu": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_cast": [_c_void_p, _c_int, _c_void_p, _c_int, _c_ll, _c_void_p],
        "tuff_fill_u32": [_c_void_p, ctypes.c_uint32, _c_ll, _c_void_p],
        "tuff_scatter_i32": [_c_void_p, _c_int, _c_void_p, _c_int, _c_void_p, _c_int, _c_void_p],
    },
    "gemm_f32": {
        "tuff_gemm_f32": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    },
    "gemm_bf16": {
        "tuff_gemm_bf16": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_workspace": [_c_int, _c_int, _c_int, _c_int, ctypes.POINTER(_c_ll)],
        "tuff_gemm_bf16_emit_layout": [_c_int, _c_int, _c_int, ctypes.POINTER(_c_int), ctypes.POINTER(_c_int)],
        "tuff_gemm_bf16_scaled_supported": [_c_int, _c_int, _c_int],
        "tuff_gemm_bf16_accum_emit": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p, _c_void_p,
                                      _c_void_p, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_scaled": [_c_void_p, _c_void_p, _c_int, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                  _c_int, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_conv": [_c_void_p, _c_int, _c_void_p, _c_float, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_int,
                                _c_int, _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_conv64": [_c_void_p, _c_void_p, _c_int, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                  _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
        "tuff_gemm_bf16_normed": [_c_void_p, _c_void_p, _c_void_p, _c_float, _c_void_p, _c_void_p, _c_int, _c_int, _c_int,
                                  _c_int, _c_void_p],
    },
    "rope_kv": {
        "tuff_qkv_post": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                          _c_void_p, _c_void_p, _c_int, _c_float,
                          _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_void_p, _c_int, _c_void_p],
        "tuff_rope_table": [_c_void_p, _c_int, _c_int, _c_void_p, _c_void_p],
        "tuff_kv_write": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p,
                          _c_int, _c_int, _c_int, _c_int, _c_void_p],
    },
    "attention": {
        "tuff_attention_general": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
                                   _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                   _c_float, _c_void_p],
    },
    "attention_mfma": {
        "tuff_attention_mfma": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                                _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p],
        "tuff_attention_merge": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_void_p],
        "tuff_attention_decode_fused": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                        _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_float,
                                        _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                                        _c_void_p],
        "tuff_attention_mfma_static": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int,
                                       _c_void_p, _c_int, _c_int, _c_void_p, _c_void_p,
                                       _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_void_p],
    },
    "attention_prefill": {
        "tuff_attention_prefill": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_int,
                                   _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int,
                                   _c_void_p, _c_void_p, _c_void_p],
        "tuff_attention_prefill_block_columns": [_c_int],
    },
    "shortconv": {
        "tuff_shortconv_fwd": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p,
                               _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
        "tuff_shortconv_decode": [_c_void_p, _c_void_p, _c_int, _c_void_p, _c_void_p, _c_int, _c_void_p,
                                  _c_int, _c_int, _c_int, _c_void_p],
        "tuff_shortconv_state": [_c_void_p, _c_int, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                 _c_int, _c_int, _c_int, _c_void_p],
    },
    "sampling": {
        "tuff_argmax": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
        "tuff_sample": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                        _c_int, _c_int, _c_void_p],
        "tuff_repeat_penalty": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    },
}

_libs: dict[str, ctypes.CDLL] = {}

# TUFF_TRACE=1: GPU time by kernel class.  Every entry point of the kernel libraries is timed with a pair of
# events around its launches (an entry point is a class of kernels: the attention of single tokens is its
# partition kernel and its merge), and trace_report() prints calls, total, mean, least and most per class, in the
# manner of the reference's TUFF_TRACE report (src/cupti_profiler.cu:115-181, switched on at src/main.c:1787-1789).
# Events cannot be recorded into a graph, so an engine records no steps while this is on, and the step's time is
# that of its launches one by one.
TRACE = os.environ.get("TUFF_TRACE", "")[:1] == "1"
_trace_open: list = []                   # (class, start event, end event) not yet read
_trace_stats: dict = {}                  # class -> [calls, total ms, least ms, most ms]


def _trace_fold(everything: bool) -> None:
    """Reads the events that have completed (all of them after a synchronisation) into the statistics."""
    if everything:
        torch.cuda.synchronize()
    keep = []
    for name, a, b in _trace_open:
        if not everything and not b.query():
            keep.append((name, a, b))
            continue
        ms = a.elapsed_time(b)
        st = _trace_stats.setdefault(name, [0, 0.0, float("inf"), 0.0])
        st[0] += 1
        st[1] += ms
        st[2] = min(st[2], ms)
        st[3] = max(st[3], ms)
    _trace_open[:] = keep


def _traced(name: str, fn):
    def call(*args):
        if torch.cuda.is_current_stream_capturing():
            return fn(*args)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        rc = fn(*args)
        b.record()
        _trace_open.append((name, a, b))
        if len(_trace_open) >= 4096:
            _trace_fold(False)
        return rc
    return call


def trace_reset() -> None:
    _trace_fold(True)
    _trace_stats.clear()


def trace_stats() -> dict:
    """{kernel class: (calls, total ms, least ms, most ms)} since the last trace_reset()."""
    _trace_fold(True)
    return {k: tuple(v) for k, v in _trace_stats.items()}


def trace_report(out) -> None:
    stats = sorted(trace_stats().items(), key=lambda kv: -kv[1][1])
    total = sum(v[1] for _, v in stats)
    line = "=" * 104
    print(f"\n{line}\n{'GPU TIME BY KERNEL CLASS (TUFF_TRACE)':^104}\n{line}", file=out)
    print(f"Total GPU time in kernel classes: {total:.3f} ms\n", file=out)
    print(f"{'Kernel class (entry point)':<44} | {'Calls':>7} | {'Total(ms)':>10} | {'Avg(us)':>9} | {'Min(us)':>9} | "
          f"{'Max(us)':>9} | {'GPU Time%':>9}", file=out)
    print("-" * 104, file=out)
    for name, (calls, ms, lo, hi) in stats:
        print(f"{name:<44} | {calls:>7} | {ms:>10.3f} | {1e3 * ms / calls:>9.2f} | {1e3 * lo:>9.2f} | {1e3 * hi:>9.2f} | "
              f"{100 * ms / total if total else 0:>8.1f}%", file=out)
    print(line, file=out)


def load(module: str) -> ctypes.CDLL:
    """The loaded library of a kernel module; compiled at first use if it is not built yet."""
    lib = _libs.get(module)
    if lib is None:
        path = build.ensure_built(module)
        lib = ctypes.CDLL(path)
        for name, argtypes in _SIGNATURES.get(module, {}).items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
            if TRACE and argtypes and argtypes[-1] is _c_void_p:        # (the last argument is the stream: it launches)
                setattr(lib, name, _traced(name, fn))
        _libs[module] = lib
    return lib


def loaded_modules() -> list[str]:
    return sorted(_libs)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _stream() -> int:
    """Handle of torch's current stream on the current device (the stream a graph is being
    recorded on, inside a recording).  Called once a launch, so through the cheapest way there is."""
    if _raw_stream is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DT_F32
    if t.dtype == torch.bfloat16:
        return DT_BF16
    raise KernelError(f"unsupported element type {t.dtype}; kernels take float32 and bfloat16")


def _gpu(name: str, t: torch.Tensor, dtype=None, shape=None) -> int:
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on '{t.device}'; the kernels run on the GPU only "
                          f"and there is no CPU fallback")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor must be contiguous (shape {tuple(t.shape)}, stride {t.stride()})")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if shape is not None and tuple(shape) != t.shape:        # torch.Size compares equal to a tuple
        if len(shape) != t.dim() or any(s is not None and s != g for s, g in zip(shape, t.shape)):
            raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")
    return t.data_ptr()


def _opt(name, t, dtype=None, shape=None) -> Optional[int]:
    return None if t is None else _gpu(name, t, dtype, shape)


def _check(code: int, what: str) -> None:
    if code != 0:
        if code == -2:
            raise KernelError(f"{what}: the kernel refuses these sizes")
        if code == -7:
            raise KernelError(f"{what}: the step needs more work space than the library's static array holds")
        raise KernelError(f"{what}: launch failed with HIP error {code}")


# ------------------------------------------------------------------------ row kernels
def embed_rows(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t] = table[tokens[t]] * scale, float32."""
    n, d = out.shape
    _check(load("elementwise").tuff_embed_rows(
        _gpu("table", table, shape=(None, d)), _dt(table), _gpu("tokens", tokens, torch.int32, (n,)),
        _gpu("out", out, torch.float32), n, d, float(scale), _stream()), "embed_rows")


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """y[r, c] += bias[c] in place (y float32 or bfloat16 [rows, N], bias float32 [N])."""
    rows, N = y.shape
    _gpu("y", y)
    _gpu("bias", bias, torch.float32, (N,))
    _check(load("elementwise").tuff_add_bias(y.data_ptr(), _dt(y), bias.data_ptr(), rows, N, _stream()), "add_bias")


def scale_cap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> None:
    """x <- x * scale, then, with cap > 0, x <- cap * tanh(x / cap); float32, in place."""
    _gpu("x", x, torch.float32)
    _check(load("elementwise").tuff_scale_cap(x.data_ptr(), x.numel(), float(scale), float(cap), _stream()), "scale_cap")


def rmsnorm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, eps: float,
            rows: Optional[torch.Tensor] = None) -> None:
    n, d = out.shape
    if rows is None:
        _gpu("x", x, torch.float32, (n, d))
    else:
        _gpu("x", x, torch.float32, (None, d))
    _check(load("elementwise").tuff_rmsnorm(
        x.data_ptr(), _gpu("w", w, shape=(d,)), _dt(w), _gpu("out", out), _dt(out),
        _opt("rows", rows, torch.int32, (n,)), n, d, float(eps), _stream()), "rmsnorm")


def swiglu(gu: torch.Tensor, act: torch.Tensor) -> None:
    n, F = act.shape
    _check(load("elementwise").tuff_swiglu(
        _gpu("gu", gu, act.dtype, (n, 2 * F)), _gpu("act", act), _dt(act), n, F, _stream()), "swiglu")


def cast(inp: torch.Tensor, out: torch.Tensor) -> None:
    if inp.numel() != out.numel():
        raise KernelError(f"cast: {inp.numel()} elements in, {out.numel()} out")
    _check(load("elementwise").tuff_cast(_gpu("inp", inp), _dt(inp), _gpu("out", out), _dt(out),
                                         inp.numel(), _stream()), "cast")


def fill_u32(t: torch.Tensor, value: int = 0) -> None:
    """Sets every 32-bit word of `t` to `value` (t must be a 4-byte type)."""
    if t.element_size() != 4:
        raise KernelError("fill_u32: tensor elements must be 4 bytes wide")
    if not t.is_cuda or not t.is_contiguous():
        raise KernelError("fill_u32: contiguous GPU tensor required")
    _check(load("elementwise").tuff_fill_u32(t.data_ptr(), value, t.numel(), _stream()), "fill_u32")


def scatter_i32(dst: torch.Tensor, src: torch.Tensor, idx: torch.Tensor) -> None:
    """dst[idx[i]] = src[idx[n + i]] for i < n = len(idx) / 2; all int32 on the GPU."""
    n = idx.shape[0] // 2
    _check(load("elementwise").tuff_scatter_i32(_gpu("dst", dst, torch.int32), dst.numel(), _gpu("src", src, torch.int32),
                                                src.numel(), _gpu("idx", idx, torch.int32, (2 * n,)), n, _stream()),
           "scatter_i32")


# ------------------------------------------------------------------------------ GEMM
class TiledWeight:
    """A bfloat16 weight [N, K] in the order the matrix kernels stream it: blocks of 16 rows x 32 k,
    [ceil(N/16)][ceil(K/32)] of them, each 1 KB with piece l of 16 bytes = row l % 16,
    k 8 (l // 16) .. 8 (l // 16) + 7; rows and k beyond the matrix are zero."""

    def __init__(self, blocks: torch.Tensor, N: int, K: int):
        self.blocks, self.shape = blocks, (int(N), int(K))
        self.dtype, self.device = blocks.dtype, blocks.device

    def data_ptr(self) -> int:
        return self.blocks.data_ptr()

    def rows(self) -> torch.Tensor:
        """The weight back in row-major order [N, K] (a copy)."""
        N, K = self.shape
        t = self.blocks.view(-1, self.blocks.shape[1], 4, 16, 8).permute(0, 3, 1, 2, 4)
        return t.reshape(t.shape[0] * 16, -1)[:N, :K].contiguous()


def tile_weight(w: torch.Tensor) -> TiledWeight:
    """The tile-major copy of a row-major bfloat16 weight [N, K].  Made once when a weight is bound."""
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise KernelError(f"tile_weight: a bfloat16 matrix is needed, got {w.dtype} {tuple(w.shape)}")
    N, K = w.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    if (Np, Kp) != (N, K):
        padded = torch.zeros(Np, Kp, dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
        w = padded
    blocks = w.view(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    return TiledWeight(blocks.view(Np // 16, Kp // 32, 64, 8), N, K)


def _tiled(w, N: int, K: int) -> TiledWeight:
    """w as the bfloat16 kernels take it.  A plain tensor is converted on the spot (tests and single
    calls; the parts bind tiled weights)."""
    if not isinstance(w, TiledWeight):
        _gpu("w", w, torch.bfloat16, (N, K))
        w = tile_weight(w)
    if not w.blocks.is_cuda or not w.blocks.is_contiguous() or w.shape != (N, K):
        raise KernelError(f"w: a tiled weight {(N, K)} on the GPU is needed, got {w.shape} on {w.device}")
    return w


def _bf16_mode(out: torch.Tensor, accumulate: bool, swiglu: bool, M: int, N: int) -> int:
    if swiglu:
        if accumulate or out.dtype != torch.bfloat16 or N % 2:
            raise KernelError("gemm: the SwiGLU epilogue writes bfloat16 [M, N/2] and cannot accumulate")
        _gpu("out", out, shape=(M, N // 2))
        return OUT_SWIGLU
    _gpu("out", out, shape=(M, N))
    if out.dtype == torch.float32:
        return OUT_F32_ACCUM if accumulate else OUT_F32
    if out.dtype == torch.bfloat16:
        if accumulate:
            raise KernelError("gemm: accumulation needs a float32 output")
        return OUT_BF16
    raise KernelError(f"gemm: unsupported output type {out.dtype}")


def gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         swiglu: bool = False) -> None:
    """out (=|+=) x @ w.T.  x [M, K], w [N, K] of one dtype; float32 operands give the true
    float32 product, bfloat16 operands the matrix-core product with float32 accumulation.
    `out` is float32 (stored or accumulated into) or, for bfloat16 operands, bfloat16.
    swiglu (bfloat16 only): the rows of w are gate and up rows interleaved and out [M, N/2] is
    silu(gate) * up."""
    M, K = x.shape
    N = w.shape[0]
    _gpu("x", x)
    if x.dtype == torch.float32:
        if isinstance(w, TiledWeight):
            raise KernelError("gemm: float32 activations with a tiled bfloat16 weight")
        _gpu("w", w, x.dtype, (N, K))
        if out.dtype != torch.float32 or swiglu:
            raise KernelError("gemm: float32 operands need a float32 output and have no fused epilogue")
        _gpu("out", out, shape=(M, N))
        _check(load("gemm_f32").tuff_gemm_f32(x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K,
                                              int(accumulate), _stream()), "gemm_f32")
        return
    if x.dtype != torch.bfloat16:
        raise KernelError(f"gemm: unsupported operand type {x.dtype}")
    if K % 8 != 0:
        raise KernelError(f"gemm: the bfloat16 kernels need an inner size that is a multiple of 8, got {K}")
    w = _tiled(w, N, K)
    mode = _bf16_mode(out, accumulate, swiglu, M, N)
    ws = _gemm_workspace(M, N, K, x.device)
    _check(load("gemm_bf16").tuff_gemm_bf16(x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, mode,
                                            None if ws is None else ws.data_ptr(), _stream()), "gemm_bf16")


NORMED_MAX_ROWS, NORMED_MAX_K = 16, 8192      # gemm_normed: the norm inside the product's kernel
EMIT_MAX_ROWS = 64                            # gemm_accum_emit / gemm_scaled: the skinny products; beyond, the tiled one


def gemm_normed(x: torch.Tensor, norm_w: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor, *,
                rows: Optional[torch.Tensor] = None, accumulate: bool = False, swiglu: bool = False) -> None:
    """out (=|+=) rmsnorm(x[rows]) @ w.T in one kernel, for at most 16 rows: x float32 [*, K],
    norm_w float32 [K], w bfloat16 [N, K].  The row's 1/rms scales the result, the norm weight
    the operand."""
    K = x.shape[1]
    M = x.shape[0] if rows is None else rows.shape[0]
    N = w.shape[0]
    _gpu("x", x, torch.float32)
    _gpu("norm_w", norm_w, torch.float32, (K,))
    w = _tiled(w, N, K)
    _opt("rows", rows, torch.int32, (M,))
    if M > NORMED_MAX_ROWS or K > NORMED_MAX_K or K % 8:
        raise KernelError(f"gemm_normed: at most {NORMED_MAX_ROWS} rows and an inner size that is a multiple of 8 "
                          f"up to {NORMED_MAX_K}; got {M} rows, inner size {K}")
    mode = _bf16_mode(out, accumulate, swiglu, M, N)
    _check(load("gemm_bf16").tuff_gemm_bf16_normed(
        x.data_ptr(), None if rows is None else rows.data_ptr(), norm_w.data_ptr(), float(eps), w.data_ptr(),
        out.data_ptr(), M, N, K, mode, _stream()), "gemm_bf16_normed")


_emit_layouts: dict = {}


def gemm_emit_layout(M: int, N: int, K: int) -> Optional[tuple]:
    """(tiles, rows): shape of the sums of squares gemm_accum_emit leaves for a product of M rows
    with N outputs and inner size K, or None where such a product cannot leave them (more than 64 rows
    and an inner size that is no multiple of 64, a product cut along K, a last block of columns that is
    not whole)."""
    key = (M if M > 16 else 0, N, K)                   # (which kernel takes 17 to 64 rows depends on all three)
    if key not in _emit_layouts:
        t, r = _c_int(0), _c_int(0)
        _check(load("gemm_bf16").tuff_gemm_bf16_emit_layout(M, N, K, ctypes.byref(t), ctypes.byref(r)), "gemm_emit_layout")
        _emit_layouts[key] = (int(t.value), int(r.value)) if t.value > 0 else None
    return _emit_layouts[key]


def gemm_accum_emit(x: torch.Tensor, w, residual: torch.Tensor, next_norm_w: torch.Tensor,
                    xw: torch.Tensor, ss: torch.Tensor) -> None:
    """residual += x @ w.T, and for the RMSNorm that follows: xw = the new residual times next_norm_w as
    bfloat16, ss [gemm_emit_layout(M, N, K)] = per-tile sums of squares of each row."""
    M, K = x.shape
    N = w.shape[0]
    _gpu("x", x, torch.bfloat16)
    w = _tiled(w, N, K)
    _gpu("residual", residual, torch.float32, (M, N))
    _gpu("next_norm_w", next_norm_w, torch.float32, (N,))
    _gpu("xw", xw, torch.bfloat16, (M, N))
    layout = gemm_emit_layout(M, N, K) if K % 8 == 0 else None
    if layout is None:
        raise KernelError(f"gemm_accum_emit: a product of {M} rows, {N} outputs and inner size {K} cannot leave the next "
                          f"norm's operand (ask gemm_emit_layout first)")
    _gpu("ss", ss, torch.float32, layout)
    ws = _gemm_workspace(M, N, K, x.device, emit=True)
    _check(load("gemm_bf16").tuff_gemm_bf16_accum_emit(x.data_ptr(), w.data_ptr(), residual.data_ptr(), M, N, K,
                                                       next_norm_w.data_ptr(), xw.data_ptr(), ss.data_ptr(),
                                                       None if ws is None else ws.data_ptr(), _stream()),
           "gemm_bf16_accum_emit")


_scaled_ok: dict = {}


def gemm_scaled_supported(M: int, N: int, K: int, out_dtype=torch.bfloat16, accumulate: bool = False) -> bool:
    """Whether gemm_scaled takes this product: any with at most 64 rows; with more, bfloat16 (or SwiGLU)
    outputs of products that run in one piece."""
    if K % 8:
        return False
    if M <= EMIT_MAX_ROWS:
        return True
    if accumulate or out_dtype != torch.bfloat16:
        return False
    key = (M, N, K)
    if key not in _scaled_ok:
        _scaled_ok[key] = bool(load("gemm_bf16").tuff_gemm_bf16_scaled_supported(M, N, K))
    return _scaled_ok[key]


def gemm_scaled(xw: torch.Tensor, ss: torch.Tensor, eps: float, w, out: torch.Tensor, *,
                accumulate: bool = False, swiglu: bool = False) -> None:
    """out (=|+=) rmsnorm(x) @ w.T from what gemm_accum_emit left for the same number of rows:
    xw = bf16(x * norm weight) and the per-tile sums of squares ss; each row of the product is
    scaled by 1 / sqrt(sum(ss) / K + eps)."""
    M, K = xw.shape
    N = w.shape[0]
    _gpu("xw", xw, torch.bfloat16)
    if not gemm_scaled_supported(M, N, K, out.dtype, accumulate):
        raise KernelError(f"gemm_scaled: a product of {M} rows, {N} outputs, inner size {K} into {out.dtype} is not "
                          f"supported (ask gemm_scaled_supported first)")
    _gpu("ss", ss, torch.float32, (None, 16 if M <= 16 else 64 if M <= EMIT_MAX_ROWS else M))
    w = _tiled(w, N, K)
    mode = _bf16_mode(out, accumulate, swiglu, M, N)
    ws = _gemm_workspace(M, N, K, xw.device)
    _check(load("gemm_bf16").tuff_gemm_bf16_scaled(xw.data_ptr(), ss.data_ptr(), ss.shape[0], float(eps), w.data_ptr(),
                                                   out.data_ptr(), M, N, K, mode,
                                                   None if ws is None else ws.data_ptr(), _stream()), "gemm_bf16_scaled")


CONV_MAX_ROWS = 32                            # gemm_conv: one token a row (the norm inside: at most NORMED_MAX_ROWS)


def conv_group_rows(w_in: torch.Tensor) -> torch.Tensor:
    """The input projection [3 d, K] of a gated short convolution (rows: B, then C, then X) with its
    rows regrouped for gemm_conv: sixteen channels a group, each group as [its B rows | its C rows |
    its X rows].  d must be a multiple of 16."""
    three_d, K = w_in.shape
    d = three_d // 3
    if three_d != 3 * d or d % 16:
        raise KernelError(f"conv_group_rows: [3 d, K] with d a multiple of 16 is needed, got {tuple(w_in.shape)}")
    return w_in.view(3, d // 16, 16, K).permute(1, 0, 2, 3).reshape(three_d, K).contiguous()


def gemm_conv(x: torch.Tensor, w, out: torch.Tensor, *, conv_w: torch.Tensor, state: torch.Tensor, state_slot: torch.Tensor,
              norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, ss: Optional[torch.Tensor] = None) -> None:
    """Input projection and gated short convolution of single tokens (row r is request r's token, at
    most 32 rows) in one kernel: out [M, d] bfloat16 = C * conv(B * X) with (B, C, X) = x @ w.T, and
    the rows' states shifted.  w: conv_group_rows() of the projection, tiled.  x: bfloat16 [M, K]; or
    the float32 residual stream with norm_w and eps (the RMSNorm runs inside); or bf16(x * norm weight)
    with ss and eps as gemm_accum_emit leaves them."""
    M, K = x.shape
    d = out.shape[1]
    taps = conv_w.shape[1]
    _gpu("out", out, torch.bfloat16, (M, d))
    w = _tiled(w, 3 * d, K)
    _gpu("conv_w", conv_w, shape=(d, taps))
    _gpu("state", state, torch.float32, (None, taps - 1, d))
    _gpu("state_slot", state_slot, torch.int32, (M,))
    if M > CONV_MAX_ROWS or K % 8 or d % 16 or not 2 <= taps <= 17:
        raise KernelError(f"gemm_conv: at most {CONV_MAX_ROWS} rows, an inner size that is a multiple of 8, a width that is a "
                          f"multiple of 16 and 2 to 17 taps; got {M} rows, inner size {K}, width {d}, {taps} taps")
    kind, nw_ptr, ss_ptr, n_ss = 0, None, None, 0
    if ss is not None:
        _gpu("x", x, torch.bfloat16)
        _gpu("ss", ss, torch.float32, (None, 16 if M <= 16 else 64))
        kind, ss_ptr, n_ss = 2, ss.data_ptr(), ss.shape[0]
    elif norm_w is not None:
        _gpu("x", x, torch.float32)
        _gpu("norm_w", norm_w, torch.float32, (K,))
        if K > NORMED_MAX_K or M > NORMED_MAX_ROWS:
            raise KernelError(f"gemm_conv: the norm inside needs an inner size up to {NORMED_MAX_K} and at most "
                              f"{NORMED_MAX_ROWS} rows, got {K} and {M}")
        kind, nw_ptr = 1, norm_w.data_ptr()
    else:
        _gpu("x", x, torch.bfloat16)
    _check(load("gemm_bf16").tuff_gemm_bf16_conv(
        x.data_ptr(), kind, nw_ptr, float(eps), ss_ptr, n_ss, w.data_ptr(), out.data_ptr(), M, d, K,
        conv_w.data_ptr(), _dt(conv_w), taps, state.data_ptr(), state_slot.data_ptr(), _stream()), "gemm_bf16_conv")


CONV64_MAX_ROWS = 64                          # gemm_conv64: one token a row


def gemm_conv64(x: torch.Tensor, w, out: torch.Tensor, *, conv_w: torch.Tensor, state: torch.Tensor, state_slot: torch.Tensor,
                eps: float = 0.0, ss: Optional[torch.Tensor] = None) -> None:
    """gemm_conv for 33 to 64 rows, in two kernels (the projection's partial tiles; the kernel that adds
    them and runs the convolution), without the projected rows ever being written.  w: the projection
    [3 d, K] as the checkpoint has it (B | C | X), tiled.  x: bfloat16 [M, K], or bf16(x * norm weight)
    with ss [tiles][64] and eps as gemm_accum_emit leaves them for these rows."""
    M, K = x.shape
    d = out.shape[1]
    taps = conv_w.shape[1]
    _gpu("x", x, torch.bfloat16)
    _gpu("out", out, torch.bfloat16, (M, d))
    w = _tiled(w, 3 * d, K)
    _gpu("conv_w", conv_w, shape=(d, taps))
    _gpu("state", state, torch.float32, (None, taps - 1, d))
    _gpu("state_slot", state_slot, torch.int32, (M,))
    if not CONV_MAX_ROWS < M <= CONV64_MAX_ROWS or K % 8 or d % 16 or not 2 <= taps <= 17:
        raise KernelError(f"gemm_conv64: {CONV_MAX_ROWS + 1} to {CONV64_MAX_ROWS} rows, an inner size that is a multiple of 8, a width that is "
                          f"a multiple of 16 and 2 to 17 taps; got {M} rows, inner size {K}, width {d}, {taps} taps")
    ss_ptr, n_ss = None, 0
    if ss is not None:
        _gpu("ss", ss, torch.float32, (None, 64))
        ss_ptr, n_ss = ss.data_ptr(), ss.shape[0]
    ws = _gemm_workspace(M, 3 * d, K, x.device, emit=True)
    _check(load("gemm_bf16").tuff_gemm_bf16_conv64(
        x.data_ptr(), ss_ptr, n_ss, float(eps), w.data_ptr(), out.data_ptr(), M, d, K,
        conv_w.data_ptr(), _dt(conv_w), taps, state.data_ptr(), state_slot.data_ptr(), ws.data_ptr(), _stream()), "gemm_bf16_conv64")


_plans: dict = {}


def _gemm_workspace(M: int, N: int, K: int, device, emit: bool = False) -> Optional[torch.Tensor]:
    """The float32 work space a bfloat16 product of this shape needs, or None.  Taken anew for every
    call: the allocator hands the same block out again."""
    if M <= 16:
        return None
    key = (M, N, K, emit)
    n = _plans.get(key)
    if n is None:
        a = _c_ll(0)
        load("gemm_bf16").tuff_gemm_bf16_workspace(M, N, K, int(emit), ctypes.byref(a))
        n = _plans[key] = int(a.value)
    return torch.empty(n, dtype=torch.float32, device=device) if n else None


# ----------------------------------------------------------------- q/k/v post-processing
def qkv_post(qkv, q_out, *, H, Hkv, hd, positions, eps=0.0, q_norm_w=None, k_norm_w=None,
             inv_freq=None, rotary_dim=0, interleaved=False, k_out=None,
             k_cache=None, v_cache=None, slot_mapping=None, page_size=1, angles=None) -> None:
    T = qkv.shape[0]
    dt = qkv.dtype
    _gpu("qkv", qkv, shape=(T, (H + 2 * Hkv) * hd))
    _gpu("q_out", q_out, dt, (T, H * hd))
    _opt("k_out", k_out, dt, (T, Hkv * hd))
    if (k_cache is None) != (v_cache is None):
        raise KernelError("qkv_post: k_cache and v_cache go together")
    if k_cache is not None:
        if slot_mapping is None:
            raise KernelError("qkv_post: a cache write needs slot_mapping")
        P = k_cache.shape[0]
        _gpu("k_cache", k_cache, dt, (P, Hkv, page_size, hd))
        _gpu("v_cache", v_cache, dt, (P, Hkv, hd, page_size))
        _gpu("slot_mapping", slot_mapping, torch.int32, (T,))
    norm_dt = DT_F32
    if q_norm_w is not None or k_norm_w is not None:
        if q_norm_w is None or k_norm_w is None or q_norm_w.dtype != k_norm_w.dtype:
            raise KernelError("qkv_post: q and k norm weights go together and share a dtype")
        _gpu("q_norm_w", q_norm_w, shape=(hd,))
        _gpu("k_norm_w", k_norm_w, shape=(hd,))
        norm_dt = _dt(q_norm_w)
    if inv_freq is not None:
        if rotary_dim <= 0 or rotary_dim > hd or rotary_dim % 2:
            raise KernelError(f"qkv_post: rotary_dim {rotary_dim} must be even and within the head size {hd}")
        _gpu("inv_freq", inv_freq, torch.float32, (rotary_dim // 2,))
        _opt("angles", angles, torch.float32, (None, 2, rotary_dim // 2))      # rope_table(inv_freq, n)
    _gpu("positions", positions, torch.int32, (T,))
    if hd > 256:
        raise KernelError(f"qkv_post: head size {hd} above 256 is not supported")
    p = lambda t: None if t is None else t.data_ptr()
    _check(load("rope_kv").tuff_qkv_post(
        qkv.data_ptr(), q_out.data_ptr(), p(k_out), p(k_cache), p(v_cache), _dt(qkv),
        p(q_norm_w), p(k_norm_w), norm_dt, float(eps), p(inv_freq), int(rotary_dim), int(interleaved),
        positions.data_ptr(), p(slot_mapping), T, H, Hkv, hd, page_size,
        p(angles) if inv_freq is not None else None, 0 if angles is None else angles.shape[0], _stream()), "qkv_post")


def rope_table(inv_freq: torch.Tensor, n_pos: int) -> torch.Tensor:
    """float32 [n_pos, 2, len(inv_freq)]: cosines and sines of pos * inv_freq, bit for bit what the
    rotation kernels compute for themselves."""
    n_freq = inv_freq.shape[0]
    _gpu("inv_freq", inv_freq, torch.float32, (n_freq,))
    out = torch.empty(int(n_pos), 2, n_freq, dtype=torch.float32, device=inv_freq.device)
    _check(load("rope_kv").tuff_rope_table(inv_freq.data_ptr(), n_freq, int(n_pos), out.data_ptr(), _stream()), "rope_table")
    return out


def kv_write(k, v, k_cache, v_cache, slot_mapping, *, Hkv, hd, page_size) -> None:
    T = k.shape[0]
    dt = k.dtype
    _gpu("k", k, shape=(T, Hkv * hd))
    _gpu("v", v, dt, (T, Hkv * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, dt, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, dt, (P, Hkv, hd, page_size))
    _gpu("slot_mapping", slot_mapping, torch.int32, (T,))
    _check(load("rope_kv").tuff_kv_write(k.data_ptr(), v.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                         _dt(k), slot_mapping.data_ptr(), T, Hkv, hd, page_size, _stream()),
           "kv_write")


# -------------------------------------------------------------------------- attention
def attention_general(q, k_cache, v_cache, out, *, block_table, req_of_token, positions,
                      H, Hkv, hd, page_size, window=0, scale=None) -> None:
    T = q.shape[0]
    dt = q.dtype
    _gpu("q", q, shape=(T, H * hd))
    _gpu("out", out, dt, (T, H * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, dt, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, dt, (P, Hkv, hd, page_size))
    _gpu("block_table", block_table, torch.int32)
    if block_table.dim() != 2:
        raise KernelError("attention: block_table must be [requests, blocks]")
    _gpu("req_of_token", req_of_token, torch.int32, (T,))
    _gpu("positions", positions, torch.int32, (T,))
    if hd > 256 or H % Hkv:
        raise KernelError(f"attention: head size {hd} / heads {H}:{Hkv} not supported")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    _check(load("attention").tuff_attention_general(
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _dt(q),
        block_table.data_ptr(), block_table.shape[1], req_of_token.data_ptr(), positions.data_ptr(),
        T, H, Hkv, hd, page_size, int(window or 0), float(scale), _stream()), "attention_general")


ATTN_PARTITION = 256        # keys a partition of the matrix-core attention kernel covers


def attention_mfma_supported(dtype, hd: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and hd % 8 == 0 and hd <= 256 and page_size % 16 == 0


def attention_mfma(q, k_cache, v_cache, out, *, block_table, blocks, nb, req_info, positions,
                   H, Hkv, hd, page_size, max_ctx_len, window=0, scale=None) -> None:
    """Matrix-core attention over the paged bfloat16 cache.  blocks: int32 [n_blocks, 2] from
    query_blocks(), or None when every request's columns fit one block (block b = request b).
    req_info: int32 [R, 4] = (first token in the step, tokens, first position, -) per request.
    max_ctx_len bounds every position + 1 of the step."""
    T = q.shape[0]
    if not attention_mfma_supported(q.dtype, hd, page_size):
        raise KernelError(f"attention_mfma: needs bfloat16, a head size that is a multiple of 8 (got {hd}) "
                          f"and a page size that is a multiple of 16 (got {page_size})")
    _gpu("q", q, torch.bfloat16, (T, H * hd))
    _gpu("out", out, torch.bfloat16, (T, H * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, hd, page_size))
    _gpu("block_table", block_table, torch.int32)
    R = req_info.shape[0]
    _gpu("req_info", req_info, torch.int32, (R, 4))
    if block_table.dim() != 2 or block_table.shape[0] != R:
        raise KernelError("attention_mfma: block_table must be [requests, blocks]")
    n_parts = max(1, -(-int(max_ctx_len) // ATTN_PARTITION))
    if block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_mfma: block_table is narrower than the longest context")
    G = H // Hkv
    if blocks is None:
        if G > 16 * nb:
            raise KernelError("attention_mfma: without a block list a request's columns must fit one block")
        nblk = R
    else:
        nblk = blocks.shape[0]
        _gpu("blocks", blocks, torch.int32, (nblk, 2))
    _gpu("positions", positions, torch.int32, (T,))
    if nb not in (1, 2, 4) or (hd > 128 and nb == 4) or H % Hkv:
        raise KernelError(f"attention_mfma: unsupported column blocking nb={nb} for head size {hd}")
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    ws_o = torch.empty(T * H * n_parts * hd, dtype=torch.float32, device=q.device)
    ws_ml = torch.empty(T * H * n_parts * 2, dtype=torch.float32, device=q.device)
    _check(load("attention_mfma").tuff_attention_mfma(
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), ws_o.data_ptr(), ws_ml.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], None if blocks is None else blocks.data_ptr(), nblk, nb,
        req_info.data_ptr(), positions.data_ptr(), T, H, Hkv, hd, page_size,
        int(window or 0), float(scale), n_parts, _stream()), "attention_mfma")


def attention_decode_fused_supported(dtype, H: int, Hkv: int, hd: int, page_size: int, rotary_dim: int, interleaved: bool) -> bool:
    """A step of single tokens can go from the projected q/k/v rows to the attention output in one
    kernel and its merge: bfloat16, heads of 64 rotated whole in half-split pairs, at most sixteen
    query heads a kv head."""
    return (dtype == torch.bfloat16 and hd == 64 and rotary_dim == 64 and not interleaved and page_size % 16 == 0
            and H % Hkv == 0 and H // Hkv <= 16)


def attention_decode_fused(qkv, k_cache, v_cache, out, *, block_table, req_info, positions, inv_freq, H, Hkv, page_size,
                           max_ctx_len, slot_mapping=None, q_norm_w=None, k_norm_w=None, eps=0.0, window=0, scale=None,
                           angles=None) -> None:
    """Attention of a step in which every request has one token (row r of qkv is request r's), from the
    projected rows qkv [R, (H + 2 Hkv) * 64]: QK-norm, rotation, the write of the new key and value
    into the cache (slot_mapping; None: the cache is only read), attention over the cache, merge.
    angles: rope_table(inv_freq, n) or None; positions below n take their cosines and sines from it
    (computing them costs the kernel more than everything else it does for a short context)."""
    R = qkv.shape[0]
    hd = 64
    _gpu("qkv", qkv, torch.bfloat16, (R, (H + 2 * Hkv) * hd))
    _gpu("out", out, torch.bfloat16, (R, H * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, hd, page_size))
    _gpu("block_table", block_table, torch.int32)
    _gpu("req_info", req_info, torch.int32, (R, 4))
    _gpu("positions", positions, torch.int32, (R,))
    _opt("slot_mapping", slot_mapping, torch.int32, (R,))
    _gpu("inv_freq", inv_freq, torch.float32, (hd // 2,))
    _opt("angles", angles, torch.float32, (None, 2, hd // 2))
    if block_table.dim() != 2 or block_table.shape[0] != R:
        raise KernelError("attention_decode_fused: block_table must be [requests, blocks]")
    if block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_decode_fused: block_table is narrower than the longest context")
    if not attention_decode_fused_supported(qkv.dtype, H, Hkv, hd, page_size, hd, False):
        raise KernelError(f"attention_decode_fused: heads {H}:{Hkv} / page size {page_size} not supported")
    norm_dt = DT_F32
    if q_norm_w is not None or k_norm_w is not None:
        if q_norm_w is None or k_norm_w is None or q_norm_w.dtype != k_norm_w.dtype:
            raise KernelError("attention_decode_fused: q and k norm weights go together and share a dtype")
        _gpu("q_norm_w", q_norm_w, shape=(hd,))
        _gpu("k_norm_w", k_norm_w, shape=(hd,))
        norm_dt = _dt(q_norm_w)
    n_parts = max(1, -(-int(max_ctx_len) // ATTN_PARTITION))
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    ws_o = torch.empty(R * H * n_parts * hd, dtype=torch.float32, device=qkv.device)
    ws_ml = torch.empty(R * H * n_parts * 2, dtype=torch.float32, device=qkv.device)
    p = lambda t: None if t is None else t.data_ptr()
    _check(load("attention_mfma").tuff_attention_decode_fused(
        qkv.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), ws_o.data_ptr(), ws_ml.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], req_info.data_ptr(), positions.data_ptr(), p(slot_mapping),
        p(q_norm_w), p(k_norm_w), norm_dt, float(eps), inv_freq.data_ptr(), p(angles),
        0 if angles is None else angles.shape[0], R, H, Hkv, page_size,
        int(window or 0), float(scale), n_parts, _stream()), "attention_decode_fused")


def attention_prefill_block_columns(hd: int) -> int:
    """Columns (token, head in the kv group) a query block of attention_prefill holds."""
    return 128 if hd <= 128 else 64


PREFILL_WORKGROUP_SLOTS = 512    # workgroups of attention_prefill the part runs side by side (two a CU); with at most
                                 # half as many blocks the keys are cut into segments, a workgroup a segment
PREFILL_MIN_SEGMENT = 1024       # keys; shorter segments are not worth their merge


def attention_prefill(q, k_cache, v_cache, out, *, block_table, blocks, req_info,
                      H, Hkv, hd, page_size, max_ctx_len, window=0, scale=None, positions=None) -> None:
    """Matrix-core attention for steps with prompt portions: a workgroup walks over all keys of a
    block of query columns, keys and values staged through LDS; writes `out` directly.
    blocks: int32 [n_blocks, 2] from query_blocks(q_len, G, attention_prefill_block_columns(hd) // 16),
    or None when every request's columns fit one block (block b = request b).
    positions (int32 [T], optional): with them, a step with few blocks and long contexts (a short
    portion far into a long prompt) cuts the keys into segments, a workgroup a segment, and merges the
    segments' results as a step of single tokens merges its partitions.  Then every row of `out` is
    written, also those of tokens no block covers (with meaningless values)."""
    T = q.shape[0]
    if not attention_mfma_supported(q.dtype, hd, page_size):
        raise KernelError(f"attention_prefill: needs bfloat16, a head size that is a multiple of 8 (got {hd}) "
                          f"and a page size that is a multiple of 16 (got {page_size})")
    _gpu("q", q, torch.bfloat16, (T, H * hd))
    _gpu("out", out, torch.bfloat16, (T, H * hd))
    P = k_cache.shape[0]
    _gpu("k_cache", k_cache, torch.bfloat16, (P, Hkv, page_size, hd))
    _gpu("v_cache", v_cache, torch.bfloat16, (P, Hkv, hd, page_size))
    _gpu("block_table", block_table, torch.int32)
    R = req_info.shape[0]
    _gpu("req_info", req_info, torch.int32, (R, 4))
    if block_table.dim() != 2 or block_table.shape[0] != R:
        raise KernelError("attention_prefill: block_table must be [requests, blocks]")
    if block_table.shape[1] * page_size < int(max_ctx_len):
        raise KernelError("attention_prefill: block_table is narrower than the longest context")
    if H % Hkv:
        raise KernelError("attention_prefill: the query heads must be a multiple of the kv heads")
    G = H // Hkv
    if blocks is None:
        if G > attention_prefill_block_columns(hd):
            raise KernelError("attention_prefill: without a block list a request's columns must fit one block")
        nblk = R
    else:
        nblk = blocks.shape[0]
        _gpu("blocks", blocks, torch.int32, (nblk, 2))
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    n_segs, seg_keys, ws_o, ws_ml = 1, 0, None, None
    workgroups = nblk * Hkv
    if positions is not None and 0 < 2 * workgroups <= PREFILL_WORKGROUP_SLOTS and int(max_ctx_len) >= 2 * PREFILL_MIN_SEGMENT:
        # as many segments as fill the slots once, not more: what does not fit waits for a second round
        want = min(PREFILL_WORKGROUP_SLOTS // workgroups, int(max_ctx_len) // PREFILL_MIN_SEGMENT, 64)
        seg_keys = -(-(-(-int(max_ctx_len) // want)) // 64) * 64
        n_segs = -(-int(max_ctx_len) // seg_keys)
    if n_segs > 1:
        _gpu("positions", positions, torch.int32, (T,))
        ws_o = torch.empty(T * H * n_segs * hd, dtype=torch.float32, device=q.device)
        ws_ml = torch.empty(T * H * n_segs * 2, dtype=torch.float32, device=q.device)
    else:
        n_segs, seg_keys = 1, 0
    _check(load("attention_prefill").tuff_attention_prefill(
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], None if blocks is None else blocks.data_ptr(), nblk,
        req_info.data_ptr(), H, Hkv, hd, page_size, int(window or 0), float(scale), n_segs, seg_keys,
        None if ws_o is None else ws_o.data_ptr(), None if ws_ml is None else ws_ml.data_ptr(), _stream()), "attention_prefill")
    if n_segs > 1:
        _check(load("attention_mfma").tuff_attention_merge(ws_o.data_ptr(), ws_ml.data_ptr(), out.data_ptr(), positions.data_ptr(),
                                                           T, H, hd, int(window or 0), n_segs, seg_keys, _stream()),
               "attention_merge")


def query_blocks(q_len, G: int, nb: int, ctx_len=None):
    """Host list of query blocks for attention_mfma and attention_prefill: for request r with q_len[r]
    tokens the columns (token, head in group) are cut into blocks of 16 * nb.  Returns int32
    [n_blocks, 2] = (request, first column).  With ctx_len (tokens of each request in the cache after
    the step) the blocks whose last column sees the most keys come first (attention_prefill starts
    its workgroups in the list's order, and the longest should not start last); the order has no
    influence on any result."""
    import numpy as np
    q_len = np.asarray(q_len, dtype=np.int64)
    per = -(-(q_len * G) // (16 * nb))
    blk_req = np.repeat(np.arange(len(q_len)), per)
    starts = np.concatenate([[0], np.cumsum(per)])[:-1]
    blk_col0 = (np.arange(int(per.sum())) - np.repeat(starts, per)) * 16 * nb
    if ctx_len is not None and len(blk_req):
        ctx_len = np.asarray(ctx_len, dtype=np.int64)
        last_tok = np.minimum(q_len[blk_req] - 1, (blk_col0 + 16 * nb - 1) // G)
        keys = ctx_len[blk_req] - q_len[blk_req] + last_tok + 1
        order = np.argsort(-keys, kind="stable")
        blk_req, blk_col0 = blk_req[order], blk_col0[order]
    return np.stack([blk_req, blk_col0], axis=1).astype(np.int32)


# ------------------------------------------------------------------------- short conv
def shortconv_fwd(bcx, conv_w, state, out, *, req_of_token, q_start, state_slot, K, q_len=None) -> None:
    """The gated short convolution of a step's tokens, each request's earlier values from its state slot.
    With q_len (int32 [requests]) the state of every request with tokens in the step is rewritten too,
    as shortconv_state would afterwards; without, the state is only read."""
    T, d = out.shape
    dt = out.dtype
    _gpu("bcx", bcx, dt, (T, 3 * d))
    _gpu("out", out)
    _gpu("conv_w", conv_w, shape=(d, K))
    _gpu("state", state, torch.float32, (None, K - 1, d))
    R = q_start.shape[0]
    _gpu("req_of_token", req_of_token, torch.int32, (T,))
    _gpu("q_start", q_start, torch.int32, (R,))
    _gpu("state_slot", state_slot, torch.int32, (R,))
    if q_len is not None:
        _gpu("q_len", q_len, torch.int32, (R,))
    _check(load("shortconv").tuff_shortconv_fwd(
        bcx.data_ptr(), conv_w.data_ptr(), _dt(conv_w), state.data_ptr(), out.data_ptr(), _dt(out),
        req_of_token.data_ptr(), q_start.data_ptr(), None if q_len is None else q_len.data_ptr(), state_slot.data_ptr(),
        T, d, K, _stream()), "shortconv_fwd")


def shortconv_decode(bcx, conv_w, state, out, *, state_slot, K) -> None:
    """Output and state update in one kernel for a step in which every request has one token
    (row r of bcx is request r's token)."""
    R, d = out.shape
    dt = out.dtype
    _gpu("bcx", bcx, dt, (R, 3 * d))
    _gpu("out", out)
    _gpu("conv_w", conv_w, shape=(d, K))
    _gpu("state", state, torch.float32, (None, K - 1, d))
    _gpu("state_slot", state_slot, torch.int32, (R,))
    _check(load("shortconv").tuff_shortconv_decode(
        bcx.data_ptr(), conv_w.data_ptr(), _dt(conv_w), state.data_ptr(), out.data_ptr(), _dt(out),
        state_slot.data_ptr(), R, d, K, _stream()), "shortconv_decode")


def shortconv_state(bcx, state, *, q_start, q_len, state_slot, K) -> None:
    d = state.shape[2]
    R = q_start.shape[0]
    _gpu("bcx", bcx, shape=(None, 3 * d))
    _gpu("state", state, torch.float32, (None, K - 1, d))
    _gpu("q_start", q_start, torch.int32, (R,))
    _gpu("q_len", q_len, torch.int32, (R,))
    _gpu("state_slot", state_slot, torch.int32, (R,))
    _check(load("shortconv").tuff_shortconv_state(
        bcx.data_ptr(), _dt(bcx), state.data_ptr(), q_start.data_ptr(), q_len.data_ptr(),
        state_slot.data_ptr(), R, d, K, _stream()), "shortconv_state")


# --------------------------------------------------------------------------- sampling
def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    R, V = logits.shape
    _check(load("sampling").tuff_argmax(_gpu("logits", logits, torch.float32), _gpu("out", out, torch.int32, (R,)),
                                        R, V, _stream()), "argmax")


def sample(logits, out, *, temps=None, top_ks=None, top_ps=None, min_ps=None, uniforms=None) -> None:
    """One token per row: greedy where temps[r] <= 0 (or temps is None), else the reference's
    chain min-p -> top-k -> top-p -> draw with the host-supplied uniform of that row."""
    R, V = logits.shape
    _gpu("logits", logits, torch.float32)
    _gpu("out", out, torch.int32, (R,))
    if temps is not None and uniforms is None:
        raise KernelError("sample: stochastic rows need uniforms")
    p = lambda n, t, dt: None if t is None else _gpu(n, t, dt, (R,))
    _check(load("sampling").tuff_sample(
        logits.data_ptr(), p("temps", temps, torch.float32), p("top_ks", top_ks, torch.int32),
        p("top_ps", top_ps, torch.float32), p("min_ps", min_ps, torch.float32),
        p("uniforms", uniforms, torch.float32), out.data_ptr(), R, V, _stream()), "sample")


def repeat_penalty(logits, recent, counts, penalties) -> None:
    """In place: each row's logits penalised once per entry of its ring of recent tokens."""
    R, V = logits.shape
    cap = recent.shape[1]
    _gpu("logits", logits, torch.float32)
    _gpu("recent", recent, torch.int32, (R, cap))
    _gpu("counts", counts, torch.int32, (R,))
    _gpu("penalties", penalties, torch.float32, (R,))
    _check(load("sampling").tuff_repeat_penalty(logits.data_ptr(), recent.data_ptr(), counts.data_ptr(),
                                                penalties.data_ptr(), R, cap, V, _stream()), "repeat_penalty")
