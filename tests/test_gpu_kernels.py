"""Each HIP kernel alone against a plain float64 reference, at sizes the engine's models do
not use (odd widths, head sizes from 16 to 256, several page sizes)."""
import math

import numpy as np
import pytest
import torch

from plain import lfm2_plain as plain

pytestmark = pytest.mark.gpu


def _r(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ------------------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 100, 33), (65, 130, 17), (130, 65, 250), (64, 64, 64)])
def test_gemm_f32(gpu, M, N, K):
    from tuff_amd.csrc import ops
    x, w = _r(M, K, seed=1), _r(N, K, seed=2)
    y0 = _r(M, N, seed=3)
    want = x.double() @ w.double().T
    out = torch.empty(M, N, device=gpu)
    ops.gemm(x.to(gpu), w.to(gpu), out)
    bound = 4e-7 * K * x.abs().max() * w.abs().max()
    assert (out.cpu().double() - want).abs().max() <= bound
    acc = y0.to(gpu)
    ops.gemm(x.to(gpu), w.to(gpu), acc, accumulate=True)
    assert (acc.cpu().double() - (want + y0.double())).abs().max() <= bound + 1e-6
    # a row does not depend on the other rows of the call
    if M > 1:
        one = torch.empty(1, N, device=gpu)
        ops.gemm(x[M - 1:].to(gpu), w.to(gpu), one)
        assert torch.equal(one[0], out[M - 1])


@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (5, 1000, 96), (17, 33, 40), (64, 777, 240), (65, 130, 136),
                                   (200, 300, 328), (300, 64, 2048), (128, 128, 64), (2, 2048, 8192),
                                   (72, 2048, 8192), (512, 2050, 2048), (130, 1026, 1000),
                                   (33, 100, 2048), (64, 2048, 8192), (20, 64, 1024), (48, 200, 512), (16, 24, 4096),
                                   (8, 6144, 2048), (32, 6144, 2048), (24, 2048, 8192), (31, 40, 72), (32, 16400, 2048),
                                   # each shape of block of the tiled kernel, with ragged edges and a partial last step
                                   (1100, 8200, 72), (1030, 8190, 136), (1100, 4001, 200), (257, 129, 520),
                                   # the same with K a multiple of 64: operands go straight into LDS
                                   (1100, 8200, 192), (1030, 8190, 128), (1100, 4001, 256), (257, 129, 512), (100, 40, 64),
                                   # few blocks and a short K: blocks of 64 x 64, ragged in M and N
                                   (200, 1000, 1536), (65, 70, 3072), (500, 1536, 1536), (130, 2049, 320),
                                   # 17 to 64 rows, a wide output and a short K: blocks of 64 x 64 of the tiled kernel
                                   (17, 9216, 128), (40, 16390, 2048), (64, 24576, 192), (33, 10240, 3072)])
def test_gemm_bf16(gpu, M, N, K):
    from tuff_amd.csrc import ops
    x, w = _r(M, K, seed=4, dtype=torch.bfloat16), _r(N, K, seed=5, dtype=torch.bfloat16)
    want = x.double() @ w.double().T
    scale = float(want.abs().max())
    f32 = torch.empty(M, N, device=gpu)
    ops.gemm(x.to(gpu), w.to(gpu), f32)
    assert (f32.cpu().double() - want).abs().max() <= 1e-5 * scale + 1e-6 * K
    b16 = torch.empty(M, N, device=gpu, dtype=torch.bfloat16)
    ops.gemm(x.to(gpu), w.to(gpu), b16)
    assert (b16.cpu().double() - want).abs().max() <= 2 ** -8 * scale
    y0 = _r(M, N, seed=6)
    acc = y0.to(gpu)
    ops.gemm(x.to(gpu), w.to(gpu), acc, accumulate=True)
    assert (acc.cpu().double() - (want + y0.double())).abs().max() <= 1e-5 * scale + 1e-6 * K
    # the same call again gives the same bits (split-K partials are added in a fixed order), and
    # among M <= 16 a row does not depend on the other rows of the call
    again = torch.empty(M, N, device=gpu)
    ops.gemm(x.to(gpu), w.to(gpu), again)
    assert torch.equal(again, f32)
    if 1 < M <= 16:
        one = torch.empty(1, N, device=gpu)
        ops.gemm(x[M - 1:].to(gpu), w.to(gpu), one)
        assert torch.equal(one[0], f32[M - 1])


@pytest.mark.parametrize("M,N,K", [(1, 32, 64), (8, 512, 240), (16, 6144, 2048), (5, 200, 96), (64, 384, 256),
                                   (40, 2050, 2048), (24, 2050, 2048), (32, 16384, 2048), (300, 130, 136), (2048, 512, 128), (1100, 8200, 72),
                                   (200, 384, 1024), (72, 4100, 2048),
                                   (1030, 8202, 136), (1100, 4002, 200), (1030, 8202, 128), (1100, 4002, 192), (120, 13826, 1536),
                                   (17, 16384, 2048), (64, 13824, 1536), (25, 12290, 640)])
def test_gemm_bf16_swiglu_epilogue(gpu, M, N, K):
    """Rows of w are gate and up rows interleaved; the output is silu(gate) * up."""
    from tuff_amd.csrc import ops
    x, w = _r(M, K, seed=4, dtype=torch.bfloat16), _r(N, K, seed=5, dtype=torch.bfloat16)
    y = x.double() @ w.double().T
    g, u = y[:, 0::2], y[:, 1::2]
    want = g / (1 + torch.exp(-g)) * u
    out = torch.empty(M, N // 2, device=gpu, dtype=torch.bfloat16)
    ops.gemm(x.to(gpu), w.to(gpu), out, swiglu=True)
    assert (out.cpu().double() - want).abs().max() <= 2 ** -8 * float(want.abs().max()) + 1e-4 * K ** 0.5


@pytest.mark.parametrize("M,N,K", [(1, 16, 64), (8, 6144, 2048), (16, 130, 240), (3, 1000, 96), (7, 65536, 2048), (2, 48, 8192)])
@pytest.mark.parametrize("use_rows", [False, True])
def test_gemm_with_the_norm_inside(gpu, M, N, K, use_rows):
    """y = rmsnorm(x) w^T in one kernel equals the norm kernel followed by the product, to the
    rounding of the bfloat16 operand, and is close to the float64 value."""
    from tuff_amd.csrc import ops
    n_x = M + 3 if use_rows else M
    x = _r(n_x, K, seed=1, scale=2.0)
    nw = 1 + _r(K, seed=2, scale=0.1)
    w = _r(N, K, seed=3, scale=0.05, dtype=torch.bfloat16)
    rows = torch.randperm(n_x, generator=torch.Generator().manual_seed(4))[:M].to(torch.int32) if use_rows else None
    xs = x[rows.long()] if use_rows else x
    eps = 1e-5
    want = plain.rms_norm(xs.double(), nw.double(), eps) @ w.double().T
    out = torch.empty(M, N, device=gpu)
    ops.gemm_normed(x.to(gpu), nw.to(gpu), eps, w.to(gpu), out, rows=None if rows is None else rows.to(gpu))
    scale = float(want.abs().max())
    assert (out.cpu().double() - want).abs().max() <= 2 ** -7 * scale
    # accumulate and swiglu epilogues
    y0 = _r(M, N, seed=6)
    acc = y0.to(gpu)
    ops.gemm_normed(x.to(gpu), nw.to(gpu), eps, w.to(gpu), acc, rows=None if rows is None else rows.to(gpu), accumulate=True)
    assert (acc.cpu().double() - (want + y0.double())).abs().max() <= 2 ** -7 * scale
    sw = torch.empty(M, N // 2, device=gpu, dtype=torch.bfloat16)
    ops.gemm_normed(x.to(gpu), nw.to(gpu), eps, w.to(gpu), sw, rows=None if rows is None else rows.to(gpu), swiglu=True)
    g, u = want[:, 0::2], want[:, 1::2]
    ref = g / (1 + torch.exp(-g)) * u
    assert (sw.cpu().double() - ref).abs().max() <= 2 ** -6 * max(float(ref.abs().max()), scale * 0.1)
    # a row does not depend on the other rows of the call
    if M > 1:
        one = torch.empty(1, N, device=gpu)
        r1 = (rows[M - 1:] if use_rows else torch.tensor([M - 1], dtype=torch.int32)).to(gpu)
        ops.gemm_normed(x.to(gpu), nw.to(gpu), eps, w.to(gpu), one, rows=r1)
        assert torch.equal(one[0], out[M - 1])


@pytest.mark.parametrize("M,d,K1,N2", [(1, 64, 192, 512), (8, 2048, 8192, 6144), (16, 240, 328, 777 * 2), (5, 96, 96, 40),
                                       (17, 96, 96, 40), (32, 2048, 8192, 6144), (24, 240, 328, 777 * 2), (40, 2048, 8192, 6144), (64, 240, 328, 777 * 2), (33, 64, 192, 512),
                                       (64, 2048, 2048, 65536),
                                       # the product that follows is wide with a short K: the tiled kernel reads these row sums
                                       (17, 192, 96, 9216), (40, 2048, 2048, 16384), (64, 1536, 512, 13824), (25, 128, 64, 10242),
                                       # ... and the residual stream itself is that wide
                                       (20, 9216, 128, 512), (40, 10240, 64, 96),
                                       # 33 to 64 rows of a medium-wide residual stream
                                       (48, 2304, 512, 3072), (64, 4096, 256, 4096), (33, 2064, 96, 2100)])
def test_gemm_that_prepares_the_next_norm(gpu, M, d, K1, N2):
    """residual += a @ w1.T leaves bf16(residual * norm weight) and per-tile row sums of squares;
    the next product scales its rows by them: together rmsnorm(residual) @ w2.T."""
    from tuff_amd.csrc import ops
    a = _r(M, K1, seed=1, dtype=torch.bfloat16)
    w1 = _r(d, K1, seed=2, scale=0.05, dtype=torch.bfloat16)
    res0 = _r(M, d, seed=3)
    nw = 1 + _r(d, seed=4, scale=0.1)
    w2 = _r(N2, d, seed=5, scale=0.05, dtype=torch.bfloat16)
    eps = 1e-5
    res = res0.to(gpu)
    xw = torch.empty(M, d, dtype=torch.bfloat16, device=gpu)
    ss = torch.full(ops.gemm_emit_layout(M, d, K1), float("nan"), device=gpu)
    ops.gemm_accum_emit(a.to(gpu), w1.to(gpu), res, nw.to(gpu), xw, ss)
    want_res = res0.double() + a.double() @ w1.double().T
    assert (res.cpu().double() - want_res).abs().max() <= 1e-5 * float(want_res.abs().max()) + 1e-6 * K1
    plain_acc = res0.to(gpu)
    ops.gemm(a.to(gpu), w1.to(gpu), plain_acc, accumulate=True)
    assert torch.equal(plain_acc, res)                       # the residual itself is what the plain product gives
    assert (xw.cpu().double() - want_res * nw.double()).abs().max() <= 2 ** -8 * float((want_res * nw).abs().max())
    assert (ss.cpu().double()[:, :M].sum(0) - (want_res ** 2).sum(1)).abs().max() <= 1e-4 * float((want_res ** 2).sum(1).max())
    want = plain.rms_norm(want_res, nw.double(), eps) @ w2.double().T
    out = torch.empty(M, N2, device=gpu)
    ops.gemm_scaled(xw, ss, eps, w2.to(gpu), out)
    assert (out.cpu().double() - want).abs().max() <= 2 ** -7 * float(want.abs().max())
    sw = torch.empty(M, N2 // 2, device=gpu, dtype=torch.bfloat16)
    ops.gemm_scaled(xw, ss, eps, w2.to(gpu), sw, swiglu=True)
    g, u = want[:, 0::2], want[:, 1::2]
    ref = g / (1 + torch.exp(-g)) * u
    assert (sw.cpu().double() - ref).abs().max() <= 2 ** -6 * max(float(ref.abs().max()), 0.1 * float(want.abs().max()))


@pytest.mark.parametrize("M,d,K1,N2", [(2048, 2048, 2048, 6144), (1000, 2048, 8192, 3072), (130, 256, 128, 512),
                                       (700, 1536, 6912, 13824), (4096, 2048, 2048, 16384), (65, 192, 64, 384),
                                       (512, 2040, 8192, 2048), (300, 256, 8192, 512)])
def test_tiled_gemm_that_prepares_the_next_norm(gpu, M, d, K1, N2):
    """The same for more than 64 rows (the tiled product): each wave of the accumulating product leaves the
    sums of squares of its rows over its columns, and the next product scales its rows."""
    from tuff_amd.csrc import ops
    a = _r(M, K1, seed=1, dtype=torch.bfloat16)
    w1 = _r(d, K1, seed=2, scale=K1 ** -0.5, dtype=torch.bfloat16)
    res0 = _r(M, d, seed=3)
    nw = 1 + _r(d, seed=4, scale=0.1)
    w2 = _r(N2, d, seed=5, scale=d ** -0.5, dtype=torch.bfloat16)
    eps = 1e-5
    layout = ops.gemm_emit_layout(M, d, K1)
    assert layout is not None and layout[1] == M
    res = res0.to(gpu)
    xw = torch.empty(M, d, dtype=torch.bfloat16, device=gpu)
    ss = torch.full(layout, float("nan"), device=gpu)
    ops.gemm_accum_emit(a.to(gpu), w1.to(gpu), res, nw.to(gpu), xw, ss)
    plain_acc = res0.to(gpu)
    ops.gemm(a.to(gpu), w1.to(gpu), plain_acc, accumulate=True)
    assert torch.equal(plain_acc, res)                       # the residual itself is what the plain product gives
    got_res = res.cpu().double()
    assert (xw.cpu().double() - got_res * nw.double()).abs().max() <= 2 ** -8 * float((got_res * nw).abs().max())
    assert (ss.cpu().double().sum(0) - (got_res ** 2).sum(1)).abs().max() <= 1e-5 * float((got_res ** 2).sum(1).max())
    want = plain.rms_norm(got_res, nw.double(), eps) @ w2.double().T
    assert ops.gemm_scaled_supported(M, N2, d) and not ops.gemm_scaled_supported(M, N2, d, torch.float32)
    out = torch.empty(M, N2, dtype=torch.bfloat16, device=gpu)
    ops.gemm_scaled(xw, ss, eps, w2.to(gpu), out)
    assert (out.cpu().double() - want).abs().max() <= 2 ** -6 * float(want.abs().max())
    sw = torch.empty(M, N2 // 2, device=gpu, dtype=torch.bfloat16)
    ops.gemm_scaled(xw, ss, eps, w2.to(gpu), sw, swiglu=True)
    g, u = want[:, 0::2], want[:, 1::2]
    ref = g / (1 + torch.exp(-g)) * u
    assert (sw.cpu().double() - ref).abs().max() <= 2 ** -5 * max(float(ref.abs().max()), 0.1 * float(want.abs().max()))


def test_products_that_cannot_prepare_the_next_norm_say_so(gpu):
    from tuff_amd.csrc import ops
    assert ops.gemm_emit_layout(300, 2048, 8192) == (32, 300)     # cut into slices: the kernel that adds them emits
    assert ops.gemm_emit_layout(500, 200, 256) is None            # a last block of columns that is not whole
    assert ops.gemm_emit_layout(500, 256, 136) is None            # K no multiple of 64
    assert not ops.gemm_scaled_supported(500, 256, 136) and ops.gemm_scaled_supported(300, 2048, 8192)
    with pytest.raises(ops.KernelError, match="cannot leave"):
        ops.gemm_accum_emit(torch.zeros(500, 136, dtype=torch.bfloat16, device=gpu), torch.zeros(256, 136, dtype=torch.bfloat16, device=gpu),
                            torch.zeros(500, 256, device=gpu), torch.ones(256, device=gpu),
                            torch.empty(500, 256, dtype=torch.bfloat16, device=gpu), torch.empty(4, 500, device=gpu))


def test_gemm_refuses_what_it_cannot_do(gpu):
    from tuff_amd.csrc import ops
    x = torch.zeros(2, 12, dtype=torch.bfloat16, device=gpu)
    w = torch.zeros(4, 12, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ops.KernelError, match="multiple of 8"):
        ops.gemm(x, w, torch.empty(2, 4, device=gpu))
    with pytest.raises(ops.KernelError, match="no CPU fallback"):
        ops.gemm(torch.zeros(2, 8), torch.zeros(4, 8), torch.zeros(2, 4))
    x16 = torch.zeros(2, 16, dtype=torch.bfloat16, device=gpu)
    w16 = torch.zeros(4, 16, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ops.KernelError, match="expected shape"):
        ops.gemm(x16, w16, torch.empty(3, 4, device=gpu))
    with pytest.raises(ops.KernelError, match="at most 16 rows"):
        ops.gemm_normed(torch.zeros(17, 16, device=gpu), torch.ones(16, device=gpu), 1e-5, w16, torch.empty(17, 4, device=gpu))


# ------------------------------------------------------------------------- row kernels
@pytest.mark.parametrize("n,d", [(5, 64), (3, 777), (1, 2048), (9, 240)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(gpu, n, d, out_dtype):
    from tuff_amd.csrc import ops
    x, w = _r(n, d, seed=7, scale=3.0), 1 + _r(d, seed=8, scale=0.1)
    for eps in (1e-5, 0.5):
        want = plain.rms_norm(x.double(), w.double(), eps)
        out = torch.empty(n, d, device=gpu, dtype=out_dtype)
        ops.rmsnorm(x.to(gpu), w.to(gpu), out, eps)
        tol = 1e-5 if out_dtype == torch.float32 else 2 ** -8 * float(want.abs().max())
        assert (out.cpu().double() - want).abs().max() <= tol
    rows = torch.tensor([n - 1, 0], dtype=torch.int32)
    out = torch.empty(2, d, device=gpu, dtype=out_dtype)
    ops.rmsnorm(x.to(gpu), w.to(torch.bfloat16).to(gpu), out, 1e-5, rows.to(gpu))
    want = plain.rms_norm(x.double(), w.to(torch.bfloat16).double(), 1e-5)[rows.long()]
    assert (out.cpu().double() - want).abs().max() <= (1e-5 if out_dtype == torch.float32 else 2 ** -8 * float(want.abs().max()))


def test_embed_and_swiglu(gpu):
    from tuff_amd.csrc import ops
    table = _r(50, 24, seed=9, dtype=torch.bfloat16)
    toks = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    out = torch.empty(4, 24, device=gpu)
    ops.embed_rows(table.to(gpu), toks.to(gpu), out)
    assert torch.equal(out.cpu(), table[toks.long()].float())
    ops.embed_rows(table.to(gpu), toks.to(gpu), out, scale=1.5)
    assert torch.equal(out.cpu(), table[toks.long()].float() * 1.5)
    # a bias onto rows of either type, and logits scaled under a soft cap
    bias = _r(24, seed=12)
    for dt in (torch.float32, torch.bfloat16):
        y = _r(5, 24, seed=11, dtype=dt)
        got = y.to(gpu)
        ops.add_bias(got, bias.to(gpu))
        assert torch.equal(got.cpu(), (y.float() + bias).to(dt))
    x = _r(3, 37, seed=13, scale=4.0)
    got = x.to(gpu)
    ops.scale_cap(got, 0.5, 1.25)
    assert (got.cpu().double() - 1.25 * torch.tanh(x.double() * 0.5 / 1.25)).abs().max() < 1e-6
    got = x.to(gpu)
    ops.scale_cap(got, 2.0)
    assert torch.equal(got.cpu(), x * 2.0)
    for dt in (torch.float32, torch.bfloat16):
        gu = _r(7, 2 * 13, seed=10, scale=2.0, dtype=dt)
        act = torch.empty(7, 13, device=gpu, dtype=dt)
        ops.swiglu(gu.to(gpu), act)
        g, u = gu[:, :13].double(), gu[:, 13:].double()
        want = g / (1 + torch.exp(-g)) * u
        assert (act.cpu().double() - want).abs().max() <= (1e-6 if dt == torch.float32 else 2 ** -8 * float(want.abs().max()))
    z = torch.zeros(2, 8, device=gpu)
    ops.swiglu(torch.zeros(2, 16, device=gpu), z)
    assert (z == 0).all()                                # g = 0 gives 0


# --------------------------------------------------------------- q/k/v post-processing
def _interleaved_rope(x, pos, base):
    hd = x.shape[-1]
    j = torch.arange(hd // 2, dtype=torch.float64)
    a = pos.double()[:, None] * base ** (-2 * j / hd)
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = x0 * c - x1 * s
    out[..., 1::2] = x0 * s + x1 * c
    return out


@pytest.mark.parametrize("H,Hkv,hd,ps", [(4, 2, 16, 16), (4, 1, 24, 8), (3, 3, 80, 16), (2, 1, 256, 4), (5, 5, 128, 64)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_qkv_post(gpu, H, Hkv, hd, ps, dt):
    from tuff_amd.csrc import ops
    T, eps, base = 11, 1e-5, 10000.0
    qkv = _r(T, (H + 2 * Hkv) * hd, seed=11, dtype=dt)
    qw, kw = 1 + _r(hd, seed=12, scale=0.1), 1 + _r(hd, seed=13, scale=0.1)
    pos = torch.tensor([0, 1, 2, 3, 100, 101, 7, 8, 9, 1000, 31], dtype=torch.int32)
    n_pages = 8
    slots = torch.randperm(n_pages * ps, generator=torch.Generator().manual_seed(1))[:T].to(torch.int32)
    j = torch.arange(hd // 2, dtype=torch.float64)
    inv_freq = (base ** (-2 * j / hd)).float()
    kc = torch.zeros(n_pages, Hkv, ps, hd, dtype=dt, device=gpu)
    vc = torch.zeros(n_pages, Hkv, hd, ps, dtype=dt, device=gpu)
    q = torch.empty(T, H * hd, dtype=dt, device=gpu)
    ops.qkv_post(qkv.to(gpu), q, H=H, Hkv=Hkv, hd=hd, positions=pos.to(gpu), eps=eps, q_norm_w=qw.to(gpu),
                 k_norm_w=kw.to(gpu), inv_freq=inv_freq.to(gpu), rotary_dim=hd, k_cache=kc, v_cache=vc,
                 slot_mapping=slots.to(gpu), page_size=ps)
    x = qkv.double()
    qs, ks, vs = x[:, :H * hd].reshape(T, H, hd), x[:, H * hd:(H + Hkv) * hd].reshape(T, Hkv, hd), x[:, (H + Hkv) * hd:].reshape(T, Hkv, hd)
    want_q = plain.rope_neox(plain.rms_norm(qs, qw.double(), eps), pos, base)
    want_k = plain.rope_neox(plain.rms_norm(ks, kw.double(), eps), pos, base)
    # float32 angles: pos * theta carries a relative error of 2^-24, so 1000 rad is known to 6e-5
    tol = 2e-4 if dt == torch.float32 else 2 ** -7
    assert (q.cpu().double().reshape(T, H, hd) - want_q).abs().max() <= tol * float(want_q.abs().max())
    got_k = kc.cpu().double().permute(0, 2, 1, 3).reshape(n_pages * ps, Hkv, hd)[slots.long()]
    got_v = vc.cpu().double().permute(0, 3, 1, 2).reshape(n_pages * ps, Hkv, hd)[slots.long()]
    assert (got_k - want_k).abs().max() <= tol * float(want_k.abs().max())
    assert torch.equal(got_v, vs)
    # nothing else in the cache was touched
    untouched = torch.ones(n_pages * ps, dtype=torch.bool)
    untouched[slots.long()] = False
    assert (kc.cpu().permute(0, 2, 1, 3).reshape(n_pages * ps, -1)[untouched] == 0).all()
    # interleaved pairs, no norm, partial rotary dim
    rd = hd // 2 if (hd // 2) % 2 == 0 else hd
    q2 = torch.empty(T, H * hd, dtype=dt, device=gpu)
    k2 = torch.empty(T, Hkv * hd, dtype=dt, device=gpu)
    jf = torch.arange(rd // 2, dtype=torch.float64)
    ops.qkv_post(qkv.to(gpu), q2, H=H, Hkv=Hkv, hd=hd, positions=pos.to(gpu), k_out=k2,
                 inv_freq=(base ** (-2 * jf / rd)).float().to(gpu), rotary_dim=rd, interleaved=True)
    want = qs.clone()
    want[..., :rd] = _interleaved_rope(qs[..., :rd], pos, base)
    assert (q2.cpu().double().reshape(T, H, hd) - want).abs().max() <= tol * float(want.abs().max())
    wantk = ks.clone()
    wantk[..., :rd] = _interleaved_rope(ks[..., :rd], pos, base)
    assert (k2.cpu().double().reshape(T, Hkv, hd) - wantk).abs().max() <= tol * float(wantk.abs().max())


@pytest.mark.parametrize("ps", [16, 32, 64])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_qkv_post_heads_of_64(gpu, dt, ps):
    """The kernel for heads of 64 channels: sixteen lanes a token, v rows of sixteen tokens written in
    runs.  Slots as a prompt gives them (runs of whole pages from a page's start), runs that begin in
    the middle of a page, scattered slots, a last group of fewer than sixteen tokens, slots that are
    not to be written; against the plain formulas, and bit for bit against the same tokens in steps
    of 1, 5 and 16."""
    from tuff_amd.csrc import ops
    H, Hkv, hd, eps, base = 6, 3, 64, 1e-6, 1000000.0
    T = 16 * 7 + 5
    qkv = _r(T, (H + 2 * Hkv) * hd, seed=21, dtype=dt)
    qw, kw = 1 + _r(hd, seed=22, scale=0.1), 1 + _r(hd, seed=23, scale=0.1)
    pos = (torch.arange(T, dtype=torch.int32) * 3 + 2) % 1500
    n_pages = 40
    slots = torch.empty(T, dtype=torch.int64)
    slots[0:32] = torch.arange(32) + 5 * ps                 # two whole groups from a page's start
    slots[32:48] = torch.arange(16) + 9 * ps + 8             # a run that begins in the middle of a page
    slots[48:64] = torch.randperm(16, generator=torch.Generator().manual_seed(2)) + 11 * ps   # one page, shuffled
    slots[64:112] = torch.arange(48) + 20 * ps               # pages in a row
    slots[112:] = torch.arange(5) + 30 * ps                  # the last, short group
    write = torch.ones(T, dtype=torch.bool)
    write[70] = False
    slot_arg = torch.where(write, slots, torch.full_like(slots, -1)).to(torch.int32)
    inv_freq = (base ** (-2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float()
    dev = lambda x: x.to(gpu)

    def run(step):
        kc = torch.zeros(n_pages, Hkv, ps, hd, dtype=dt, device=gpu)
        vc = torch.zeros(n_pages, Hkv, hd, ps, dtype=dt, device=gpu)
        q = torch.empty(T, H * hd, dtype=dt, device=gpu)
        for a in range(0, T, step):
            b = min(T, a + step)
            ops.qkv_post(dev(qkv[a:b]), q[a:b], H=H, Hkv=Hkv, hd=hd, positions=dev(pos[a:b]), eps=eps, q_norm_w=dev(qw),
                         k_norm_w=dev(kw), inv_freq=dev(inv_freq), rotary_dim=hd, k_cache=kc, v_cache=vc,
                         slot_mapping=dev(slot_arg[a:b]), page_size=ps)
        return q, kc, vc
    q, kc, vc = run(T)
    x = qkv.double()
    qs, ks, vs = x[:, :H * hd].reshape(T, H, hd), x[:, H * hd:(H + Hkv) * hd].reshape(T, Hkv, hd), x[:, (H + Hkv) * hd:].reshape(T, Hkv, hd)
    want_q = plain.rope_neox(plain.rms_norm(qs, qw.double(), eps), pos, base)
    want_k = plain.rope_neox(plain.rms_norm(ks, kw.double(), eps), pos, base)
    tol = 2e-4 if dt == torch.float32 else 2 ** -7
    assert (q.cpu().double().reshape(T, H, hd) - want_q).abs().max() <= tol * float(want_q.abs().max())
    flat_k = kc.cpu().double().permute(0, 2, 1, 3).reshape(n_pages * ps, Hkv, hd)
    flat_v = vc.cpu().double().permute(0, 3, 1, 2).reshape(n_pages * ps, Hkv, hd)
    assert (flat_k[slots[write]] - want_k[write]).abs().max() <= tol * float(want_k.abs().max())
    assert torch.equal(flat_v[slots[write]], vs[write])
    untouched = torch.ones(n_pages * ps, dtype=torch.bool)
    untouched[slots[write]] = False
    assert (flat_k[untouched] == 0).all() and (flat_v[untouched] == 0).all()
    for step in (1, 5, 16):
        q2, k2, v2 = run(step)
        assert torch.equal(q, q2) and torch.equal(kc, k2) and torch.equal(vc, v2), f"steps of {step} differ"


@pytest.mark.parametrize("H,Hkv,hd,rot,inter", [(6, 3, 64, 64, False), (4, 2, 80, 80, False), (3, 1, 48, 32, True), (2, 2, 128, 64, False)])
def test_qkv_post_with_a_table_of_angles_gives_the_same_bits(gpu, H, Hkv, hd, rot, inter):
    """Cosines and sines taken from rope_table() instead of computed in the kernel: the same queries and
    the same cache, bit for bit, also for positions beyond the table's end."""
    from tuff_amd.csrc import ops
    T, ps, dt = 150, 16, torch.bfloat16
    qkv = _r(T, (H + 2 * Hkv) * hd, seed=31, dtype=dt).to(gpu)
    qw, kw = (1 + _r(hd, seed=32, scale=0.1)).to(gpu), (1 + _r(hd, seed=33, scale=0.1)).to(gpu)
    pos = ((torch.arange(T, dtype=torch.int32) * 37) % 3000).to(gpu)
    slots = torch.randperm(T + 10, generator=torch.Generator().manual_seed(4))[:T].to(torch.int32).to(gpu)
    inv_freq = (1e6 ** (-2 * torch.arange(rot // 2, dtype=torch.float64) / rot)).float().to(gpu)
    table = ops.rope_table(inv_freq, 2000)
    assert table.shape == (2000, 2, rot // 2)
    a = (torch.arange(2000, dtype=torch.float32, device=gpu)[:, None] * inv_freq[None]).double()
    assert (table[:, 0].double() - torch.cos(a)).abs().max() < 1e-6 and (table[:, 1].double() - torch.sin(a)).abs().max() < 1e-6
    outs = []
    for angles in (None, table):
        n_pages = (T + 10) // ps + 1
        kc = torch.zeros(n_pages, Hkv, ps, hd, dtype=dt, device=gpu)
        vc = torch.zeros(n_pages, Hkv, hd, ps, dtype=dt, device=gpu)
        q = torch.empty(T, H * hd, dtype=dt, device=gpu)
        ops.qkv_post(qkv, q, H=H, Hkv=Hkv, hd=hd, positions=pos, eps=1e-5, q_norm_w=qw, k_norm_w=kw, inv_freq=inv_freq,
                     rotary_dim=rot, interleaved=inter, k_cache=kc, v_cache=vc, slot_mapping=slots, page_size=ps, angles=angles)
        outs.append((q, kc, vc))
    assert all(torch.equal(x, y) for x, y in zip(*outs))


def test_qkv_post_many_tokens_equal_few(gpu):
    """With many tokens a wave takes several heads of a token in turn; the result is, bit for
    bit, that of the same tokens in small steps."""
    from tuff_amd.csrc import ops
    T, H, Hkv, hd, ps, dt = 3000, 7, 3, 48, 16, torch.bfloat16
    qkv = _r(T, (H + 2 * Hkv) * hd, seed=11, dtype=dt).to(gpu)
    qw, kw = (1 + _r(hd, seed=12, scale=0.1)).to(gpu), (1 + _r(hd, seed=13, scale=0.1)).to(gpu)
    pos = torch.arange(T, dtype=torch.int32, device=gpu) + 5
    slots = torch.randperm(T + 32, generator=torch.Generator().manual_seed(1))[:T].to(torch.int32).to(gpu)
    inv_freq = (10000.0 ** (-2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float().to(gpu)
    n_pages = (T + 32) // ps + 1

    def run(step):
        kc = torch.zeros(n_pages, Hkv, ps, hd, dtype=dt, device=gpu)
        vc = torch.zeros(n_pages, Hkv, hd, ps, dtype=dt, device=gpu)
        q = torch.empty(T, H * hd, dtype=dt, device=gpu)
        for a in range(0, T, step):
            b = min(T, a + step)
            ops.qkv_post(qkv[a:b], q[a:b], H=H, Hkv=Hkv, hd=hd, positions=pos[a:b], eps=1e-5, q_norm_w=qw, k_norm_w=kw,
                         inv_freq=inv_freq, rotary_dim=hd, k_cache=kc, v_cache=vc, slot_mapping=slots[a:b], page_size=ps)
        return q, kc, vc
    q1, k1, v1 = run(T)
    q2, k2, v2 = run(100)
    assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(v1, v2)


# -------------------------------------------------------------------------- attention
def _attention_reference(q, K, V, pos, window, scale):
    """q [H, hd]; K, V [n, Hkv, hd] of one request; keys lo..pos."""
    H, hd = q.shape
    g = H // K.shape[1]
    lo = max(0, pos - window + 1) if window else 0
    k = K[lo:pos + 1].repeat_interleave(g, dim=1)
    v = V[lo:pos + 1].repeat_interleave(g, dim=1)
    s = torch.einsum("hd,thd->ht", q, k) * scale
    p = torch.softmax(s, dim=-1)
    return torch.einsum("ht,thd->hd", p, v)


def _paged_case(gpu, dt, H, Hkv, hd, ps, lens, window, seed=0):
    """Requests of the given lengths with shuffled pages; queries for the last few tokens of each."""
    g = torch.Generator().manual_seed(seed)
    n_blocks = [-(-n // ps) for n in lens]
    n_pages = sum(n_blocks) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    kc = _r(n_pages, Hkv, ps, hd, seed=seed + 1, dtype=dt)
    vc = _r(n_pages, Hkv, hd, ps, seed=seed + 2, dtype=dt)           # V pages are [kv_head][hd][offset]
    maxb = max(n_blocks) + 1
    table = torch.full((len(lens), maxb), -1, dtype=torch.int32)
    Ks, Vs = [], []
    for r, nb in enumerate(n_blocks):
        pages = [perm.pop() for _ in range(nb)]
        table[r, :nb] = torch.tensor(pages, dtype=torch.int32)
        Ks.append(kc[pages].permute(0, 2, 1, 3).reshape(nb * ps, Hkv, hd).double())
        Vs.append(vc[pages].permute(0, 3, 1, 2).reshape(nb * ps, Hkv, hd).double())
    req, pos = [], []
    for r, n in enumerate(lens):
        for p in sorted({0, n // 2, max(0, n - 2), n - 1}):
            req.append(r)
            pos.append(p)
    T = len(req)
    q = _r(T, H * hd, seed=seed + 3, dtype=dt)
    return kc, vc, table, torch.tensor(req, dtype=torch.int32), torch.tensor(pos, dtype=torch.int32), q, Ks, Vs


@pytest.mark.parametrize("H,Hkv,hd,ps", [(4, 2, 16, 16), (4, 1, 24, 8), (3, 3, 80, 16), (2, 1, 256, 32),
                                          (8, 2, 64, 64), (6, 2, 128, 16), (1, 1, 48, 1)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_general(gpu, H, Hkv, hd, ps, dt, window):
    from tuff_amd.csrc import ops
    lens = [1, 63, 64, 65, 200, 130]
    kc, vc, table, req, pos, q, Ks, Vs = _paged_case(gpu, dt, H, Hkv, hd, ps, lens, window)
    out = torch.empty(q.shape, dtype=dt, device=gpu)
    ops.attention_general(q.to(gpu), kc.to(gpu), vc.to(gpu), out, block_table=table.to(gpu),
                          req_of_token=req.to(gpu), positions=pos.to(gpu), H=H, Hkv=Hkv, hd=hd,
                          page_size=ps, window=window)
    scale = 1 / math.sqrt(hd)
    for t in range(len(req)):
        want = _attention_reference(q[t].double().reshape(H, hd), Ks[req[t]], Vs[req[t]], int(pos[t]), window, scale)
        got = out[t].cpu().double().reshape(H, hd)
        tol = 2e-6 if dt == torch.float32 else 2 ** -7
        assert (got - want).abs().max() <= tol * max(1.0, float(want.abs().max())), (t, int(req[t]), int(pos[t]))


def _mixed_step_case(gpu, reqs, H, Hkv, hd, ps):
    """A step over requests given as (tokens already in the cache, tokens of this step), pages
    shuffled, stale pages full of NaN."""
    dt = torch.bfloat16
    n_blocks = [-(-(past + n) // ps) for past, n in reqs]
    n_pages = sum(n_blocks) + 2
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(7)).tolist()
    kc = torch.full((n_pages, Hkv, ps, hd), float("nan"), dtype=dt)
    vc = torch.full((n_pages, Hkv, hd, ps), float("nan"), dtype=dt)
    table = torch.full((len(reqs), max(n_blocks)), -1, dtype=torch.int32)
    Ks, Vs, q_start, q_len, pos = [], [], [], [], []
    for r, ((past, n), nb_) in enumerate(zip(reqs, n_blocks)):
        pages = torch.tensor([perm.pop() for _ in range(nb_)])
        table[r, :nb_] = pages.to(torch.int32)
        K = _r(past + n, Hkv, hd, seed=50 + r, dtype=dt)
        V = _r(past + n, Hkv, hd, seed=70 + r, dtype=dt)
        t = torch.arange(past + n)
        kc[pages[t // ps], :, t % ps, :] = K
        vc[pages[t // ps], :, :, t % ps] = V
        Ks.append(K.double())
        Vs.append(V.double())
        q_start.append(len(pos))
        q_len.append(n)
        pos += list(range(past, past + n))
    q = _r(len(pos), H * hd, seed=90, dtype=dt)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    req_info = i32([[qs, ql, past, past + ql] for qs, ql, (past, _) in zip(q_start, q_len, reqs)])
    return dict(kc=kc.to(gpu), vc=vc.to(gpu), table=table.to(gpu), q=q, Ks=Ks, Vs=Vs, q_len=q_len,
                positions=i32(pos), req_info=req_info, max_ctx_len=max(p + n for p, n in reqs))


def _check_step(case, reqs, got, H, hd, window, tag):
    scale = 1 / math.sqrt(hd)
    assert torch.isfinite(got).all(), tag
    t = 0
    for r, (past, n) in enumerate(reqs):
        for j in range(n):
            want = _attention_reference(case["q"][t].double().reshape(H, hd), case["Ks"][r], case["Vs"][r], past + j,
                                        window, scale)
            assert (got[t] - want).abs().max() <= 2 ** -6 * max(1.0, float(want.abs().max())), (tag, r, j)
            t += 1


@pytest.mark.parametrize("H,Hkv,hd,ps", [(4, 2, 16, 16), (4, 1, 24, 16), (3, 3, 80, 16), (2, 1, 256, 32),
                                          (32, 8, 64, 16), (8, 2, 128, 64), (32, 1, 64, 16), (5, 5, 40, 48)])
@pytest.mark.parametrize("window", [0, 37, 300])
def test_attention_mfma(gpu, H, Hkv, hd, ps, window):
    """A mixed step: a decoded token deep in a long request, a prompt portion in the middle of
    another, a whole short prompt, a first token.  Stale pages hold NaN."""
    from tuff_amd.csrc import ops
    reqs = [(699, 1), (230, 50), (0, 33), (0, 1), (255, 3), (511, 2)]
    case = _mixed_step_case(gpu, reqs, H, Hkv, hd, ps)
    T = case["q"].shape[0]
    for nb in ([1, 2, 4] if hd <= 128 else [1, 2]):
        blocks = torch.from_numpy(ops.query_blocks(case["q_len"], H // Hkv, nb)).to(gpu)
        out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        ops.attention_mfma(case["q"].to(gpu), case["kc"], case["vc"], out, block_table=case["table"],
                           blocks=blocks, nb=nb, req_info=case["req_info"], positions=case["positions"], H=H, Hkv=Hkv,
                           hd=hd, page_size=ps, max_ctx_len=700, window=window)
        got = out.cpu().double().reshape(T, H, hd)
        if nb == 1:
            first = got
        else:
            assert torch.equal(got, first), "the result depends on the column blocking"
        _check_step(case, reqs, got, H, hd, window, nb)


@pytest.mark.parametrize("H,Hkv,hd,ps", [(8, 2, 64, 96), (4, 1, 64, 112), (6, 3, 32, 144), (4, 2, 128, 96), (4, 4, 64, 272)])
@pytest.mark.parametrize("window", [0, 300])
def test_attention_mfma_on_pages_that_do_not_divide_a_partition(gpu, H, Hkv, hd, ps, window):
    """Pages of 96, 112, 144 and 272 positions: a partition of 256 keys that starts inside a page touches one
    page more than 256 / page size rounded up (the partition at key 256 of pages of 96: pages 2 to 5).
    Contexts beyond 1,100 keys, every partition start among them; stale pages hold NaN."""
    from tuff_amd.csrc import ops
    reqs = [(1199, 1), (1150, 40), (0, 33), (255, 3), (511, 2), (767, 1), (1023, 2), (300, 1)]
    case = _mixed_step_case(gpu, reqs, H, Hkv, hd, ps)
    T = case["q"].shape[0]
    blocks = torch.from_numpy(ops.query_blocks(case["q_len"], H // Hkv, 1)).to(gpu)
    out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
    ops.attention_mfma(case["q"].to(gpu), case["kc"], case["vc"], out, block_table=case["table"],
                       blocks=blocks, nb=1, req_info=case["req_info"], positions=case["positions"], H=H, Hkv=Hkv,
                       hd=hd, page_size=ps, max_ctx_len=case["max_ctx_len"], window=window)
    _check_step(case, reqs, out.cpu().double().reshape(T, H, hd), H, hd, window, ps)


def _decode_case(gpu, R, H, Hkv, ps, lens, seed=0, nan_pool=True):
    """R requests with lens[r] tokens in the cache after this step; the step brings each one's last
    token as a projected row [q heads | k heads | v heads] of heads of 64.  Pages shuffled."""
    hd, dt = 64, torch.bfloat16
    g = torch.Generator().manual_seed(seed)
    n_blocks = [-(-n // ps) for n in lens]
    n_pages = sum(n_blocks) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    fill = float("nan") if nan_pool else 0.0
    kc = torch.full((n_pages, Hkv, ps, hd), fill, dtype=dt)
    vc = torch.full((n_pages, Hkv, hd, ps), fill, dtype=dt)
    table = torch.full((R, max(n_blocks) + 1), -1, dtype=torch.int32)
    slots = []
    for r, (n, nb_) in enumerate(zip(lens, n_blocks)):
        pages = torch.tensor([perm.pop() for _ in range(nb_)])
        table[r, :nb_] = pages.to(torch.int32)
        t = torch.arange(n - 1)                                           # everything but the step's own token
        kc[pages[t // ps], :, t % ps, :] = _r(n - 1, Hkv, hd, seed=seed + 10 + r, dtype=dt)
        vc[pages[t // ps], :, :, t % ps] = _r(n - 1, Hkv, hd, seed=seed + 40 + r, dtype=dt)
        slots.append(int(pages[(n - 1) // ps]) * ps + (n - 1) % ps)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    return dict(kc=kc.to(gpu), vc=vc.to(gpu), table=table.to(gpu), qkv=_r(R, (H + 2 * Hkv) * hd, seed=seed + 3, dtype=dt).to(gpu),
                positions=i32([n - 1 for n in lens]), slots=i32(slots),
                req_info=i32([[r, 1, n - 1, n] for r, n in enumerate(lens)]), max_ctx_len=max(lens))


@pytest.mark.parametrize("H,Hkv,ps", [(32, 8, 16), (6, 3, 64), (16, 1, 32), (8, 2, 96), (4, 1, 112)])
@pytest.mark.parametrize("window", [0, 300])
@pytest.mark.parametrize("norm_dt", [torch.float32, torch.bfloat16, None])
def test_attention_decode_fused_equals_the_separate_kernels(gpu, H, Hkv, ps, window, norm_dt):
    """A step of single tokens from the projected rows in one kernel (norm, rotation, cache write,
    attention) against the kernel that prepares q and writes the cache followed by the attention
    kernel: the same cache and the same output, bit for bit; stale pages hold NaN."""
    from tuff_amd.csrc import ops
    hd, eps, base = 64, 1e-6, 1e6
    lens = [700, 1, 257, 256, 33, 1025, 64, 1290]
    R = len(lens)
    qw = kw = None
    if norm_dt is not None:
        qw, kw = (1 + _r(hd, seed=5, scale=0.1)).to(norm_dt).to(gpu), (1 + _r(hd, seed=6, scale=0.1)).to(norm_dt).to(gpu)
    inv_freq = (base ** (-2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float().to(gpu)
    outs = []
    angles = ops.rope_table(inv_freq, 600)                  # reaches some of the positions, not all
    for fused in (False, True, "with a table of angles"):
        c = _decode_case(gpu, R, H, Hkv, ps, lens)
        out = torch.full((R, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        common = dict(block_table=c["table"], req_info=c["req_info"], positions=c["positions"], H=H, Hkv=Hkv,
                      page_size=ps, max_ctx_len=c["max_ctx_len"], window=window)
        if fused:
            ops.attention_decode_fused(c["qkv"], c["kc"], c["vc"], out, inv_freq=inv_freq, slot_mapping=c["slots"],
                                       q_norm_w=qw, k_norm_w=kw, eps=eps, angles=angles if fused is not True else None,
                                       **common)
        else:
            q = torch.empty(R, H * hd, dtype=torch.bfloat16, device=gpu)
            ops.qkv_post(c["qkv"], q, H=H, Hkv=Hkv, hd=hd, positions=c["positions"], eps=eps, q_norm_w=qw, k_norm_w=kw,
                         inv_freq=inv_freq, rotary_dim=hd, k_cache=c["kc"], v_cache=c["vc"], slot_mapping=c["slots"],
                         page_size=ps)
            ops.attention_mfma(q, c["kc"], c["vc"], out, blocks=None, nb=1, hd=hd, **common)
        outs.append((out.float().cpu(), c["kc"].float().cpu(), c["vc"].float().cpu()))
    (o0, k0, v0) = outs[0]
    same = lambda a, b: torch.equal(torch.nan_to_num(a, nan=12345.0), torch.nan_to_num(b, nan=12345.0))
    for (o1, k1, v1) in outs[1:]:
        assert torch.isfinite(o1).all()
        assert same(k0, k1) and same(v0, v1), "the two ways write different keys or values"
        assert torch.equal(o0, o1)
    # reading only: nothing is written, the token's own key is then not in the cache (NaN there would show)
    c = _decode_case(gpu, R, H, Hkv, ps, [n + 1 for n in lens], nan_pool=False)
    before = (c["kc"].clone(), c["vc"].clone())
    out = torch.empty((R, H * hd), dtype=torch.bfloat16, device=gpu)
    ops.attention_decode_fused(c["qkv"], c["kc"], c["vc"], out, inv_freq=inv_freq, slot_mapping=None, q_norm_w=qw, k_norm_w=kw,
                               eps=eps, block_table=c["table"], req_info=c["req_info"], positions=c["positions"], H=H, Hkv=Hkv,
                               page_size=ps, max_ctx_len=c["max_ctx_len"], window=window)
    assert torch.equal(before[0], c["kc"]) and torch.equal(before[1], c["vc"])


def test_attention_of_single_tokens_is_the_same_with_one_wave_or_four_a_partition(gpu):
    """Few requests: four waves share a partition of 256 keys; many: one wave walks it.  A request's
    result is the same bit for bit in either company."""
    from tuff_amd.csrc import ops
    H, Hkv, hd, ps = 32, 8, 64, 16
    lens = [2100, 37, 513] + [1800 + 7 * i for i in range(29)]           # 32 requests, 9 partitions: 2304 workgroups
    inv_freq = (1e6 ** (-2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float().to(gpu)
    qw = (1 + _r(hd, seed=5, scale=0.1)).to(gpu)

    def run(n_req, fused):
        c = _decode_case(gpu, len(lens), H, Hkv, ps, lens, nan_pool=False)
        sub = dict(block_table=c["table"][:n_req].contiguous(), req_info=c["req_info"][:n_req].contiguous(),
                   positions=c["positions"][:n_req].contiguous(), H=H, Hkv=Hkv, page_size=ps, max_ctx_len=c["max_ctx_len"])
        out = torch.empty((n_req, H * hd), dtype=torch.bfloat16, device=gpu)
        if fused:
            ops.attention_decode_fused(c["qkv"][:n_req].contiguous(), c["kc"], c["vc"], out, inv_freq=inv_freq,
                                       slot_mapping=c["slots"][:n_req].contiguous(), q_norm_w=qw, k_norm_w=qw, eps=1e-5, **sub)
        else:
            ops.attention_mfma(c["qkv"][:n_req, :H * hd].contiguous(), c["kc"], c["vc"], out, blocks=None, nb=1, hd=hd, **sub)
        return out.float().cpu()
    for fused in (False, True):
        few, many = run(3, fused), run(len(lens), fused)
        assert torch.isfinite(many).all() and torch.equal(few, many[:3]), f"fused={fused}"


@pytest.mark.parametrize("H,Hkv", [(32, 8), (6, 3), (5, 5), (16, 1)])
def test_attention_of_single_tokens_does_not_depend_on_the_order_of_its_workgroups(gpu, H, Hkv):
    """Large launches number their workgroups with the kv head changing fastest, small ones with the
    partition: the same bits either way (forced both ways here), fused and not."""
    import ctypes
    from tuff_amd.csrc import ops
    hd, ps = 64, 16
    lens = [700, 1, 257, 256, 33, 1025, 64]
    R = len(lens)
    inv_freq = (1e6 ** (-2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float().to(gpu)
    qw = (1 + _r(hd, seed=5, scale=0.1)).to(gpu)
    lib = ops.load("attention_mfma")
    lib.tuff_attention_kv_fast_waves.argtypes = [ctypes.c_int]
    lib.tuff_attention_kv_fast_waves.restype = ctypes.c_int

    def run(fused):
        c = _decode_case(gpu, R, H, Hkv, ps, lens)
        common = dict(block_table=c["table"], req_info=c["req_info"], positions=c["positions"], H=H, Hkv=Hkv,
                      page_size=ps, max_ctx_len=c["max_ctx_len"])
        out = torch.full((R, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        if fused:
            ops.attention_decode_fused(c["qkv"], c["kc"], c["vc"], out, inv_freq=inv_freq, slot_mapping=c["slots"],
                                       q_norm_w=qw, k_norm_w=qw, eps=1e-5, **common)
        else:
            c["kc"].nan_to_num_(0.0); c["vc"].nan_to_num_(0.0)             # the step's own key is not written here
            ops.attention_mfma(c["qkv"][:, :H * hd].contiguous(), c["kc"], c["vc"], out, blocks=None, nb=1, hd=hd, **common)
        torch.cuda.synchronize()
        return out.float().cpu(), c["kc"].float().cpu()

    for fn in (lib.tuff_attention_stage_k_waves, lib.tuff_attention_few_waves):
        fn.argtypes, fn.restype = [ctypes.c_int], ctypes.c_int
    before = lib.tuff_attention_kv_fast_waves(-1)
    staged, few = lib.tuff_attention_stage_k_waves(-1), lib.tuff_attention_few_waves(-1)
    try:
        for fused in (False, True):
            lib.tuff_attention_kv_fast_waves(1 << 30)
            o_part, k_part = run(fused)
            lib.tuff_attention_kv_fast_waves(0)
            o_kv, k_kv = run(fused)
            assert torch.isfinite(o_part).all()
            assert torch.equal(o_part, o_kv), f"fused={fused}"
            assert torch.equal(torch.nan_to_num(k_part, nan=1e9), torch.nan_to_num(k_kv, nan=1e9))
            # ... and as the largest launches run: one wave a partition, the keys through LDS
            lib.tuff_attention_few_waves(0)
            lib.tuff_attention_stage_k_waves(0)
            o_lds, k_lds = run(fused)
            lib.tuff_attention_stage_k_waves(1 << 30)
            o_one, _ = run(fused)
            lib.tuff_attention_few_waves(few)
            assert torch.equal(o_lds, o_one) and torch.equal(o_lds, o_part), f"fused={fused}: keys through LDS"
            assert torch.equal(torch.nan_to_num(k_part, nan=1e9), torch.nan_to_num(k_lds, nan=1e9))
    finally:
        lib.tuff_attention_kv_fast_waves(before)
        lib.tuff_attention_stage_k_waves(staged)
        lib.tuff_attention_few_waves(few)


@pytest.mark.parametrize("H,Hkv,hd,ps", [(32, 8, 64, 16), (6, 3, 64, 64), (4, 2, 40, 16), (3, 1, 48, 32), (8, 2, 56, 16)])
def test_attention_of_single_tokens_with_keys_through_lds_or_not(gpu, H, Hkv, hd, ps):
    """Large launches ask for the keys of heads of up to 64 channels as they lie in memory and put them into the
    operands' order through LDS, small ones read them in that order at once: the same bits either way (forced both
    ways here), and close to the plain attention."""
    import ctypes
    from tuff_amd.csrc import ops
    lens = [700, 1, 257, 256, 33, 1025, 64, 17, 300]
    R = len(lens)
    lib = ops.load("attention_mfma")
    lib.tuff_attention_stage_k_waves.argtypes = [ctypes.c_int]
    lib.tuff_attention_stage_k_waves.restype = ctypes.c_int
    lib.tuff_attention_few_waves.argtypes = [ctypes.c_int]
    lib.tuff_attention_few_waves.restype = ctypes.c_int
    case = _paged_case(gpu, torch.bfloat16, H, Hkv, hd, ps, lens, 0)
    kc, vc, table, req, pos, q, Ks, Vs = case
    # the last token of every request
    last = [int(torch.nonzero((req == i) & (pos == lens[i] - 1))[0]) for i in range(R)]
    q1 = q[last].contiguous().to(gpu)
    info = torch.tensor([[i, 1, lens[i] - 1, lens[i]] for i in range(R)], dtype=torch.int32, device=gpu)
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=gpu)
    outs = []
    before = lib.tuff_attention_stage_k_waves(-1)
    few = lib.tuff_attention_few_waves(0)                 # one wave a partition, as large launches have it
    try:
        for waves in (1 << 30, 0):
            lib.tuff_attention_stage_k_waves(waves)
            out = torch.full((R, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
            ops.attention_mfma(q1, kc.to(gpu), vc.to(gpu), out, blocks=None, nb=1, hd=hd, block_table=table.to(gpu), req_info=info,
                               positions=positions, H=H, Hkv=Hkv, page_size=ps, max_ctx_len=max(lens))
            torch.cuda.synchronize()
            outs.append(out.float().cpu())
    finally:
        lib.tuff_attention_stage_k_waves(before)
        lib.tuff_attention_few_waves(few)
    assert torch.isfinite(outs[0]).all() and torch.equal(outs[0], outs[1])
    G = H // Hkv
    for i in range(R):
        K, V = Ks[i][:lens[i]], Vs[i][:lens[i]]                           # [n, Hkv, hd] of the request, float64
        qi = q[last[i]].double().view(H, hd)
        for h in range(H):
            p = torch.softmax(K[:, h // G] @ qi[h] / hd ** 0.5, 0)
            want = p @ V[:, h // G]
            got = outs[1][i].view(H, hd)[h].double()
            assert (got - want).abs().max() <= 2 ** -6 * max(float(want.abs().max()), 0.05), (i, h)


@pytest.mark.parametrize("H,Hkv,hd,ps", [(4, 2, 16, 16), (4, 1, 24, 16), (3, 3, 80, 16), (2, 1, 256, 32),
                                          (32, 8, 64, 16), (8, 2, 128, 64), (32, 1, 64, 16), (5, 5, 40, 48),
                                          (6, 2, 96, 80)])
@pytest.mark.parametrize("window", [0, 37, 300])
def test_attention_prefill(gpu, H, Hkv, hd, ps, window):
    """Prompt portions of several blocks of columns, starting anywhere, beside single tokens; a
    token's result must not depend on where its portion started."""
    from tuff_amd.csrc import ops
    cols = ops.attention_prefill_block_columns(hd)

    def run(reqs):
        case = _mixed_step_case(gpu, reqs, H, Hkv, hd, ps)
        T = case["q"].shape[0]
        blocks = torch.from_numpy(ops.query_blocks(case["q_len"], H // Hkv, cols // 16)).to(gpu)
        out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        ops.attention_prefill(case["q"].to(gpu), case["kc"], case["vc"], out, block_table=case["table"],
                              blocks=blocks, req_info=case["req_info"], H=H, Hkv=Hkv, hd=hd, page_size=ps,
                              max_ctx_len=case["max_ctx_len"], window=window)
        got = out.cpu().double().reshape(T, H, hd)
        _check_step(case, reqs, got, H, hd, window, "prefill")
        return case, got

    reqs = [(699, 1), (230, 150), (0, 333), (0, 1), (255, 3), (1100, 70)]
    case, got = run(reqs)
    # the blocks listed with the most keys first, as the attention part lists them: the same bits
    T = case["q"].shape[0]
    ctx_len = [past + n for past, n in reqs]
    sorted_blocks = ops.query_blocks(case["q_len"], H // Hkv, cols // 16, ctx_len)
    plain_blocks = ops.query_blocks(case["q_len"], H // Hkv, cols // 16)
    assert sorted(map(tuple, sorted_blocks.tolist())) == sorted(map(tuple, plain_blocks.tolist()))
    assert sorted_blocks[0].tolist() == [5, (70 * (H // Hkv) - 1) // cols * cols]      # the last block of the request at 1,170
    out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
    ops.attention_prefill(case["q"].to(gpu), case["kc"], case["vc"], out, block_table=case["table"],
                          blocks=torch.from_numpy(sorted_blocks).to(gpu), req_info=case["req_info"], H=H, Hkv=Hkv, hd=hd,
                          page_size=ps, max_ctx_len=case["max_ctx_len"], window=window)
    assert torch.equal(out.cpu().double().reshape(T, H, hd), got), "the result depends on the order of the blocks"
    # tokens 70..149 of request 1 (positions 300..379) again, as a step of their own that starts
    # at position 300: bit for bit the same
    first = sum(n for _, n in reqs[:1]) + 70
    sel = torch.arange(first, first + 80)
    q3 = case["q"][sel]
    # give the single request the keys and values of request 1 of the first step
    K, V = case["Ks"][1].to(torch.bfloat16), case["Vs"][1].to(torch.bfloat16)
    n_blk = -(-380 // ps)
    kc = torch.full((n_blk + 1, Hkv, ps, hd), float("nan"), dtype=torch.bfloat16)
    vc = torch.full((n_blk + 1, Hkv, hd, ps), float("nan"), dtype=torch.bfloat16)
    t = torch.arange(380)
    kc[t // ps, :, t % ps, :] = K
    vc[t // ps, :, :, t % ps] = V
    table = torch.arange(n_blk, dtype=torch.int32)[None].to(gpu)
    out = torch.full((80, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
    blocks = torch.from_numpy(ops.query_blocks([80], H // Hkv, cols // 16)).to(gpu)
    ops.attention_prefill(q3.to(gpu), kc.to(gpu), vc.to(gpu), out, block_table=table, blocks=blocks,
                          req_info=torch.tensor([[0, 80, 300, 380]], dtype=torch.int32, device=gpu), H=H, Hkv=Hkv, hd=hd,
                          page_size=ps, max_ctx_len=380, window=window)
    assert torch.equal(out.cpu().double().reshape(80, H, hd), got[sel]), "the result depends on where the portion starts"


def test_attention_long_context(gpu):
    """Past 64 partitions of 256 keys (the general merge) and past many batches of page numbers:
    single tokens and a portion deep in requests of about 20,000 tokens, one with a window."""
    from tuff_amd.csrc import ops
    H, Hkv, hd, ps = 4, 2, 64, 16
    for window in (0, 5000):
        reqs = [(19999, 1), (17000, 200), (16390, 1)]
        case = _mixed_step_case(gpu, reqs, H, Hkv, hd, ps)
        T = case["q"].shape[0]
        common = dict(block_table=case["table"], req_info=case["req_info"], H=H, Hkv=Hkv, hd=hd, page_size=ps,
                      max_ctx_len=case["max_ctx_len"], window=window)
        out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        blocks = torch.from_numpy(ops.query_blocks(case["q_len"], H // Hkv, 1)).to(gpu)
        ops.attention_mfma(case["q"].to(gpu), case["kc"], case["vc"], out, blocks=blocks, nb=1,
                           positions=case["positions"], **common)
        _check_step(case, reqs, out.cpu().double().reshape(T, H, hd), H, hd, window, ("mfma", window))
        # a wider block table and more (empty) partitions, as a recorded step's buckets bring: the same bits
        wide = torch.cat([case["table"], torch.full((len(reqs), 400), -1, dtype=torch.int32, device=gpu)], dim=1).contiguous()
        out_w = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        ops.attention_mfma(case["q"].to(gpu), case["kc"], case["vc"], out_w, blocks=blocks, nb=1, positions=case["positions"],
                           **dict(common, block_table=wide, max_ctx_len=case["max_ctx_len"] + 6000))
        assert torch.equal(out, out_w), "the merge depends on how many partitions the step has room for"
        out2 = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        cols = ops.attention_prefill_block_columns(hd)
        blocks = torch.from_numpy(ops.query_blocks(case["q_len"], H // Hkv, cols // 16)).to(gpu)
        ops.attention_prefill(case["q"].to(gpu), case["kc"], case["vc"], out2, blocks=blocks, **common)
        _check_step(case, reqs, out2.cpu().double().reshape(T, H, hd), H, hd, window, ("prefill", window))


@pytest.mark.parametrize("H,Hkv,hd,ps", [(4, 2, 64, 16), (3, 1, 80, 32), (2, 2, 128, 16)])
@pytest.mark.parametrize("window", [0, 700])
def test_attention_prefill_key_segments(gpu, H, Hkv, hd, ps, window, monkeypatch):
    """A short portion far into long requests: few blocks of columns, so the keys are cut into
    segments, a workgroup a segment, and the segments merged.  Against the plain formula, and against
    the same step without segments (to the rounding of one merge).  One request is shorter than a
    segment, one ends inside a segment, stale pages hold NaN."""
    from tuff_amd.csrc import ops
    reqs = [(5000, 40), (2100, 30), (300, 17), (0, 5)]
    case = _mixed_step_case(gpu, reqs, H, Hkv, hd, ps)
    T = case["q"].shape[0]
    cols = ops.attention_prefill_block_columns(hd)
    blocks = torch.from_numpy(ops.query_blocks(case["q_len"], H // Hkv, cols // 16)).to(gpu)
    outs = {}
    for segments in (False, True):
        out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=gpu)
        ops.attention_prefill(case["q"].to(gpu), case["kc"], case["vc"], out, block_table=case["table"],
                              blocks=blocks, req_info=case["req_info"], H=H, Hkv=Hkv, hd=hd, page_size=ps,
                              max_ctx_len=case["max_ctx_len"], window=window,
                              positions=case["positions"] if segments else None)
        outs[segments] = out.cpu().double().reshape(T, H, hd)
        _check_step(case, reqs, outs[segments], H, hd, window, f"segments {segments}")
    assert 2 * blocks.shape[0] * Hkv <= ops.PREFILL_WORKGROUP_SLOTS and case["max_ctx_len"] >= 2 * ops.PREFILL_MIN_SEGMENT
    # the two ways differ in rounding only
    assert (outs[True] - outs[False]).abs().max() <= 2 ** -7 * float(outs[False].abs().max())


@pytest.mark.parametrize("kernel", ["mfma", "prefill"])
def test_attention_matrix_kernels_find_a_far_key_and_the_window_edge(gpu, kernel):
    """One key among a thousand matches the query: the output is that key's value row, wherever
    the key sits (first position, edges of pages, of steps and of partitions, the last position).
    With a window W the key at pos - W + 1 is seen and the one at pos - W is not."""
    from tuff_amd.csrc import ops
    hd, ps, n = 32, 16, 1000
    dt = torch.bfloat16
    n_pages = n // ps + 1
    table = torch.arange(n_pages, dtype=torch.int32)[None].to(gpu)

    def run(q, kc, vc, n_q, window):
        out = torch.empty(n_q, hd, dtype=dt, device=gpu)
        pos0 = n - n_q
        info = torch.tensor([[0, n_q, pos0, n]], dtype=torch.int32, device=gpu)
        common = dict(block_table=table, req_info=info, H=1, Hkv=1, hd=hd, page_size=ps, max_ctx_len=n, window=window)
        if kernel == "mfma":
            blocks = torch.from_numpy(ops.query_blocks([n_q], 1, 1)).to(gpu)
            ops.attention_mfma(q.to(gpu), kc.to(gpu), vc.to(gpu), out, blocks=blocks, nb=1,
                               positions=torch.arange(pos0, n, dtype=torch.int32, device=gpu), **common)
        else:
            blocks = torch.from_numpy(ops.query_blocks([n_q], 1, ops.attention_prefill_block_columns(hd) // 16)).to(gpu)
            ops.attention_prefill(q.to(gpu), kc.to(gpu), vc.to(gpu), out, blocks=blocks, **common)
        return out.cpu()

    for hot in (0, 15, 16, 31, 32, 63, 64, 255, 256, 447, 448, 959, 960, 998, 999):
        kc = _r(n_pages, 1, ps, hd, seed=3, scale=0.05, dtype=dt)
        vc = _r(n_pages, 1, hd, ps, seed=4, dtype=dt)
        q = torch.zeros(3, hd, dtype=dt)
        q[:, 5] = 30.0
        kc[hot // ps, 0, hot % ps, 5] = 30.0                     # score 900/sqrt(32) = 159 above the rest
        out = run(q, kc, vc, 3, 0)
        for j in range(3):                                        # queries at positions n-3, n-2, n-1
            if hot <= n - 3 + j:
                assert torch.equal(out[j], vc[hot // ps, 0, :, hot % ps]), (hot, j)
    W = 300
    for n_q in (1, 5):
        pos = n - n_q                                             # the first query of the step
        for edge, seen in ((pos - W + 1, True), (pos - W, False)):
            kc = torch.zeros(n_pages, 1, ps, hd, dtype=dt)
            vc = torch.zeros(n_pages, 1, hd, ps, dtype=dt)
            q = torch.zeros(n_q, hd, dtype=dt)
            q[:, 0] = 20.0
            kc[edge // ps, 0, edge % ps, 0] = 20.0
            vc[edge // ps, 0, :, edge % ps] = 1.0
            out = run(q, kc, vc, n_q, W)
            if seen:
                assert float(out[0].min()) > 0.99, (n_q, edge)
            else:
                assert float(out[0].abs().max()) == 0.0, (n_q, edge)


def test_attention_finds_a_far_key(gpu):
    """One key among hundreds matches the query: the output must be that key's value row,
    wherever the key sits (first position, a page's edge, a tile's edge, the last position)."""
    from tuff_amd.csrc import ops
    H = Hkv = 1
    hd, ps, n = 32, 16, 700
    for dt in (torch.float32, torch.bfloat16):
        for hot in (0, 15, 16, 63, 64, 447, 448, 699):
            kc = _r(n // ps + 1, 1, ps, hd, seed=3, scale=0.05, dtype=dt)
            vc = _r(n // ps + 1, 1, hd, ps, seed=4, dtype=dt)
            q = torch.zeros(1, hd, dtype=dt)
            q[0, 5] = 30.0
            kc[hot // ps, 0, hot % ps, 5] = 30.0                     # score 900/sqrt(32) = 159 above the rest
            table = torch.arange(n // ps + 1, dtype=torch.int32)[None]
            out = torch.empty(1, hd, dtype=dt, device=gpu)
            ops.attention_general(q.to(gpu), kc.to(gpu), vc.to(gpu), out, block_table=table.to(gpu),
                                  req_of_token=torch.zeros(1, dtype=torch.int32, device=gpu),
                                  positions=torch.tensor([n - 1], dtype=torch.int32, device=gpu),
                                  H=1, Hkv=1, hd=hd, page_size=ps)
            assert torch.equal(out.cpu()[0], vc[hot // ps, 0, :, hot % ps]), (dt, hot)


def test_attention_window_edge(gpu):
    """With window W the key at pos - W + 1 is seen and the key at pos - W is not."""
    from tuff_amd.csrc import ops
    hd, ps, W, pos = 16, 16, 40, 100
    for edge, seen in ((pos - W + 1, True), (pos - W, False)):
        kc = torch.zeros(8, 1, ps, hd)
        vc = torch.zeros(8, 1, hd, ps)
        q = torch.zeros(1, hd)
        q[0, 0] = 20.0
        kc[edge // ps, 0, edge % ps, 0] = 20.0
        vc[edge // ps, 0, :, edge % ps] = 1.0
        out = torch.empty(1, hd, device=gpu)
        ops.attention_general(q.to(gpu), kc.to(gpu), vc.to(gpu), out,
                              block_table=torch.arange(8, dtype=torch.int32, device=gpu)[None],
                              req_of_token=torch.zeros(1, dtype=torch.int32, device=gpu),
                              positions=torch.tensor([pos], dtype=torch.int32, device=gpu),
                              H=1, Hkv=1, hd=hd, page_size=ps, window=W)
        if seen:
            assert out.min() > 0.999
        else:
            assert out.abs().max() == 0


# ------------------------------------------------------------------------- short conv
@pytest.mark.parametrize("d,K", [(64, 3), (96, 4), (240, 2), (300, 7)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_shortconv(gpu, d, K, dt):
    """Two requests cut into different portions; outputs and final states equal the plain
    whole-sequence convolution."""
    from tuff_amd.csrc import ops
    lens = [23, 9]
    w = _r(d, K, seed=20, dtype=dt)
    bcx_all = [_r(n, 3 * d, seed=21 + i, dtype=dt) for i, n in enumerate(lens)]

    def whole(bcx):
        x = bcx.double()
        u = x[:, :d] * x[:, 2 * d:]
        hist = torch.cat([torch.zeros(K - 1, d, dtype=torch.float64), u])
        y = sum(hist[k:k + len(u)] * w.double()[:, k] for k in range(K))
        return x[:, d:2 * d] * y, hist[-(K - 1):]
    state = torch.zeros(4, K - 1, d, device=gpu)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=gpu)
    cuts = [[5, 1, 1, 10, 6], [1, 2, 6]]
    outs = [[], []]
    done = [0, 0]
    for step in range(5):
        rows, q_start, q_len, req_of, who = [], [], [], [], []
        for r in range(2):
            if step < len(cuts[r]):
                n = cuts[r][step]
                q_start.append(sum(q_len))
                q_len.append(n)
                req_of += [len(who)] * n
                who.append(r)
                rows.append(bcx_all[r][done[r]:done[r] + n])
                done[r] += n
        bcx = torch.cat(rows).to(gpu)
        out = torch.empty(bcx.shape[0], d, dtype=dt, device=gpu)
        meta = dict(q_start=torch.tensor(q_start, dtype=torch.int32, device=gpu),
                    state_slot=torch.tensor([[2, 0][r] for r in who], dtype=torch.int32, device=gpu))
        _conv_both_ways(ops, bcx, w.to(gpu), state, out, req_of_token=torch.tensor(req_of, dtype=torch.int32, device=gpu),
                        q_len=torch.tensor(q_len, dtype=torch.int32, device=gpu), K=K, **meta)
        for i, r in enumerate(who):
            outs[r].append(out[q_start[i]:q_start[i] + q_len[i]].cpu())
    for r in range(2):
        want, want_state = whole(bcx_all[r])
        got = torch.cat(outs[r]).double()
        tol = 1e-6 if dt == torch.float32 else 2 ** -8
        assert (got - want).abs().max() <= tol * float(want.abs().max())
        assert (state[int(slots[r])].cpu().double() - want_state).abs().max() <= 1e-6
    assert (state[1] == 0).all() and (state[3] == 0).all()       # other requests' slots untouched


def _conv_both_ways(ops, bcx, w, state, out, *, req_of_token, q_start, q_len, state_slot, K):
    """The kernel that only reads the state followed by the one that rewrites it, and the kernel that
    does both (the one the mixer runs): the same output and the same state, bit for bit.  Leaves the
    result in `state` and `out`."""
    state2, out2 = state.clone(), torch.full_like(out, float("nan"))
    ops.shortconv_fwd(bcx, w, state, out, req_of_token=req_of_token, q_start=q_start, state_slot=state_slot, K=K)
    ops.shortconv_state(bcx, state, q_start=q_start, q_len=q_len, state_slot=state_slot, K=K)
    ops.shortconv_fwd(bcx, w, state2, out2, req_of_token=req_of_token, q_start=q_start, state_slot=state_slot, K=K, q_len=q_len)
    assert torch.equal(out, out2), "output of the kernel that also rewrites the state"
    assert torch.equal(state, state2), "state of the kernel that also rewrites the state"


@pytest.mark.parametrize("d,K", [(64, 3), (96, 4), (240, 2), (300, 7)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_shortconv_single_token_kernel_equals_the_general_pair(gpu, d, K, dt):
    from tuff_amd.csrc import ops
    R = 5
    w = _r(d, K, seed=20, dtype=dt).to(gpu)
    slots = torch.tensor([3, 0, 6, 1, 4], dtype=torch.int32, device=gpu)
    s1 = _r(8, K - 1, d, seed=21).to(gpu)
    s2 = s1.clone()
    ar = torch.arange(R, dtype=torch.int32, device=gpu)
    ones = torch.ones(R, dtype=torch.int32, device=gpu)
    for step in range(4):
        bcx = _r(R, 3 * d, seed=30 + step, dtype=dt).to(gpu)
        o1 = torch.empty(R, d, dtype=dt, device=gpu)
        o2 = torch.empty(R, d, dtype=dt, device=gpu)
        _conv_both_ways(ops, bcx, w, s1, o1, req_of_token=ar, q_start=ar, q_len=ones, state_slot=slots, K=K)
        ops.shortconv_decode(bcx, w, s2, o2, state_slot=slots, K=K)
        assert torch.equal(o1, o2) and torch.equal(s1, s2), step


@pytest.mark.parametrize("d,K", [(64, 3), (96, 4), (240, 2), (2048, 3), (300, 7)])
def test_shortconv_long_portions_equal_single_tokens(gpu, d, K):
    """Portions of more than 16 tokens (eight channels a thread in bfloat16) give, bit for bit,
    what the same tokens give one at a time."""
    from tuff_amd.csrc import ops
    dt = torch.bfloat16
    lens, cuts = [70, 33], [[40, 30], [33]]
    w = _r(d, K, seed=20, dtype=dt).to(gpu)
    bcx_all = [_r(n, 3 * d, seed=21 + i, dtype=dt).to(gpu) for i, n in enumerate(lens)]
    slots = [2, 0]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    # one token at a time
    s1 = torch.zeros(4, K - 1, d, device=gpu)
    single = [[], []]
    for r in range(2):
        for t in range(lens[r]):
            o = torch.empty(1, d, dtype=dt, device=gpu)
            ops.shortconv_decode(bcx_all[r][t:t + 1], w, s1, o, state_slot=i32([slots[r]]), K=K)
            single[r].append(o)
    # in portions, both requests in one step where both have one
    s2 = torch.zeros(4, K - 1, d, device=gpu)
    got = [[], []]
    done = [0, 0]
    for step in range(2):
        who = [r for r in range(2) if step < len(cuts[r])]
        q_len = [cuts[r][step] for r in who]
        q_start = [sum(q_len[:i]) for i in range(len(who))]
        bcx = torch.cat([bcx_all[r][done[r]:done[r] + n] for r, n in zip(who, q_len)])
        out = torch.empty(bcx.shape[0], d, dtype=dt, device=gpu)
        meta = dict(q_start=i32(q_start), state_slot=i32([slots[r] for r in who]))
        _conv_both_ways(ops, bcx, w, s2, out, req_of_token=i32([i for i, n in enumerate(q_len) for _ in range(n)]),
                        q_len=i32(q_len), K=K, **meta)
        for i, r in enumerate(who):
            got[r].append(out[q_start[i]:q_start[i] + q_len[i]])
            done[r] += q_len[i]
    for r in range(2):
        assert torch.equal(torch.cat(got[r]), torch.cat(single[r])), r
    assert torch.equal(s1, s2)


@pytest.mark.parametrize("M,d,K,taps", [(1, 64, 64, 3), (8, 2048, 2048, 3), (16, 240, 328, 4), (5, 48, 96, 2), (3, 96, 8192, 7),
                                        (17, 64, 64, 3), (32, 2048, 2048, 3), (24, 240, 328, 4), (20, 96, 8192, 7)])
@pytest.mark.parametrize("norm", ["none", "inside", "scaled"])
def test_gemm_with_the_convolution_in_its_epilogue(gpu, M, d, K, taps, norm):
    """Input projection and gated short convolution of single tokens in one kernel, against the plain
    formulas on the same bfloat16 inputs: out = C * conv(B * X) over each row's state, and the state
    shifted by u = B * X.  With the norm inside the product and with the row scales another product left."""
    from tuff_amd.csrc import ops
    if norm == "inside" and M > 16:
        pytest.skip("the norm inside the product is for at most 16 rows")
    eps = 1e-5
    w_in = _r(3 * d, K, seed=1, scale=K ** -0.5, dtype=torch.bfloat16)
    conv_w = _r(d, taps, seed=2, scale=0.5, dtype=torch.bfloat16)
    slots = torch.randperm(M + 3, generator=torch.Generator().manual_seed(3))[:M].to(torch.int32)
    state0 = _r(M + 3, taps - 1, d, seed=4)
    x32 = _r(M, K, seed=5)
    nw = 1 + _r(K, seed=6, scale=0.1)
    w = ops.tile_weight(ops.conv_group_rows(w_in.to(gpu)))
    state = state0.clone().to(gpu)
    out = torch.full((M, d), float("nan"), dtype=torch.bfloat16, device=gpu)
    kw = dict(conv_w=conv_w.to(gpu), state=state, state_slot=slots.to(gpu))
    if norm == "none":
        h = x32.to(torch.bfloat16)
        ops.gemm_conv(h.to(gpu), w, out, **kw)
        h = h.double()
    elif norm == "inside":
        ops.gemm_conv(x32.to(gpu), w, out, norm_w=nw.to(gpu), eps=eps, **kw)
        h = (x32 * nw).to(torch.bfloat16).double() / torch.sqrt((x32.double() ** 2).mean(-1, keepdim=True) + eps)
    else:
        xw = (x32 * nw).to(torch.bfloat16)
        tiles = 5
        ss = torch.zeros(tiles, 16 if M <= 16 else 64)
        cut = [K * t // tiles for t in range(tiles + 1)]
        for t in range(tiles):
            ss[t, :M] = (x32[:, cut[t]:cut[t + 1]] ** 2).sum(-1)
        ops.gemm_conv(xw.to(gpu), w, out, ss=ss.to(gpu), eps=eps, **kw)
        h = xw.double() / torch.sqrt((x32.double() ** 2).mean(-1, keepdim=True) + eps)
    bcx = (h @ w_in.double().T).to(torch.bfloat16).double()
    B, C, X = bcx[:, :d], bcx[:, d:2 * d], bcx[:, 2 * d:]
    u = B * X
    st = state0[slots.long()].double()                                   # [M, taps - 1, d]
    y = (st * conv_w.double().T[:taps - 1][None]).sum(1) + u * conv_w.double()[:, taps - 1]
    want = C * y
    got = out.cpu().double()
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() <= 2 ** -6 * float(want.abs().max()), (got - want).abs().max()
    new_state = state.cpu().double()
    want_state = torch.cat([st[:, 1:], u[:, None]], dim=1)
    assert (new_state[slots.long()] - want_state).abs().max() <= 2 ** -6 * float(want_state.abs().max())
    others = torch.ones(M + 3, dtype=torch.bool)
    others[slots.long()] = False
    assert torch.equal(new_state[others], state0[others].double())      # nobody else's state was touched
    with pytest.raises(ops.KernelError, match="at most 32 rows"):
        ops.gemm_conv(torch.zeros(33, K, dtype=torch.bfloat16, device=gpu), w, torch.empty(33, d, dtype=torch.bfloat16, device=gpu),
                      conv_w=conv_w.to(gpu), state=state, state_slot=torch.zeros(33, dtype=torch.int32, device=gpu))


@pytest.mark.parametrize("M,d,K,taps", [(33, 64, 64, 3), (64, 2048, 2048, 3), (40, 240, 328, 4), (48, 48, 96, 2), (50, 96, 8192, 7)])
@pytest.mark.parametrize("norm", ["none", "scaled"])
def test_gemm_with_the_convolution_in_the_kernel_that_adds_its_slices(gpu, M, d, K, taps, norm):
    """33 to 64 single tokens: the kernel that adds the projection's partial tiles runs the convolution.
    Against the plain formulas, and bit for bit against the projection followed by the kernel for single
    tokens (the same sums in the same order, rounded to bfloat16 at the same place)."""
    from tuff_amd.csrc import ops
    eps = 1e-5
    w_in = _r(3 * d, K, seed=1, scale=K ** -0.5, dtype=torch.bfloat16)
    conv_w = _r(d, taps, seed=2, scale=0.5, dtype=torch.bfloat16).to(gpu)
    slots = torch.randperm(M + 3, generator=torch.Generator().manual_seed(3))[:M].to(torch.int32)
    state0 = _r(M + 3, taps - 1, d, seed=4)
    x32 = _r(M, K, seed=5)
    nw = 1 + _r(K, seed=6, scale=0.1)
    w = ops.tile_weight(w_in.to(gpu))
    state, state2 = state0.clone().to(gpu), state0.clone().to(gpu)
    out = torch.full((M, d), float("nan"), dtype=torch.bfloat16, device=gpu)
    bcx = torch.empty(M, 3 * d, dtype=torch.bfloat16, device=gpu)
    kw = dict(conv_w=conv_w, state=state, state_slot=slots.to(gpu))
    if norm == "none":
        h = x32.to(torch.bfloat16)
        ops.gemm_conv64(h.to(gpu), w, out, **kw)
        ops.gemm(h.to(gpu), w, bcx)
        h = h.double()
    else:
        xw = (x32 * nw).to(torch.bfloat16)
        tiles = 5
        ss = torch.zeros(tiles, 64)
        cut = [K * t // tiles for t in range(tiles + 1)]
        for t in range(tiles):
            ss[t, :M] = (x32[:, cut[t]:cut[t + 1]] ** 2).sum(-1)
        ops.gemm_conv64(xw.to(gpu), w, out, ss=ss.to(gpu), eps=eps, **kw)
        ops.gemm_scaled(xw.to(gpu), ss.to(gpu), eps, w, bcx)
        h = xw.double() / torch.sqrt((x32.double() ** 2).mean(-1, keepdim=True) + eps)
    ref = (h @ w_in.double().T).to(torch.bfloat16).double()
    B, C, X = ref[:, :d], ref[:, d:2 * d], ref[:, 2 * d:]
    u = B * X
    st = state0[slots.long()].double()
    y = (st * conv_w.cpu().double().T[:taps - 1][None]).sum(1) + u * conv_w.cpu().double()[:, taps - 1]
    want = C * y
    got = out.cpu().double()
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() <= 2 ** -6 * float(want.abs().max()), (got - want).abs().max()
    want_state = torch.cat([st[:, 1:], u[:, None]], dim=1)
    assert (state.cpu().double()[slots.long()] - want_state).abs().max() <= 2 ** -6 * float(want_state.abs().max())
    others = torch.ones(M + 3, dtype=torch.bool)
    others[slots.long()] = False
    assert torch.equal(state.cpu()[others], state0[others])               # nobody else's state was touched
    # the two-kernel way from the projected rows
    out2 = torch.empty(M, d, dtype=torch.bfloat16, device=gpu)
    ops.shortconv_decode(bcx, conv_w, state2, out2, state_slot=slots.to(gpu), K=taps)
    if norm == "none":
        assert torch.equal(out, out2) and torch.equal(state, state2)
    else:                                      # with one slice the projection adds the sums of squares in another order
        assert (out.float() - out2.float()).abs().max() <= 2 ** -7 * float(out2.float().abs().max())


def test_shortconv_last_tap_is_the_current_token(gpu):
    from tuff_amd.csrc import ops
    d, K = 32, 3
    w = torch.zeros(d, K)
    w[:, K - 1] = 1.0
    bcx = _r(6, 3 * d, seed=30)
    out = torch.empty(6, d, device=gpu)
    z = torch.zeros(1, dtype=torch.int32, device=gpu)
    ops.shortconv_fwd(bcx.to(gpu), w.to(gpu), torch.zeros(1, K - 1, d, device=gpu), out,
                      req_of_token=torch.zeros(6, dtype=torch.int32, device=gpu), q_start=z, state_slot=z, K=K)
    want = bcx[:, d:2 * d] * bcx[:, :d] * bcx[:, 2 * d:]
    assert torch.allclose(out.cpu(), want, atol=1e-6)


def test_scatter_of_token_ids(gpu):
    from tuff_amd.csrc import ops
    dst = torch.arange(100, 137, dtype=torch.int32)
    src = torch.arange(1000, 1011, dtype=torch.int32)
    places, sources = [36, 0, 5, 17], [10, 3, 3, 0]
    d = dst.to(gpu)
    ops.scatter_i32(d, src.to(gpu), torch.tensor(places + sources, dtype=torch.int32, device=gpu))
    want = dst.clone()
    want[places] = src[sources]
    assert torch.equal(d.cpu(), want)
    for bad in ([37, 0], [0, 11], [-1, 0]):           # an index out of range writes nothing
        ops.scatter_i32(d, src.to(gpu), torch.tensor(bad, dtype=torch.int32, device=gpu))
        assert torch.equal(d.cpu(), want)


# --------------------------------------------------------------------------- sampling
def test_argmax_ties_go_to_the_lowest_index(gpu):
    from tuff_amd.csrc import ops
    l = _r(5, 1000, seed=40)
    l[0, 17] = l[0, 700] = 9.0
    l[1, 999] = 9.0
    l[2, :] = 0.0
    l[3, 0] = 9.0
    out = torch.empty(5, dtype=torch.int32, device=gpu)
    ops.argmax(l.to(gpu), out)
    assert out.cpu().tolist() == [17, 999, 0, 0, int(l[4].argmax())]
    out2 = torch.empty(5, dtype=torch.int32, device=gpu)
    ops.sample(l.to(gpu), out2)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("params", [dict(temp=0.8), dict(temp=1.0, top_k=5), dict(temp=0.7, top_p=0.9),
                                    dict(temp=1.3, min_p=0.05), dict(temp=0.9, top_k=40, top_p=0.8, min_p=0.01),
                                    dict(temp=2.0, top_k=1)])
def test_sample_matches_the_plain_sampler(gpu, params):
    """The same draws give the same tokens as the plain restatement of the reference's sampler,
    except where the draw falls within float32 rounding of a boundary between two candidates."""
    from plain.sampler_plain import PlainSampler
    from tuff_amd.csrc import ops
    V, R = 3001, 64
    logits = _r(R, V, seed=41, scale=3.0)
    plain_s = PlainSampler(seed=123, **params)
    us, want = [], []
    for r in range(R):
        probe = PlainSampler(seed=123, **params)
        probe.rng.s = list(plain_s.rng.s)
        us.append(float(probe.rng.uniform()))
        want.append(plain_s.sample(logits[r].numpy()))
    out = torch.empty(R, dtype=torch.int32, device=gpu)
    f = lambda key, default, dt: torch.full((R,), params.get(key, default), dtype=dt, device=gpu)
    ops.sample(logits.to(gpu), out, temps=f("temp", 0.0, torch.float32), top_ks=f("top_k", 0, torch.int32),
               top_ps=f("top_p", 1.0, torch.float32), min_ps=f("min_p", 0.0, torch.float32),
               uniforms=torch.tensor(us, dtype=torch.float32, device=gpu))
    got = out.cpu().tolist()
    differ = [r for r in range(R) if got[r] != want[r]]
    for r in differ:
        # allowed only if the two tokens are neighbours in the sorted order and r is at their border
        p = torch.softmax(logits[r].double() / params["temp"], 0)
        order = torch.argsort(-p)
        rank = {int(t): i for i, t in enumerate(order)}
        assert abs(rank[got[r]] - rank[want[r]]) == 1, (r, got[r], want[r])
    assert len(differ) <= 1


def _exact_draw(logits_row, params, u):
    """The reference's sampling order (src/sampler.c:115-230) with every sum in float64: the candidates in (value
    descending, index ascending) order and the rank of the first whose cumulative probability reaches the draw."""
    import numpy as np
    l = logits_row.numpy().astype(np.float32)
    scaled = (l - l.max()) * (np.float32(1.0) / np.float32(params["temp"]))          # float32, as both samplers form it
    keep = np.nonzero(scaled >= (np.float32(math.log(params["min_p"])) if 0 < params.get("min_p", 0) < 1 else np.float32(-1e30)))[0]
    order = keep[np.lexsort((keep, -scaled[keep].astype(np.float64)))]
    if params.get("top_k", 0) > 0:
        order = order[:params["top_k"]]
    mass = np.exp(scaled[order].astype(np.float64))
    cum = np.cumsum(mass)
    active = len(order)
    if 0 < params.get("top_p", 1.0) < 1:
        active = int(np.searchsorted(cum, np.float64(np.float32(params["top_p"])) * cum[-1], side="left")) + 1
    rank = int(np.searchsorted(cum[:active], np.float64(np.float32(u)) * cum[active - 1], side="left"))
    return order, min(rank, active - 1), mass / cum[-1]


def test_sample_at_a_border_of_the_cumulative_sums_is_the_exact_answer(gpu):
    """A vocabulary of 47,098 at temperature 1 with top_p 0.95 and min_p 0.02 (a case that a search over seeds
    found): the kernel's pick and the plain float32 sampler's lie 32 candidates apart.  The reference's sampler adds
    its float32 probabilities one after the other (src/sampler.c:185-226), so after 44,000 terms its running sum is
    off by up to 44,000 roundings and the candidate at which it reaches the draw is uncertain by that much
    probability; the kernel adds 40-bit fixed-point probabilities exactly.  So: the kernel's pick is the float64
    answer (to one candidate: its exp is float32), and the plain sampler's pick is as far from it as its rounding
    explains and no further."""
    import random
    from plain.sampler_plain import PlainSampler
    from tuff_amd.csrc import ops
    seed, row = 9633, 0
    rng = random.Random(seed)                                  # the search's own generation, step by step
    V = rng.choice([rng.randint(1, 40), rng.randint(41, 3000), rng.randint(3001, 70000)])
    R = rng.randint(1, 12)
    kind = rng.random()
    logits = torch.randn(R, V, generator=torch.Generator().manual_seed(seed)) * rng.choice([0.1, 1.0, 3.0, 10.0])
    if kind < 0.3:
        logits = (logits * 2).round() / 2
    elif kind < 0.4:
        logits[:, ::3] = -1e30
    params = dict(temp=rng.choice([0.0, 0.3, 0.8, 1.0, 1.7]), top_k=rng.choice([0, 0, 1, 5, 40, 5000]),
                  top_p=rng.choice([1.0, 1.0, 0.95, 0.5, 0.1]), min_p=rng.choice([0.0, 0.0, 0.02, 0.3]))
    assert V == 47098 and params == dict(temp=1.0, top_k=0, top_p=0.95, min_p=0.02)
    plain_s = PlainSampler(seed=seed + 1, **params)
    probe = PlainSampler(seed=seed + 1, **params)
    u = float(probe.rng.uniform())
    want = plain_s.sample(logits[row].numpy())
    out = torch.empty(1, dtype=torch.int32, device=gpu)
    f = lambda key, dt: torch.full((1,), params[key], dtype=dt, device=gpu)
    ops.sample(logits[row:row + 1].to(gpu), out, temps=f("temp", torch.float32), top_ks=f("top_k", torch.int32),
               top_ps=f("top_p", torch.float32), min_ps=f("min_p", torch.float32),
               uniforms=torch.tensor([u], dtype=torch.float32, device=gpu))
    got = int(out[0])
    order, exact, prob = _exact_draw(logits[row], params, u)
    rank = {int(t): i for i, t in enumerate(order)}
    assert abs(rank[got] - exact) <= 1, (rank[got], exact)
    assert got != want                                          # the case is one where the two samplers differ ...
    a, b = sorted((rank[got], rank[want]))
    between = float(prob[a:b + 1].sum())
    assert between <= len(order) * 2.0 ** -24, (between, len(order))   # ... by no more than sequential float32 sums explain


def test_sample_top_k_ties_and_uniform_logits(gpu):
    from tuff_amd.csrc import ops
    V = 500
    l = torch.zeros(3, V)
    out = torch.empty(3, dtype=torch.int32, device=gpu)
    u = torch.tensor([0.0, 0.5, 0.999999], dtype=torch.float32, device=gpu)
    ones = torch.ones(3, device=gpu)
    ops.sample(l.to(gpu), out, temps=ones, uniforms=u)
    assert out.cpu().tolist() == [0, 249, 499]           # equal values are ordered by index
    ops.sample(l.to(gpu), out, temps=ones, top_ks=torch.full((3,), 10, dtype=torch.int32, device=gpu), uniforms=u)
    assert out.cpu().tolist() == [0, 4, 9]
    # zeros of either sign are equal values too
    l[:, 1::3] = -0.0
    ops.sample(l.to(gpu), out, temps=ones, uniforms=u)
    assert out.cpu().tolist() == [0, 249, 499]
    ops.sample(l.to(gpu), out, temps=ones, top_ks=torch.full((3,), 10, dtype=torch.int32, device=gpu), uniforms=u)
    assert out.cpu().tolist() == [0, 4, 9]


def test_repeat_penalty(gpu):
    from tuff_amd.csrc import ops
    l = torch.tensor([[2.0, -2.0, 1.0, 4.0]] * 2)
    recent = torch.tensor([[0, 1, 0, 9], [3, 3, 3, 3]], dtype=torch.int32)
    g = l.to(gpu)
    ops.repeat_penalty(g, recent.to(gpu), torch.tensor([3, 2], dtype=torch.int32, device=gpu),
                       torch.tensor([2.0, 1.0], device=gpu))
    assert g.cpu().tolist() == [[0.5, -4.0, 1.0, 4.0], [2.0, -2.0, 1.0, 4.0]]
