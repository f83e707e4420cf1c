"""Projection y = x W^T with W [out, in] row-major, as every projection of the reference
(`dst[row] = W[row, :] . x`, src/lfm25_gpu.cu:148-202).  Several checkpoint tensors with the
same input can be stacked into one weight, so q/k/v or gate/up are one product.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..csrc import ops
from .base import Runtime, WeightDecl


class Linear:
    def __init__(self, names: Sequence[str] | str, in_features: int,
                 out_features: Sequence[int] | int, aliases: Sequence[Sequence[str]] | None = None,
                 swiglu_pair: bool = False, bias: Sequence[str] | str | None = None):
        """swiglu_pair: the two stacked tensors are the gate and the up matrix of a SwiGLU; with
        bfloat16 weights their rows are interleaved so that forward(..., swiglu=True) can apply
        silu(gate) * up in the product's epilogue.
        bias: checkpoint names of a bias vector per stacked tensor ([out] each), y = x W^T + b.  The
        products' epilogues have no bias: it is added by a kernel of its own after the product, and a
        projection with one takes none of the fused ways (activation, convolution or the next norm in
        the product's epilogue); the result is the same function."""
        self.names = [names] if isinstance(names, str) else list(names)
        outs = [out_features] if isinstance(out_features, int) else list(out_features)
        if len(outs) != len(self.names):
            raise ValueError("one output size per stacked tensor")
        self.in_features, self.outs = int(in_features), [int(o) for o in outs]
        self.out_features = sum(self.outs)
        self.aliases = [tuple(a) for a in aliases] if aliases else [()] * len(self.names)
        self.weight = None            # bound: ops.TiledWeight (bfloat16) or a float32 tensor [out, in]
        self.swiglu_pair = bool(swiglu_pair)
        self.weight_grouped = None    # bound, for a conv's input projection: the weight with its rows regrouped
        if self.swiglu_pair and (len(self.names) != 2 or self.outs[0] != self.outs[1]):
            raise ValueError("a SwiGLU pair is two tensors of one shape")
        self.interleaved = False
        self.bias_names = None if bias is None else ([bias] if isinstance(bias, str) else list(bias))
        if self.bias_names is not None and len(self.bias_names) != len(self.names):
            raise ValueError("one bias per stacked tensor")
        self.bias = None              # bound: float32 [out]

    def weight_decls(self) -> list[WeightDecl]:
        decls = [WeightDecl(n, (o, self.in_features), "normal", aliases=a, role="projection")
                 for n, o, a in zip(self.names, self.outs, self.aliases)]
        if self.bias_names is not None:
            decls += [WeightDecl(n, (o,), "normal") for n, o in zip(self.bias_names, self.outs)]
        return decls

    def bind(self, weights: dict[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        ws = [weights[n] for n in self.names]
        if len(ws) == 1:
            self.weight = ws[0]
        else:
            if len({w.dtype for w in ws}) != 1:
                ws = [w.to(torch.float32) for w in ws]
            if self.swiglu_pair and ws[0].dtype == torch.bfloat16 and self.bias_names is None:
                self.weight = torch.stack(ws, dim=1).reshape(self.out_features, self.in_features).contiguous()
                self.interleaved = True
            else:
                self.weight = torch.cat(ws, dim=0).contiguous()
        if self.weight.dtype == torch.bfloat16:
            if self.in_features % 8 != 0:
                raise ValueError(f"{self.names[0]}: the bfloat16 matrix kernels need an input size that is a "
                                 f"multiple of 8, got {self.in_features}")
            self.weight = ops.tile_weight(self.weight)       # the order the kernels stream it in
        if self.bias_names is not None:
            self.bias = torch.cat([weights[n].to(torch.float32).reshape(-1) for n in self.bias_names]).contiguous()

    def group_rows_for_conv(self) -> bool:
        """Call after bind(), for the input projection of a gated short convolution: keeps a second copy of
        the weight with its rows regrouped, so that forward_conv() can run projection and convolution of
        single tokens in one kernel.  False (and nothing kept) where the kernels cannot."""
        w = self.weight
        if not isinstance(w, ops.TiledWeight) or self.out_features % 48 or len(self.names) != 1 or self.bias is not None:
            return False
        self.weight_grouped = ops.tile_weight(ops.conv_group_rows(w.rows()))
        return True

    def forward_conv(self, x, *, conv_w, state, state_slot) -> Optional[torch.Tensor]:
        """x as for forward(), one token a row.  Returns C * conv(B * X) [T, out / 3] in bfloat16 with the
        states shifted, or None where this needs the separate kernels (nothing is touched then).  Up to 32
        rows: one kernel, from the regrouped weight; 33 to 64 rows: the kernel that adds the projection's
        partial tiles runs the convolution."""
        from .norm import PendingNorm
        if self.weight_grouped is None:
            return None
        pending = x if isinstance(x, PendingNorm) else None
        T = pending.shape[0] if pending is not None else x.shape[0]
        if T > ops.CONV64_MAX_ROWS:
            return None
        kw = {}
        if pending is not None:
            if pending.pre is not None:
                x, kw = pending.pre[0], dict(ss=pending.pre[1], eps=pending.norm.eps)
            elif T <= ops.NORMED_MAX_ROWS and pending.rows is None and self.in_features <= ops.NORMED_MAX_K:
                x, kw = pending.x, dict(norm_w=pending.norm.weight_f32, eps=pending.norm.eps)
            else:
                x = pending.tensor()
        if not kw and x.dtype != torch.bfloat16:
            return None
        y = torch.empty(T, self.out_features // 3, dtype=torch.bfloat16, device=self.weight_grouped.device)
        if T <= ops.CONV_MAX_ROWS:
            ops.gemm_conv(x, self.weight_grouped, y, conv_w=conv_w, state=state, state_slot=state_slot, **kw)
        else:
            ops.gemm_conv64(x, self.weight, y, conv_w=conv_w, state=state, state_slot=state_slot, **kw)
        return y

    def forward(self, x, *, out_dtype: Optional[torch.dtype] = None,
                accumulate_into: Optional[torch.Tensor] = None, swiglu: bool = False,
                next_norm=None) -> Optional[torch.Tensor]:
        """x [T, in] in the compute dtype, or a PendingNorm.  Returns a new [T, out] tensor of
        `out_dtype` (default: the compute dtype), or adds into `accumulate_into` (float32) and
        returns None.  swiglu (interleaved pairs only): returns silu(gate) * up, [T, out/2].
        next_norm (with accumulate_into): the norm that reads the sum next; where the kernels can,
        the product leaves it its operand and row sums (norm.announce_operand)."""
        from .norm import PendingNorm
        w = self.weight
        if swiglu and not self.interleaved:
            raise TypeError(f"{self.names[0]}: no fused SwiGLU for this weight")
        pending = x if isinstance(x, PendingNorm) else None
        if pending is not None and self.bias is not None:
            x, pending = pending.tensor(), None        # with a bias: the plain product, then the bias
        if pending is not None:
            T = pending.shape[0]
            # the row scales left by the product before, or the norm inside this product
            want_out = torch.float32 if accumulate_into is not None else (out_dtype or self.rt.dtype)
            fused = w.dtype == torch.bfloat16 and self.in_features % 8 == 0 and (
                ops.gemm_scaled_supported(T, self.out_features, self.in_features, want_out, accumulate_into is not None)
                if pending.pre is not None
                else T <= ops.NORMED_MAX_ROWS and self.in_features <= ops.NORMED_MAX_K)
            if not fused:
                x, pending = pending.tensor(), None
        if pending is None:
            T = x.shape[0]
            if x.dtype != w.dtype:
                # a weight stored in 32-bit stays so: run this product in float32
                if w.dtype != torch.float32:
                    raise TypeError(f"{self.names[0]}: activation {x.dtype} with weight {w.dtype}")
                x32 = torch.empty(x.shape, dtype=torch.float32, device=x.device)
                ops.cast(x, x32)
                x = x32

        def product(out, accumulate=False):
            if pending is not None and pending.pre is not None:
                ops.gemm_scaled(pending.pre[0], pending.pre[1], pending.norm.eps, w, out,
                                accumulate=accumulate, swiglu=swiglu)
            elif pending is not None:
                ops.gemm_normed(pending.x, pending.norm.weight_f32, pending.norm.eps, w, out, rows=pending.rows,
                                accumulate=accumulate, swiglu=swiglu)
            else:
                ops.gemm(x, w, out, accumulate=accumulate, swiglu=swiglu)

        dev = w.device
        if accumulate_into is not None:
            nxt = next_norm if self.bias is None else None      # the sum is not final before the bias is in
            layout = None
            if (nxt is not None and pending is None and w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
                    and self.in_features % 8 == 0):
                layout = ops.gemm_emit_layout(T, self.out_features, self.in_features)
            if layout is not None:
                # the norm that follows reads the sum just made: leave it its operand and row sums
                xw = torch.empty(T, self.out_features, dtype=torch.bfloat16, device=dev)
                ss = torch.empty(layout, dtype=torch.float32, device=dev)
                ops.gemm_accum_emit(x, w, accumulate_into, nxt.weight_f32, xw, ss)
                nxt.announce_operand(accumulate_into, xw, ss)
                return None
            product(accumulate_into, accumulate=True)
            if self.bias is not None:
                ops.add_bias(accumulate_into, self.bias)
            return None
        want = out_dtype or self.rt.dtype
        width = self.out_features // 2 if swiglu else self.out_features
        if w.dtype == torch.float32 and want != torch.float32:
            y32 = torch.empty(T, width, dtype=torch.float32, device=dev)
            product(y32)
            if self.bias is not None:
                ops.add_bias(y32, self.bias)
            y = torch.empty(T, width, dtype=want, device=dev)
            ops.cast(y32, y)
            return y
        if self.bias is not None and want != torch.float32:
            # the bias goes onto the float32 sum, which is then rounded once
            y32 = torch.empty(T, width, dtype=torch.float32, device=dev)
            product(y32)
            ops.add_bias(y32, self.bias)
            y = torch.empty(T, width, dtype=want, device=dev)
            ops.cast(y32, y)
            return y
        y = torch.empty(T, width, dtype=want, device=dev)
        product(y)
        if self.bias is not None:
            ops.add_bias(y, self.bias)
        return y
