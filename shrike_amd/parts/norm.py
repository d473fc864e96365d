"""RMSNorm fused with the residual add that precedes it."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import HiddenState, Norm, ParamSpec, register_norm


class RMSNorm(Norm):
    """y = x * rsqrt(mean(x^2) + eps) * (offset + weight) in float32, one cast at the
    end (reference: shrike/models/qwen.py:70-74, where the offset is 0).  A weight that
    is stored around zero (offset 1) gets its offset when it is loaded, in float32."""

    launches_follow_shape = True

    def params(self):
        offset = float(getattr(self.spec, "offset", 0.0))
        return [ParamSpec(self.tensor_name("weight"), (self.width,), init="norm" if offset == 0.0 else "norm_zero",
                          keep_float32=True)]

    def load(self, tensors, runtime):
        self.weight = tensors[self.tensor_name("weight")]
        offset = float(getattr(self.spec, "offset", 0.0))
        if offset != 0.0:
            self.weight = (self.weight.to(torch.float32) + offset).contiguous()
        self.eps = float(self.spec.eps)

    def forward(self, ctx, hidden: HiddenState, rows=None, write_resid=True) -> torch.Tensor:
        n = hidden.resid.shape[0] if rows is None else rows.shape[0]
        out = ctx.buffer(f"normed", (n, self.width), ctx.dtype)
        if hidden.pending is not None and hidden.pending_norm is not None and len(hidden.pending_norm) == 3:
            hidden.settle(ctx)  # an addend with a layer norm of its own joins by that norm's kernel
        if hidden.pending is not None and hidden.pending_norm is not None:
            dweight, deps = hidden.pending_norm
            ops.add_normed_rmsnorm(hidden.resid, hidden.pending, dweight, deps, self.weight, self.eps, out,
                                   rows, write_resid)
        else:
            ops.add_rmsnorm(hidden.resid, hidden.pending, self.weight, self.eps, out, rows, write_resid)
        if write_resid:
            if hidden.pending is not None:
                hidden.cast = None  # the stream has changed under a copy that an earlier kernel left
            hidden.pending = hidden.pending_norm = None
        return out


register_norm("rmsnorm", RMSNorm)


class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * weight + bias in float32, var the mean of the squared
    deviations, one cast at the end.  What is pending joins the stream in the same kernel,
    also where it is normed by a layer norm of its own first (a norm after a sublayer)."""

    launches_follow_shape = True

    def params(self):
        out = [ParamSpec(self.tensor_name("weight"), (self.width,), init="norm", keep_float32=True)]
        if getattr(self.spec, "bias", True):
            out.append(ParamSpec(self.tensor_name("bias"), (self.width,), init="bias", keep_float32=True))
        return out

    def load(self, tensors, runtime):
        self.weight = tensors[self.tensor_name("weight")].contiguous()
        self.bias = tensors[self.tensor_name("bias")].contiguous() if getattr(self.spec, "bias", True) else None
        self.eps = float(self.spec.eps)

    def as_pending(self) -> tuple:
        """What HiddenState.pending_norm takes for an output that this norm brings to the stream."""
        return (self.weight, self.bias, self.eps)

    def normalize_(self, x: torch.Tensor) -> torch.Tensor:
        """x <- norm(x) for float32 rows, in place (a stream that starts normed)."""
        ops.add_layernorm(x, weight=self.weight, bias=self.bias, eps=self.eps, out=x, write_resid=False)
        return x

    def forward(self, ctx, hidden: HiddenState, rows=None, write_resid=True) -> torch.Tensor:
        n = hidden.resid.shape[0] if rows is None else rows.shape[0]
        out = ctx.buffer("normed", (n, self.width), ctx.dtype)
        dnorm = hidden.pending_norm
        if hidden.pending is not None and dnorm is not None and len(dnorm) != 3:
            hidden.settle(ctx)  # an addend with a norm of another kind joins by that norm's kernel
        ops.add_layernorm(hidden.resid, hidden.pending, dnorm=dnorm if hidden.pending is not None else None,
                          weight=self.weight, bias=self.bias, eps=self.eps, out=out, rows=rows,
                          write_resid=write_resid, dtype=ctx.dtype)
        if write_resid:
            if hidden.pending is not None:
                hidden.cast = None  # the stream has changed under a copy that an earlier kernel left
            hidden.pending = hidden.pending_norm = None
        return out


register_norm("layernorm", LayerNorm)
