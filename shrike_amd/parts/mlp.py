"""Dense gated feed-forward (SwiGLU, or its sibling with a GELU gate)."""

from __future__ import annotations

import torch

from .base import FeedForward, ParamSpec, register_ffn


class SwiGLU(FeedForward):
    """down(act(gate(x)) * up(x)) without biases; act is the spec's activation,
    SiLU for the reference's model (shrike/models/qwen.py:131-136).  gate and up
    are joined into one weight at load time, so that one product yields the
    activated values."""

    launches_follow_shape = True

    def params(self):
        inter, h = self.spec.intermediate_size, self.width
        return [
            ParamSpec(self.tensor_name("gate", "gate_proj.weight"), (inter, h)),
            ParamSpec(self.tensor_name("up", "up_proj.weight"), (inter, h)),
            ParamSpec(self.tensor_name("down", "down_proj.weight"), (h, inter)),
        ]

    def check(self, runtime):
        from ..kernels import ops

        ops.activation_code(self.spec.activation)  # raises for an activation the kernels lack
        limit = getattr(self.spec, "limit", None)
        if limit is not None and not limit > 0:
            raise ValueError(f"{self.name}: limit must be positive, got {limit}")

    def load(self, tensors, runtime):
        self.inter = int(self.spec.intermediate_size)
        self.activation = self.spec.activation
        self.limit = getattr(self.spec, "limit", None)
        self.up_shift = float(getattr(self.spec, "up_shift", 0.0))
        self.w_gate_up = runtime.gated_weight(
            tensors[self.tensor_name("gate", "gate_proj.weight")], tensors[self.tensor_name("up", "up_proj.weight")],
            self.activation, self.limit, self.up_shift,
        )
        self.w_down = runtime.weight(tensors[self.tensor_name("down", "down_proj.weight")])
        self.linear_deferred = runtime.linear_deferred
        self.gated_linear = runtime.gated_linear

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        n = x.shape[0]
        act = ctx.buffer("ffn_act", (n, self.inter), ctx.dtype)
        self.gated_linear(ctx, x, self.w_gate_up, act, self.activation, self.limit, self.up_shift)
        # the norm that follows adds the output to the residual stream and can add up parts
        return self.linear_deferred(ctx, "ffn_out", act, self.w_down)


register_ffn("swiglu", SwiGLU)


class DenseFFN(FeedForward):
    """down(act(up(x))) without biases.  The xIELU activation has two learned numbers
    per layer (a tensor of two elements, p and q): softplus(p) scales the quadratic
    branch for z > 0, 1/2 + softplus(q) the flattening branch for z <= 0; both are
    formed once, in float32, when the weights are loaded."""

    launches_follow_shape = True

    def params(self):
        inter, h = self.spec.intermediate_size, self.width
        return [
            ParamSpec(self.tensor_name("up", "up_proj.weight"), (inter, h)),
            ParamSpec(self.tensor_name("down", "down_proj.weight"), (h, inter)),
            ParamSpec(self.tensor_name("act", "act"), (2,), init="bias", keep_float32=True),
        ]

    def check(self, runtime):
        if self.spec.activation != "xielu":
            raise ValueError(f"{self.name}: the dense feed-forward's activation must be 'xielu', "
                             f"got {self.spec.activation!r}")

    def load(self, tensors, runtime):
        self.inter = int(self.spec.intermediate_size)
        self.w_up = runtime.weight(tensors[self.tensor_name("up", "up_proj.weight")])
        self.w_down = runtime.weight(tensors[self.tensor_name("down", "down_proj.weight")])
        p, q = torch.nn.functional.softplus(tensors[self.tensor_name("act", "act")].to(torch.float32)).tolist()
        self.a_pos, self.a_neg = float(p), 0.5 + float(q)
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        from ..kernels import ops

        n = x.shape[0]
        up = ctx.buffer("ffn_up", (n, self.inter), ctx.dtype)
        self.linear(x, self.w_up, up)
        act = ctx.buffer("ffn_act", (n, self.inter), ctx.dtype)
        ops.xielu(up, act, self.a_pos, self.a_neg)
        return self.linear_deferred(ctx, "ffn_out", act, self.w_down)


register_ffn("dense_act", DenseFFN)
