"""A routed mixture of gated feed-forward experts, with an optional expert that every token passes."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, ParamSpec, register_ffn


class MixtureOfExperts(FeedForward):
    """Router logits come from one product with float32 output; a kernel forms the softmax, adds
    the correction for the choice only, picks the `top` experts and their weights; the experts'
    matrices are stacked [experts, ...] when the weights are loaded and every (token, chosen
    expert) pair is multiplied by its own expert's rows on the device, chosen there: nothing of
    the routing is read on the host, so steps are recorded into graphs.  The shared expert is
    the framework's dense gated product; its output is the sum's first term.  From a few
    tokens on, bfloat16 steps list each expert's pairs on the device and run the two products
    per expert on the matrix units, so that an expert's matrices are read once a step."""

    launches_follow_shape = True

    def _t(self, role: str) -> str:
        return self.tensor_name(role)

    def _expert(self, e: int, role: str) -> str:
        return f"{self.name}.e{e}.{role}"

    @property
    def gated(self) -> bool:
        return bool(getattr(self.spec, "gated", True))

    def params(self):
        s, h = self.spec, self.width
        out = []
        for e in range(s.experts):
            if self.gated:
                out.append(ParamSpec(self._expert(e, "gate"), (s.expert_size, h)))
            out += [ParamSpec(self._expert(e, "up"), (s.expert_size, h)),
                    ParamSpec(self._expert(e, "down"), (h, s.expert_size))]
        out.append(ParamSpec(self._t("router"), (s.experts, h)))
        if getattr(s, "router_bias", False):
            out.append(ParamSpec(self._t("router.b"), (s.experts,), init="bias", keep_float32=True))
        if s.correction:
            out.append(ParamSpec(self._t("correction"), (s.experts,), init="bias", keep_float32=True))
        if s.shared_size is not None:
            if self.gated:
                out.append(ParamSpec(f"{self.name}.shared.gate", (s.shared_size, h)))
            out += [ParamSpec(f"{self.name}.shared.up", (s.shared_size, h)),
                    ParamSpec(f"{self.name}.shared.down", (h, s.shared_size))]
            if getattr(s, "shared_gate", False):
                out.append(ParamSpec(f"{self.name}.shared.sg", (1, h)))
        return out

    def check(self, runtime):
        s = self.spec
        if self.gated:
            ops.activation_code(s.activation)
        elif s.activation != "relu_squared":
            raise ValueError(f"{self.name}: experts without a gate are built with the activation 'relu_squared', "
                             f"got {s.activation!r}")
        if getattr(s, "shared_gate", False) and s.shared_size is None:
            raise ValueError(f"{self.name}: a gate of the shared expert needs a shared expert")
        if not 1 <= s.top <= s.experts:
            raise ValueError(f"{self.name}: top {s.top} is outside 1..{s.experts} experts")
        if s.experts > 512 or s.top > 64:
            raise ValueError(f"{self.name}: at most 512 experts and 64 chosen ones, got {s.experts} and {s.top}")
        if s.expert_size < 1 or (s.shared_size is not None and s.shared_size < 1):
            raise ValueError(f"{self.name}: expert sizes must be positive")

    def load(self, tensors, runtime):
        s = self.spec
        stack = lambda role: torch.stack([tensors[self._expert(e, role)] for e in range(s.experts)]).contiguous()  # noqa: E731
        self.w_up, self.w_down = stack("up"), stack("down")
        # experts without a gate: relu(u) * u is the square of relu(u), so the gated kernels take the one
        # matrix in both places (they form its product once where the two are the same)
        self.w_gate = stack("gate") if self.gated else self.w_up
        self.activation = s.activation if self.gated else "relu"
        router = tensors[self._t("router")]
        bias = tensors[self._t("router.b")].to(torch.float32) if getattr(s, "router_bias", False) else None
        self.shared_gate = bool(getattr(s, "shared_gate", False))
        if self.shared_gate:
            # the shared expert's gate is one more row of the router's product (and no bias)
            router = torch.cat([router, tensors[f"{self.name}.shared.sg"].view(1, -1)], dim=0)
            if bias is not None:
                bias = torch.cat([bias, bias.new_zeros(1)])
        self.w_router = runtime.weight(router)
        self.router_bias = None if bias is None else bias.contiguous()
        self.correction = tensors[self._t("correction")].contiguous() if s.correction else None
        self.shared = None
        if s.shared_size is not None and self.gated:
            self.shared = (runtime.gated_weight(tensors[f"{self.name}.shared.gate"], tensors[f"{self.name}.shared.up"]),
                           runtime.weight(tensors[f"{self.name}.shared.down"]))
        elif s.shared_size is not None:
            self.shared = (runtime.weight(tensors[f"{self.name}.shared.up"]),
                           runtime.weight(tensors[f"{self.name}.shared.down"]))
        self.linear = runtime.linear
        self.gated_linear = runtime.gated_linear

    def forward(self, ctx, x: torch.Tensor):
        s = self.spec
        n = x.shape[0]
        logits = ctx.buffer("moe_logits", (n, s.experts + int(self.shared_gate)), torch.float32)
        self.linear(x, self.w_router, logits, bias=self.router_bias)
        chosen = ctx.buffer("moe_chosen", (n, s.top), torch.int32)
        weights = ctx.buffer("moe_weights", (n, s.top), torch.float32)
        ops.moe_route(logits[:, : s.experts], self.correction, s.top, chosen, weights)
        shared_out = None
        if self.shared is not None:
            act = ctx.buffer("moe_shared_act", (n, s.shared_size), ctx.dtype)
            if self.gated:
                self.gated_linear(ctx, x, self.shared[0], act, s.activation)
            else:
                up = ctx.buffer("moe_shared_up", (n, s.shared_size), ctx.dtype)
                self.linear(x, self.shared[0], up)
                ops.activate(up, act, s.activation)
            shared_out = ctx.buffer("moe_shared_out", (n, self.width), ctx.dtype)
            self.linear(act, self.shared[1], shared_out)
        act_buf = ctx.buffer("moe_act", (n * s.top, s.expert_size), ctx.dtype)
        out = ctx.buffer("moe_out", (n, self.width), ctx.dtype)
        scratch = None
        if ops.moe_grouped(n, self.width, s.expert_size, ctx.dtype):
            scratch = ctx.buffer("moe_scratch", (ops.moe_grouped_scratch_bytes(n, self.width, s.experts, s.top),),
                                 torch.uint8)
        ops.moe_experts(x, chosen, weights, self.w_gate, self.w_up, self.w_down, act_buf, out, self.activation,
                        add=shared_out, scratch=scratch,
                        add_gate=logits[:, s.experts] if self.shared_gate else None)
        return out


register_ffn("moe", MixtureOfExperts)
