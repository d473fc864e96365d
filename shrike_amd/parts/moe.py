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

    def params(self):
        s, h = self.spec, self.width
        out = []
        for e in range(s.experts):
            out += [ParamSpec(self._expert(e, "gate"), (s.expert_size, h)),
                    ParamSpec(self._expert(e, "up"), (s.expert_size, h)),
                    ParamSpec(self._expert(e, "down"), (h, s.expert_size))]
        out.append(ParamSpec(self._t("router"), (s.experts, h)))
        if s.correction:
            out.append(ParamSpec(self._t("correction"), (s.experts,), init="bias", keep_float32=True))
        if s.shared_size is not None:
            out += [ParamSpec(f"{self.name}.shared.gate", (s.shared_size, h)),
                    ParamSpec(f"{self.name}.shared.up", (s.shared_size, h)),
                    ParamSpec(f"{self.name}.shared.down", (h, s.shared_size))]
        return out

    def check(self, runtime):
        s = self.spec
        ops.activation_code(s.activation)
        if not 1 <= s.top <= s.experts:
            raise ValueError(f"{self.name}: top {s.top} is outside 1..{s.experts} experts")
        if s.experts > 512 or s.top > 64:
            raise ValueError(f"{self.name}: at most 512 experts and 64 chosen ones, got {s.experts} and {s.top}")
        if s.expert_size < 1 or (s.shared_size is not None and s.shared_size < 1):
            raise ValueError(f"{self.name}: expert sizes must be positive")

    def load(self, tensors, runtime):
        s = self.spec
        stack = lambda role: torch.stack([tensors[self._expert(e, role)] for e in range(s.experts)]).contiguous()  # noqa: E731
        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")
        self.w_router = runtime.weight(tensors[self._t("router")])
        self.correction = tensors[self._t("correction")].contiguous() if s.correction else None
        self.shared = None
        if s.shared_size is not None:
            self.shared = (runtime.gated_weight(tensors[f"{self.name}.shared.gate"], tensors[f"{self.name}.shared.up"]),
                           runtime.weight(tensors[f"{self.name}.shared.down"]))
        self.linear = runtime.linear
        self.gated_linear = runtime.gated_linear

    def forward(self, ctx, x: torch.Tensor):
        s = self.spec
        n = x.shape[0]
        logits = ctx.buffer("moe_logits", (n, s.experts), torch.float32)
        self.linear(x, self.w_router, logits)
        chosen = ctx.buffer("moe_chosen", (n, s.top), torch.int32)
        weights = ctx.buffer("moe_weights", (n, s.top), torch.float32)
        ops.moe_route(logits, self.correction, s.top, chosen, weights)
        shared_out = None
        if self.shared is not None:
            act = ctx.buffer("moe_shared_act", (n, s.shared_size), ctx.dtype)
            self.gated_linear(ctx, x, self.shared[0], act, s.activation)
            shared_out = ctx.buffer("moe_shared_out", (n, self.width), ctx.dtype)
            self.linear(act, self.shared[1], shared_out)
        act_buf = ctx.buffer("moe_act", (n * s.top, s.expert_size), ctx.dtype)
        out = ctx.buffer("moe_out", (n, self.width), ctx.dtype)
        scratch = None
        if ops.moe_grouped(n, self.width, s.expert_size, ctx.dtype):
            scratch = ctx.buffer("moe_scratch", (ops.moe_grouped_scratch_bytes(n, self.width, s.experts, s.top),),
                                 torch.uint8)
        ops.moe_experts(x, chosen, weights, self.w_gate, self.w_up, self.w_down, act_buf, out, s.activation,
                        add=shared_out, scratch=scratch)
        return out


register_ffn("moe", MixtureOfExperts)
