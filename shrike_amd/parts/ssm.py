"""Mixers whose cache is a state of fixed size per request: the selective scan of Mamba and
retention (linear attention with a fixed decay per head)."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, ParamSpec, PositionEncoding, StateSpec, build_part, register_mixer


class SelectiveScan(Mixer):
    """in-projection -> [u | z]; u through a short causal convolution and SiLU; W_x u -> [dt | B |
    C] in float32; dt through its own small matrix, a bias and softplus (float32); the scan;
    y * silu(z); out-projection.

    The projections, the convolution and their activations have the compute dtype; step sizes,
    decays, exponentials, B, C and the state are float32.  A request's state slot holds S
    [inner, state] and the convolution's last taps - 1 inputs; both are reached on the device
    through ctx.state_slots, and a sequence whose first row of the step is at position 0
    starts from zeros whatever the slot held."""

    launches_follow_shape = True
    state_graph_safe = True

    def _t(self, role: str) -> str:
        return self.tensor_name(role)

    def params(self):
        s, h = self.spec, self.width
        return [
            ParamSpec(self._t("in"), (2 * s.inner, h)),
            ParamSpec(self._t("conv"), (s.inner, s.conv), init="bias", keep_float32=True),
            ParamSpec(self._t("conv.b"), (s.inner,), init="bias", keep_float32=True),
            ParamSpec(self._t("x"), (s.dt_rank + 2 * s.state, s.inner)),
            ParamSpec(self._t("dt"), (s.inner, s.dt_rank), keep_float32=True),
            ParamSpec(self._t("dt.b"), (s.inner,), init="bias", keep_float32=True),
            ParamSpec(self._t("A_log"), (s.inner, s.state), init="log_rate", keep_float32=True),
            ParamSpec(self._t("D"), (s.inner,), init="norm", keep_float32=True),
            ParamSpec(self._t("o"), (h, s.inner)),
        ]

    def state_floats(self) -> int:
        s = self.spec
        return s.inner * s.state + (s.conv - 1) * s.inner

    def cache_spec(self):
        return StateSpec((self.state_floats(),), "float32")

    def check(self, runtime):
        s = self.spec
        if min(s.inner, s.state, s.dt_rank, s.conv) < 1:
            raise ValueError(f"{self.name}: inner, state, dt_rank and conv must be positive")
        if s.state > 512 or s.conv > 64 or s.dt_rank > 1024:
            raise ValueError(f"{self.name}: at most 512 states a channel, 64 taps and a step-size rank of 1024, got "
                             f"{s.state}, {s.conv} and {s.dt_rank}")
        if ops.selective_scan_state_floats(s.inner, s.state, s.conv) != self.state_floats():
            raise RuntimeError(f"{self.name}: the kernel's state layout and the cache's size disagree")

    def load(self, tensors, runtime):
        self.w_in = runtime.weight(tensors[self._t("in")])
        self.taps = tensors[self._t("conv")].contiguous()
        self.conv_bias = tensors[self._t("conv.b")].contiguous()
        self.w_x = runtime.weight(tensors[self._t("x")])
        self.w_dt = tensors[self._t("dt")].t().contiguous()  # [dt_rank, inner]: channels are neighbours in memory
        self.dt_bias = tensors[self._t("dt.b")].contiguous()
        self.a_log = tensors[self._t("A_log")].contiguous()
        self.skip = tensors[self._t("D")].contiguous()
        self.w_o = runtime.weight(tensors[self._t("o")])
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred

    def forward(self, ctx, x: torch.Tensor, cache):
        s = self.spec
        n = x.shape[0]
        state = cache.state_padded if cache.state_padded is not None else cache.state
        uz = ctx.buffer("scan_in", (n, 2 * s.inner), ctx.dtype)
        self.linear(x, self.w_in, uz)
        u = ctx.buffer("scan_u", (n, s.inner), ctx.dtype)
        ops.conv_silu(uz, self.taps, self.conv_bias, ctx.positions, ctx.token_seq, ctx.cu_q, ctx.state_slots,
                      state, s.state, u)
        low = ctx.buffer("scan_low", (n, s.dt_rank + 2 * s.state), torch.float32)
        self.linear(u, self.w_x, low)
        dt = ctx.buffer("scan_dt", (n, s.inner), torch.float32)
        ops.dt_softplus(low, self.w_dt, self.dt_bias, dt)
        gated = ctx.buffer("scan_gated", (n, s.inner), ctx.dtype)
        ops.selective_scan(dt, u, low, s.dt_rank, s.dt_rank + s.state, uz[:, s.inner:], self.a_log, self.skip,
                           s.state, s.conv, uz, ctx.positions, ctx.cu_q, ctx.state_slots, state, gated, ctx.num_seqs)
        return self.linear_deferred(ctx, "scan_out", gated, self.w_o)


register_mixer("selective_scan", SelectiveScan)


class Retention(Mixer):
    """One product yields queries, keys, values and the output gate of a token in float32;
    queries and keys are rotated (the spec's position encoding, applied to float32 rows) and
    the keys scaled; the scan carries S per head in the request's state slot (float32); the
    readout is brought to unit root mean square per head, gated by SiLU of the gate
    projection, and projected."""

    launches_follow_shape = True
    state_graph_safe = True

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.position = build_part("position", spec.position, width, name) if spec.position is not None else None

    def _t(self, role: str) -> str:
        return self.tensor_name(role)

    def params(self):
        s, h = self.spec, self.width
        qk, v = s.num_heads * s.head_dim, s.num_heads * s.value_dim
        return [ParamSpec(self._t("q"), (qk, h)), ParamSpec(self._t("k"), (qk, h)), ParamSpec(self._t("v"), (v, h)),
                ParamSpec(self._t("g"), (v, h)), ParamSpec(self._t("o"), (h, v))]

    def state_floats(self) -> int:
        s = self.spec
        return s.num_heads * s.value_dim * s.head_dim

    def cache_spec(self):
        return StateSpec((self.state_floats(),), "float32")

    def check(self, runtime):
        s = self.spec
        if min(s.num_heads, s.head_dim, s.value_dim) < 1:
            raise ValueError(f"{self.name}: heads, head_dim and value_dim must be positive")
        if s.head_dim > 1024:
            raise ValueError(f"{self.name}: head_dim {s.head_dim} is more than the 1024 the scan kernel holds")
        if len(s.decay) != s.num_heads:
            raise ValueError(f"{self.name}: {len(s.decay)} decays for {s.num_heads} heads")
        if self.position is not None:
            if type(self.position).rotary_table is PositionEncoding.rotary_table \
                    or getattr(self.position, "adjacent_pairs", False):
                raise ValueError(f"{self.name}: retention rotates pairs (i, i + rot_dim / 2) only")
        if ops.retention_state_floats(s.num_heads, s.head_dim, s.value_dim) != self.state_floats():
            raise RuntimeError(f"{self.name}: the kernel's state layout and the cache's size disagree")

    def load(self, tensors, runtime):
        s = self.spec
        self.w_in = runtime.weight(torch.cat([tensors[self._t(r)] for r in ("q", "k", "v", "g")], dim=0))
        qk, v = s.num_heads * s.head_dim, s.num_heads * s.value_dim
        self.offsets = {"q": 0, "k": qk, "v": 2 * qk, "g": 2 * qk + v}
        self.in_width = 2 * qk + 2 * v
        self.decay = torch.tensor([float(d) for d in s.decay], dtype=torch.float32, device=runtime.device)
        self.w_o = runtime.weight(tensors[self._t("o")])
        if self.position is not None:
            self.position.load(tensors, runtime)
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred

    def forward(self, ctx, x: torch.Tensor, cache):
        s, off = self.spec, self.offsets
        n = x.shape[0]
        proj = ctx.buffer("retention_proj", (n, self.in_width), torch.float32)
        self.linear(x, self.w_in, proj)
        inv_freq, rot_dim = self.position.rotary_table() if self.position is not None else (None, 0)
        if rot_dim:
            ops.rotate_half_rows(proj, off["q"], s.num_heads, s.head_dim, rot_dim, inv_freq, ctx.positions, 1.0)
        ops.rotate_half_rows(proj, off["k"], s.num_heads, s.head_dim, rot_dim, inv_freq, ctx.positions,
                             float(s.head_dim) ** -0.5)
        read = ctx.buffer("retention_read", (n, s.num_heads * s.value_dim), torch.float32)
        state = cache.state_padded if cache.state_padded is not None else cache.state
        ops.retention_scan(proj, off["q"], off["k"], off["v"], self.decay, ctx.num_seqs, s.num_heads, s.head_dim,
                           s.value_dim, ctx.positions, ctx.cu_q, ctx.state_slots, state, read)
        gated = ctx.buffer("retention_gated", (n, s.num_heads * s.value_dim), ctx.dtype)
        ops.headnorm_gate(read, proj[:, off["g"]:], None, s.eps, gated, s.num_heads, s.value_dim, gate_act="silu")
        return self.linear_deferred(ctx, "retention_out", gated, self.w_o)


register_mixer("retention", Retention)
