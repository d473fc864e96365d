"""Several mixers side by side on the same input, their outputs normed and averaged."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import CompositeSpec, Mixer, ParamSpec, build_part, register_mixer


class ParallelMixers(Mixer):
    """out = scale * sum over the branches of branch(x) / rms(branch(x)) * weight_branch.

    Every branch is a mixer of its own kind with a cache of its own kind: the cache need is
    the branches' needs side by side (a CompositeSpec), and each branch gets its own part of
    the layer's cache.  The sum is formed in float32 from the branches' outputs (tensors of
    the compute dtype, or the partial sums of split products) by the kernel that norms them
    (the one that adds a normed output to the stream, here with the sum in the stream's place);
    it leaves in float32, as one part, for the kernel that adds it to the stream."""

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.branches = [(sub, build_part("mixer", branch, width, f"{name}.{sub}")) for sub, branch in spec.branches]
        self.parts = tuple(m for _, m in self.branches) + tuple(
            p for _, m in self.branches for p in getattr(m, "parts", ()))

    @property
    def launches_follow_shape(self):
        return all(m.launches_follow_shape for _, m in self.branches)

    @property
    def graph_safe(self):
        return all(m.graph_safe for _, m in self.branches)

    @property
    def state_graph_safe(self):
        return all(m.state_graph_safe for _, m in self.branches if _keeps_state(m.cache_spec()))

    def _weight_name(self, sub: str) -> str:
        return f"{self.name}.{sub}.{self.spec.out_name}"

    def params(self):
        out = [p for _, m in self.branches for p in m.params()]
        return out + [ParamSpec(self._weight_name(sub), (self.width,), init="norm", keep_float32=True)
                      for sub, _ in self.branches]

    def cache_spec(self):
        needs = tuple((sub, m.cache_spec()) for sub, m in self.branches if m.cache_spec() is not None)
        return CompositeSpec(needs) if needs else None

    def check(self, runtime):
        if not self.branches:
            raise ValueError(f"{self.name}: no branches")
        for _, m in self.branches:
            m.check(runtime)

    def load(self, tensors, runtime):
        for _, m in self.branches:
            m.load(tensors, runtime)
        # the scale rides on the weights: scale * (unit * w) = unit * (scale * w)
        self.weights = [(tensors[self._weight_name(sub)].to(torch.float32) * float(self.spec.scale)).contiguous()
                        for sub, _ in self.branches]
        self.eps = float(self.spec.eps)

    def forward(self, ctx, x: torch.Tensor, cache):
        n = x.shape[0]
        total = ctx.buffer("parallel_sum", (1, n, self.width), torch.float32)
        ops.zero_(total)
        for (sub, m), weight in zip(self.branches, self.weights):
            out = m.forward(ctx, x, cache.parts.get(sub) if cache is not None else None)
            # total += out / rms(out) * (scale * weight), row by row, in float32
            ops.add_normed_rmsnorm(total[0], out, weight, self.eps, dtype=ctx.dtype)
        return ops.SplitSum(total)


def _keeps_state(need) -> bool:
    from .base import StateSpec

    return isinstance(need, StateSpec)


register_mixer("parallel_mixers", ParallelMixers)
