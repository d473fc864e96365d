"""Pre-norm residual block: x += mixer(norm(x)); x += ffn(norm(x))."""

from __future__ import annotations

from .base import Block, HiddenState, build_part, register_block


class PreNormResidualBlock(Block):
    """Reference: shrike/models/qwen.py:147-150.  The additions are not done
    here: each part's output is left pending and the next norm adds it."""

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.mixer_norm = build_part("norm", spec.mixer_norm, width, f"{name}.{spec.mixer_norm_name}")
        self.mixer = build_part("mixer", spec.mixer, width, f"{name}.{spec.mixer_name}")
        # a layer without a feed-forward has no second norm either
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = build_part("norm", spec.ffn_norm, width, f"{name}.{spec.ffn_norm_name}")
            self.ffn = build_part("ffn", spec.ffn, width, f"{name}.{spec.ffn_name}")
        self.parts = tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None)

    def params(self):
        return [p for part in self.parts for p in part.params()]

    def check(self, runtime):
        for part in self.parts:
            part.check(runtime)

    @property
    def graph_safe(self):
        return all(part.graph_safe for part in self.parts)

    @property
    def launches_follow_shape(self):
        return all(part.launches_follow_shape for part in self.parts)

    def load(self, tensors, runtime):
        for part in self.parts:
            part.load(tensors, runtime)

    def forward(self, ctx, hidden: HiddenState, cache) -> None:
        x = self.mixer_norm.forward(ctx, hidden)
        hidden.pending = self.mixer.forward(ctx, x, cache)
        if self.ffn is None:
            return
        x = self.ffn_norm.forward(ctx, hidden)
        hidden.pending = self.ffn.forward(ctx, x)


register_block("prenorm_residual", PreNormResidualBlock)


class ParallelResidualBlock(Block):
    """h = norm(x); x += mixer(h) + ffn(h); then the layer's side input, if it has
    one, adds to x from the step's tokens.  One norm feeds both sublayers.  The two
    outputs (tensors, or partial sums of split products) are added to the float32
    stream by one kernel, which also leaves the stream in the compute dtype for the
    side input's first product."""

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.norm = build_part("norm", spec.norm, width, f"{name}.{spec.norm_name}")
        self.mixer = build_part("mixer", spec.mixer, width, f"{name}.{spec.mixer_name}")
        self.ffn = build_part("ffn", spec.ffn, width, f"{name}.{spec.ffn_name}") if spec.ffn is not None else None
        self.side = build_part("side", spec.side, width, f"{name}.{spec.side_name}") if spec.side is not None else None
        self.parts = tuple(p for p in (self.norm, self.mixer, self.ffn, self.side) if p is not None)

    def params(self):
        return [p for part in self.parts for p in part.params()]

    def check(self, runtime):
        for part in self.parts:
            part.check(runtime)

    @property
    def graph_safe(self):
        return all(part.graph_safe for part in self.parts)

    @property
    def launches_follow_shape(self):
        return all(part.launches_follow_shape for part in self.parts)

    def load(self, tensors, runtime):
        for part in self.parts:
            part.load(tensors, runtime)

    def forward(self, ctx, hidden: HiddenState, cache) -> None:
        from ..kernels import ops

        h = self.norm.forward(ctx, hidden)
        mixed = self.mixer.forward(ctx, h, cache)
        fed = self.ffn.forward(ctx, h) if self.ffn is not None else None
        if self.side is None and fed is None:
            hidden.pending = mixed  # the next norm adds it
            return
        x = ctx.buffer("stream_cast", hidden.resid.shape, ctx.dtype) if self.side is not None else None
        ops.add_deltas(hidden.resid, mixed, fed, cast=x, dtype=ctx.dtype)
        if self.side is not None:
            self.side.forward(ctx, hidden, x)


register_block("parallel_residual", ParallelResidualBlock)


class SandwichResidualBlock(Block):
    """x += post(mixer(pre(x))); x += post'(ffn(pre'(x))): a norm before and after each
    sublayer.  Nothing is added here: a sublayer's output stays pending together with the
    norm that brings it to the stream, and the next kernel that reads the stream (the next
    norm, or whatever follows the block) norms and adds it in the same pass."""

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.mixer_norm = build_part("norm", spec.mixer_norm, width, f"{name}.{spec.mixer_norm_name}")
        self.mixer = build_part("mixer", spec.mixer, width, f"{name}.{spec.mixer_name}")
        self.mixer_post = build_part("norm", spec.mixer_post, width, f"{name}.{spec.mixer_post_name}")
        self.ffn_norm = self.ffn = self.ffn_post = None
        if spec.ffn is not None:
            self.ffn_norm = build_part("norm", spec.ffn_norm, width, f"{name}.{spec.ffn_norm_name}")
            self.ffn = build_part("ffn", spec.ffn, width, f"{name}.{spec.ffn_name}")
            self.ffn_post = build_part("norm", spec.ffn_post, width, f"{name}.{spec.ffn_post_name}")
        listed = (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post)
        self.parts = tuple(p for p in listed if p is not None) + tuple(getattr(self.mixer, "parts", ()))

    def params(self):
        own = (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post)
        return [p for part in own if part is not None for p in part.params()]

    def check(self, runtime):
        for part in (self.mixer_post, self.ffn_post):
            if part is not None and not hasattr(part, "as_pending"):
                raise ValueError(f"{self.name}: the norm after a sublayer must be one that a pending output "
                                 "can carry (layernorm)")
        for part in (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post):
            if part is not None:
                part.check(runtime)

    @property
    def graph_safe(self):
        return all(part.graph_safe for part in self.parts)

    @property
    def launches_follow_shape(self):
        return all(part.launches_follow_shape for part in self.parts)

    def load(self, tensors, runtime):
        for part in (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post):
            if part is not None:
                part.load(tensors, runtime)

    def forward(self, ctx, hidden: HiddenState, cache) -> None:
        x = self.mixer_norm.forward(ctx, hidden)
        hidden.pending = self.mixer.forward(ctx, x, cache)
        hidden.pending_norm = self.mixer_post.as_pending()
        if self.ffn is None:
            return
        x = self.ffn_norm.forward(ctx, hidden)
        hidden.pending = self.ffn.forward(ctx, x)
        hidden.pending_norm = self.ffn_post.as_pending()


register_block("sandwich_residual", SandwichResidualBlock)
