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


class PostNormResidualBlock(Block):
    """x <- norm1(alpha x + s1 * mixer(x)); x <- norm2(alpha x + s2 * ffn(x)): the norm stands
    after the sum, the stream is what the norm leaves, and the sublayers read the stream itself.
    One kernel per sublayer forms the scaled sum in float32 (adding up the parts of a split
    product in order), norms it, stores it as the float32 stream and leaves it in the compute
    dtype for the products that read it next.  A layer without a feed-forward has no second norm
    unless its spec names one and the weight file holds that norm's tensor: then the stream
    passes it with nothing added, x <- norm2(alpha x)."""

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.mixer = build_part("mixer", spec.mixer, width, f"{name}.{spec.mixer_name}")
        self.mixer_norm = build_part("norm", spec.mixer_norm, width, f"{name}.{spec.mixer_norm_name}")
        self.ffn = self.ffn_norm = None
        if spec.ffn is not None:
            self.ffn = build_part("ffn", spec.ffn, width, f"{name}.{spec.ffn_name}")
        if spec.ffn is not None or spec.ffn_norm is not None:
            self.ffn_norm = build_part("norm", spec.ffn_norm, width, f"{name}.{spec.ffn_norm_name}")
        self.parts = tuple(p for p in (self.mixer, self.mixer_norm, self.ffn, self.ffn_norm) if p is not None)
        self.parts += tuple(getattr(self.mixer, "parts", ()))
        self.mixer_scale = self.ffn_scale = None

    def _own(self):
        return tuple(p for p in (self.mixer, self.mixer_norm, self.ffn, self.ffn_norm) if p is not None)

    def _scale_names(self):
        s = self.spec
        if not s.layer_scale:
            return ()
        return (f"{self.name}.{s.mixer_scale_name}",) + ((f"{self.name}.{s.ffn_scale_name}",) if self.ffn_norm else ())

    def params(self):
        from dataclasses import replace

        from .base import ParamSpec

        out = []
        for part in self._own():
            # the second norm of a layer without a feed-forward: there only if the file has it
            loose = part is self.ffn_norm and self.ffn is None
            out += [replace(p, optional=True) if loose else p for p in part.params()]
        for i, n in enumerate(self._scale_names()):
            out.append(ParamSpec(n, (self.width,), init="norm", keep_float32=True, optional=i == 1 and self.ffn is None))
        return out

    def check(self, runtime):
        for part in (self.mixer_norm, self.ffn_norm):
            if part is not None and (getattr(part.spec, "kind", None) != "rmsnorm"):
                raise ValueError(f"{self.name}: the norm after a sum must be an RMS norm (rmsnorm)")
        for part in self._own():
            part.check(runtime)

    @property
    def graph_safe(self):
        return all(part.graph_safe for part in self.parts)

    @property
    def launches_follow_shape(self):
        return all(part.launches_follow_shape for part in self.parts)

    def load(self, tensors, runtime):
        if self.ffn is None and self.ffn_norm is not None and any(p.name not in tensors for p in self.ffn_norm.params()):
            self.ffn_norm = None  # the file has no second norm for this layer: the stream does not pass one
        for part in self._own():
            part.load(tensors, runtime)
        names = self._scale_names()
        if names:
            self.mixer_scale = tensors[names[0]].contiguous()
            self.ffn_scale = tensors[names[1]].contiguous() if self.ffn is not None else None
        self.alpha = float(self.spec.alpha)

    def forward(self, ctx, hidden: HiddenState, cache) -> None:
        import torch

        from ..kernels import ops

        hidden.settle(ctx)
        in_float32 = ctx.dtype == torch.float32
        x = hidden.resid if in_float32 else hidden.cast
        if x is None:
            x = ctx.buffer("stream_cast", hidden.resid.shape, ctx.dtype)
            ops.cast_rows(hidden.resid, x)
        out = None if in_float32 else ctx.buffer("stream_cast", hidden.resid.shape, ctx.dtype)
        mixed = self.mixer.forward(ctx, x, cache)
        ops.postnorm(hidden.resid, mixed, self.alpha, self.mixer_scale, self.mixer_norm.weight, self.mixer_norm.eps,
                     cast=out, dtype=ctx.dtype)
        if self.ffn_norm is not None:
            fed = None
            if self.ffn is not None:
                fed = self.ffn.forward(ctx, hidden.resid if in_float32 else out)
            ops.postnorm(hidden.resid, fed, self.alpha, self.ffn_scale, self.ffn_norm.weight, self.ffn_norm.eps,
                         cast=out, dtype=ctx.dtype)
        hidden.cast = out


register_block("postnorm_residual", PostNormResidualBlock)
