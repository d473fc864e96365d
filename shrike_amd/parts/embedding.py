"""Token embedding: the residual stream starts as the table's rows."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Embedding, ParamSpec, StateSpec, build_part, register_embedding


class TokenEmbedding(Embedding):
    """x[n] = table[token_ids[n]] * scale, widened to float32 (reference:
    shrike/models/qwen.py:156,161, which has no scale: the spec's default of 1)."""

    launches_follow_shape = True

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        norm = getattr(spec, "norm", None)
        # a norm that the looked-up rows pass before they become the stream
        self.norm = build_part("norm", norm, width, spec.norm_name) if norm is not None else None

    def params(self):
        own = [ParamSpec(self.tensor_name("weight"), (self.spec.vocab_size, self.width), init="embedding")]
        return own + (self.norm.params() if self.norm is not None else [])

    def check(self, runtime):
        if self.norm is not None and not hasattr(self.norm, "normalize_"):
            raise ValueError(f"{self.name}: the embedding's norm must be one that norms float32 rows in place "
                             "(layernorm)")

    def load(self, tensors, runtime):
        self.table = tensors[self.tensor_name("weight")]
        self.scale = float(getattr(self.spec, "scale", 1.0))
        if self.norm is not None:
            self.norm.load(tensors, runtime)

    def forward(self, ctx, into: str = "resid") -> torch.Tensor:
        """Into the workspace buffer `into`; a model that needs the embedding's output
        again later asks for it a second time under another name."""
        resid = ctx.buffer(into, (ctx.num_tokens, self.width), torch.float32)
        ops.embed(self.table, ctx.token_ids, resid, self.scale)
        if self.norm is not None:
            self.norm.normalize_(resid)
        return resid


register_embedding("token_lookup", TokenEmbedding)


class PairHashEmbedding(Embedding):
    """x[n] = table[token] + pairs[(previous token * mul_prev + token * mul_cur) mod buckets],
    summed in float32; the first token of a sequence takes the pair table's last row.  The
    token before a step's first token is part of the request's state: it lives in the
    request's state slot on the device (one int32), where the kernel reads it and leaves
    the step's last token, so steps replayed from graphs or launched ahead of the host find
    it without the host's help."""

    launches_follow_shape = True
    state_graph_safe = True

    def params(self):
        s = self.spec
        return [ParamSpec(self.tensor_name("weight"), (s.vocab_size, self.width), init="embedding"),
                ParamSpec(s.pair_name, (s.buckets + 1, self.width), init="embedding")]

    def cache_spec(self):
        return StateSpec((1,), "int32")

    def check(self, runtime):
        s = self.spec
        if s.buckets < 1:
            raise ValueError(f"{self.name}: buckets must be positive, got {s.buckets}")
        if max(abs(int(s.mul_prev)), abs(int(s.mul_cur))) >= 1 << 31:
            raise ValueError(f"{self.name}: the hash's multipliers must fit 32 bits")

    def load(self, tensors, runtime):
        self.table = tensors[self.tensor_name("weight")]
        self.pairs = tensors[self.spec.pair_name]

    def forward(self, ctx, into: str = "resid", cache=None) -> torch.Tensor:
        if cache is None or into != "resid":
            raise RuntimeError(f"{self.name}: the pair embedding runs once a step, with its state")
        s = self.spec
        resid = ctx.buffer(into, (ctx.num_tokens, self.width), torch.float32)
        state = cache.state_padded if cache.state_padded is not None else cache.state
        ops.embed_pairs(self.table, self.pairs, ctx.token_ids, ctx.positions, ctx.token_seq, ctx.cu_q,
                        ctx.state_slots, state.view(-1), resid, s.buckets, s.mul_prev, s.mul_cur)
        return resid


register_embedding("token_pair_hash", PairHashEmbedding)
