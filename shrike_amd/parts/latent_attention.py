"""Attention whose queries, keys and values come through low-rank latents."""

from __future__ import annotations

import torch

from ..kernels import ops
from .attention import compute_units
from .base import PAGE, Mixer, PagedSpec, PageTensor, ParamSpec, register_mixer


def latent_cache_spec(kv_rank: int, rot_dim: int, window: int | None = None, chunk: int | None = None) -> PagedSpec:
    """What a token keeps: its normed key/value latent followed by the rotated key part
    that all heads share, one row [kv_rank + rot_dim] per token, rows of a page side by
    side.  The heads' keys and values are never materialised."""
    return PagedSpec(tensors=(PageTensor("latent", (PAGE, kv_rank + rot_dim)),), window=window, chunk=chunk)


class LatentAttention(Mixer):
    """The heads' key and value matrices are folded around the attention instead of
    being applied to every cached token: with k_plain = W_uk_h c, the score's unrotated
    part q_plain . k_plain equals (W_uk_h^T q_plain) . c, and sum_j p_j W_uv_h c_j equals
    W_uv_h (sum_j p_j c_j).  So a step runs

        down = [W_dq; W_dkv] x                       one product
        c_q, row = norms, rotation, cache write       latent_prepare
        q = W_uq c_q                                  product
        q' = [W_uk_h^T q_plain_h | rot(q_rot_h)]      batched product per head + rotate_heads
        o' = attention of q' over the rows, values = the rows' latents
        o = W_uv_h o'_h                               batched product per head
        y = W_o o                                     product

    and the attention itself is that of one shared key/value head of size kv_rank +
    rot_dim: what is read per cached token does not grow with the number of heads.  With the
    spec's output gate, o is multiplied by sigmoid(W_g x) before the last product."""

    launches_follow_shape = True

    def _t(self, role: str) -> str:
        return self.tensor_name(role)

    def params(self):
        s, h = self.spec, self.width
        H = s.num_heads
        gate = [ParamSpec(self._t("g"), (H * s.value_dim, h))] if getattr(s, "output_gate", False) else []
        return gate + [
            ParamSpec(self._t("dq"), (s.q_rank, h)),
            ParamSpec(self._t("dq.norm"), (s.q_rank,), init="norm", keep_float32=True),
            ParamSpec(self._t("uq"), (H * (s.head_dim + s.rot_dim), s.q_rank)),
            ParamSpec(self._t("dkv"), (s.kv_rank + s.rot_dim, h)),
            ParamSpec(self._t("dkv.norm"), (s.kv_rank,), init="norm", keep_float32=True),
            ParamSpec(self._t("uk"), (H * s.head_dim, s.kv_rank)),
            ParamSpec(self._t("uv"), (H * s.value_dim, s.kv_rank)),
            ParamSpec(self._t("o"), (h, H * s.value_dim)),
        ]

    def cache_spec(self):
        s = self.spec
        return latent_cache_spec(s.kv_rank, s.rot_dim, s.window, s.chunk)

    def check(self, runtime):
        s = self.spec
        for name in ("num_heads", "head_dim", "value_dim", "q_rank", "kv_rank"):
            if getattr(s, name) < 1:
                raise ValueError(f"{self.name}: {name} must be positive, got {getattr(s, name)}")
        if s.rot_dim < 0 or s.rot_dim % 2:
            raise ValueError(f"{self.name}: rot_dim must be even, got {s.rot_dim}")
        if s.rotated is not None and (s.rotated < 0 or s.rotated % 2 or s.rotated > s.rot_dim):
            raise ValueError(f"{self.name}: {s.rotated} rotated elements do not fit a rotated part of {s.rot_dim}")
        if s.kv_rank + s.rot_dim > 1024:
            raise ValueError(f"{self.name}: a cached row of {s.kv_rank + s.rot_dim} elements is more than the "
                             "attention kernel's 1024")
        if s.window is not None and s.window < 1:
            raise ValueError(f"{self.name}: window must be positive, got {s.window}")

    def prepare(self, shape) -> None:
        """Among how many workgroups each token's rows are shared on the matrix-instruction
        path: few tokens with thousands of rows each (single tokens of long sequences) would
        leave most of the chip idle.  From the step's shape alone (token count and longest
        context rounded up to powers of two), so that a graph's steps all decide alike."""
        s = self.spec
        key = ("latent_attention", s.num_heads, s.kv_rank, s.rot_dim, s.window, s.chunk)
        if key in shape.notes:
            return
        nsplit = 1
        if self.mfma:
            tokens, reach = 1, int(shape.ctx_lens.max())
            while tokens < shape.num_tokens:
                tokens *= 2
            for bound in (s.window, s.chunk):
                if bound:
                    reach = min(reach, bound)
            keys = 64
            while keys < reach:
                keys *= 2
            nsplit = max(1, min(2 * compute_units() // tokens, keys // 128, 64))
        # a step with prompt portions: neighbouring tokens may share a workgroup (and what it stages)
        group = 1 if shape.num_decode == shape.num_seqs else 4
        shape.notes[key] = (nsplit, group)
        shape.launch_key.append((key, nsplit, group))

    def load(self, tensors, runtime):
        s = self.spec
        H = s.num_heads
        self.mfma = runtime.dtype == torch.bfloat16 and ops.latent_attention_supports_mfma(
            H, s.kv_rank + s.rot_dim, s.kv_rank)
        self.w_down = runtime.weight(torch.cat([tensors[self._t("dq")], tensors[self._t("dkv")]], dim=0))
        self.q_norm = tensors[self._t("dq.norm")]
        self.kv_norm = tensors[self._t("dkv.norm")]
        self.w_uq = runtime.weight(tensors[self._t("uq")])
        # per head [kv_rank, head_dim]: the transpose of the head's key matrix, so that the
        # batched product maps a query's unrotated part into the latent's space
        self.w_uk_t = tensors[self._t("uk")].view(H, s.head_dim, s.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[self._t("uv")].view(H, s.value_dim, s.kv_rank).contiguous()
        self.w_o = runtime.weight(tensors[self._t("o")])
        self.w_gate = runtime.weight(tensors[self._t("g")]) if getattr(s, "output_gate", False) else None
        d = int(s.rot_dim)
        self.inv_freq = None
        if d:
            # one rate per pair of the rotated part; pairs beyond the first `rotated` elements
            # get the rate 0: they turn by nothing and pass unchanged
            turned = d if s.rotated is None else int(s.rotated)
            rates = torch.zeros(d // 2, dtype=torch.float64)
            rates[: turned // 2] = float(s.rot_theta) ** (-torch.arange(0, turned, 2, dtype=torch.float64) / turned)
            self.inv_freq = rates.to(torch.float32).to(runtime.device)
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        s = self.spec
        n, H = x.shape[0], s.num_heads
        key_dim = s.kv_rank + s.rot_dim
        q_head = s.head_dim + s.rot_dim
        tables = ctx.block_tables[cache.group]
        down = ctx.buffer("latent_down", (n, s.q_rank + key_dim), ctx.dtype)
        self.linear(x, self.w_down, down)
        c_q = ctx.buffer("latent_cq", (n, s.q_rank), ctx.dtype)
        ops.latent_prepare(down, s.q_rank, s.kv_rank, s.rot_dim, self.q_norm, self.kv_norm, s.eps, self.inv_freq,
                           ctx.positions, ctx.token_seq, tables, c_q, cache.pools["latent"], cache.page_size,
                           write_kv=cache.owned)
        q = ctx.buffer("latent_q", (n, H * q_head), ctx.dtype)
        self.linear(c_q, self.w_uq, q)
        folded = ctx.buffer("latent_q_folded", (n, H * key_dim), ctx.dtype)
        ops.gemm_batched(q, self.w_uk_t, folded, H, q_head, key_dim)
        ops.rotate_heads(q, q_head, s.head_dim, folded, key_dim, s.kv_rank, H, s.rot_dim, self.inv_freq,
                         ctx.positions)
        mixed = ctx.buffer("latent_mixed", (n, H * s.kv_rank), ctx.dtype)
        if self.mfma:
            nsplit, group = ctx.notes[("latent_attention", H, s.kv_rank, s.rot_dim, s.window, s.chunk)]
            partial = None
            if nsplit > 1:
                partial = ctx.buffer("latent_partial", (n * H * nsplit * (s.kv_rank + 2),), torch.float32)
            ops.latent_attention_mfma(folded, mixed, H, key_dim, s.kv_rank, ctx.positions, ctx.token_seq, tables,
                                      cache.pools["latent"], cache.page_size, s.window, s.scale, chunk=s.chunk,
                                      partial=partial, nsplit=nsplit, tokens_per_group=group)
        else:
            ops.latent_attention(folded, mixed, H, key_dim, s.kv_rank, ctx.positions, ctx.token_seq, tables,
                                 cache.pools["latent"], cache.page_size, s.window, s.scale, chunk=s.chunk)
        heads_out = ctx.buffer("latent_heads", (n, H * s.value_dim), ctx.dtype)
        ops.gemm_batched(mixed, self.w_uv, heads_out, H, s.kv_rank, s.value_dim)
        if self.w_gate is not None:
            # the heads side by side times sigmoid(W_g x), x the mixer's own input
            gate = ctx.buffer("latent_gate", (n, H * s.value_dim), ctx.dtype)
            self.linear(x, self.w_gate, gate)
            ops.gate_mul(heads_out, gate, heads_out)
        return self.linear_deferred(ctx, "attn_proj", heads_out, self.w_o)


register_mixer("latent_attention", LatentAttention)
