"""A plain, slow form of the Ligipel decoder, one function per mechanism, written from
the design's equations with torch on the CPU.  It shares nothing with the package: it
takes the raw config dictionary and a dictionary of tensors by their names in the weight
file, runs one whole sequence at a time, keeps no cache, and returns logits for every
position (in the precision of the tensors it is given).

Notation: W[.] are matrices stored [out, in]; x is the residual stream [tokens, width];
positions count from 0; i is a query's position and j a key's.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(var + eps) * w + b, var the mean squared deviation."""
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(dim=-1, keepdim=True)
    return d / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps), the eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def silu(z):
    return z * torch.sigmoid(z)


def window_mask(n: int, size: int) -> torch.Tensor:
    """visible[i, j]: 0 <= i - j < size."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i - j < size)


def distance_bias(n: int, r1: torch.Tensor, r2: torch.Tensor) -> torch.Tensor:
    """[heads, n, n]: r1_h ln(1 + r2_h (i - j)) where j <= i, 0 elsewhere."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    dist = (i - j).clamp(min=0).to(r1.dtype)
    return r1[:, None, None] * torch.log1p(r2[:, None, None] * dist[None])


def sink_softmax(s: torch.Tensor, visible: torch.Tensor) -> torch.Tensor:
    """p_j = exp(s_j) / (1 + sum_j exp(s_j)) over the visible j of every row: a softmax
    with one more term whose score is 0."""
    s = s.masked_fill(~visible, float("-inf"))
    m = s.max(dim=-1, keepdim=True).values.clamp(min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(dim=-1, keepdim=True))


def mixed_head_attention(q, k, v, scale: float, window, r1, r2, talk, sink: bool = True):
    """q [n, H, D], k [n, G, D], v [n, G, V] -> [n, H, V]: scores less the distance bias, a
    sliding window (None: all earlier keys), the softmax with a sink of score 0, the weights
    mixed across heads by talk [H, H], each head on the values of its own key/value head."""
    n, H, _ = q.shape
    G, V = k.shape[1], v.shape[2]
    visible = window_mask(n, window if window is not None else n + 1)
    bias = distance_bias(n, r1, r2) if r1 is not None else torch.zeros(H, n, n, dtype=q.dtype)
    p = torch.zeros(H, n, n, dtype=q.dtype)
    for head in range(H):
        s = (q[:, head] @ k[:, head // (H // G)].T) * scale - bias[head]
        if sink:
            p[head] = sink_softmax(s, visible)
        else:
            p[head] = torch.softmax(s.masked_fill(~visible, float("-inf")), dim=-1)
    mixed = torch.einsum("hg,gij->hij", talk, p) if talk is not None else p
    out = torch.zeros(n, H, V, dtype=q.dtype)
    for head in range(H):
        out[:, head] = mixed[head] @ v[:, head // (H // G)]
    return out


def talking_attention(h, w, prefix: str, m: dict):
    """Grouped-query attention without rotation: a logarithmic distance bias, a sliding
    window, a sink of score 0, and weights mixed across heads after the softmax."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + ".q"].T).view(n, H, D)
    k = (h @ w[prefix + ".k"].T).view(n, G, D)
    v = (h @ w[prefix + ".v"].T).view(n, G, V)
    window = int(m["mask"]["size"]) if m.get("mask") else None
    out = mixed_head_attention(q, k, v, float(m["scale"]), window, w[prefix + ".r1"].to(h.dtype),
                               w[prefix + ".r2"].to(h.dtype), w[prefix + ".talk"].to(h.dtype))
    return out.reshape(n, H * V) @ w[prefix + ".o"].T


def causal_conv(x, taps, bias):
    """y[t, c] = bias[c] + sum_k taps[c, K-1-k] x[t-k, c]: the last column of `taps`
    meets the current token, zeros stand before the start."""
    n, c = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, c, dtype=x.dtype), x], dim=0)
    y = bias[None, :].expand(n, c).clone()
    for k in range(K):
        y = y + padded[k : k + n] * taps[:, k][None, :]
    return y


def scan(x, dt, A, B, C, D, S=None):
    """x, dt [n, inner]; A [inner, N]; B, C [n, N]; D [inner] -> (y [n, inner], final S):
    S <- exp(dt A) S + dt x B^T per token; y = S C + D x."""
    n, inner = x.shape
    S = torch.zeros(inner, A.shape[1], dtype=x.dtype) if S is None else S.clone()
    y = torch.zeros(n, inner, dtype=x.dtype)
    for t in range(n):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y, S


def selective_scan(h, w, prefix: str, m: dict):
    """Mamba: a per-channel linear recurrence whose step size and input/output maps
    depend on the token."""
    inner, R, N = m["inner"], m["dt_rank"], m["state"]
    xz = h @ w[prefix + ".in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, w[prefix + ".conv"].to(h.dtype), w[prefix + ".conv.b"].to(h.dtype)))
    dbc = x @ w[prefix + ".x"].T
    dt, B, C = dbc[:, :R], dbc[:, R : R + N], dbc[:, R + N :]
    dt = F.softplus(dt @ w[prefix + ".dt"].T + w[prefix + ".dt.b"].to(h.dtype))  # [n, inner]
    A = -torch.exp(w[prefix + ".A_log"].to(h.dtype))  # [inner, N]
    y, _ = scan(x, dt, A, B, C, w[prefix + ".D"].to(h.dtype))
    return (y * silu(z)) @ w[prefix + ".o"].T


def parallel_mixer(h, w, prefix: str, m: dict, eps: float):
    left = talking_attention(h, w, prefix + ".left", m["left"])
    right = selective_scan(h, w, prefix + ".right", m["right"])
    return 0.5 * (unit_rms(left, eps) * w[prefix + ".left.out"].to(h.dtype)
                  + unit_rms(right, eps) * w[prefix + ".right.out"].to(h.dtype))


def rotate_half(x, positions, dims: int, base: float):
    """Element i < dims/2 of every head pairs with element i + dims/2; the pair turns
    by position * base^(-2i/dims).  Elements from `dims` on pass unchanged."""
    if dims == 0:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def retention(q, k, v, decay, S=None):
    """q, k [n, H, D], v [n, H, V] -> (o [n, H, V], final S [H, D, V]):
    S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    n, H, D = q.shape
    V = v.shape[2]
    S = torch.zeros(H, D, V, dtype=q.dtype) if S is None else S.clone()
    o = torch.zeros(n, H, V, dtype=q.dtype)
    for t in range(n):
        for head in range(H):
            S[head] = float(decay[head]) * S[head] + k[t, head][:, None] * v[t, head][None, :]
            o[t, head] = S[head].T @ q[t, head]
    return o, S


def retention_mixer(h, positions, w, prefix: str, m: dict, eps: float):
    """Linear attention with a fixed decay per head, no softmax, no denominator; the
    readout normed per head, gated and projected."""
    n = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    dims, base = int(rot.get("dims", 0)), float(rot.get("base", 1.0))
    q = rotate_half((h @ w[prefix + ".q"].T).view(n, H, D), positions, dims, base)
    k = rotate_half((h @ w[prefix + ".k"].T).view(n, H, D), positions, dims, base) * D**-0.5
    v = (h @ w[prefix + ".v"].T).view(n, H, V)
    o, _ = retention(q, k, v, m["decay"])
    o = unit_rms(o, eps).reshape(n, H * V)
    return (o * silu(h @ w[prefix + ".g"].T)) @ w[prefix + ".o"].T


def gated_expert(h, w, prefix: str):
    return (silu(h @ w[prefix + ".gate"].T) * (h @ w[prefix + ".up"].T)) @ w[prefix + ".down"].T


def route(h, w, prefix: str, experts: int, top: int):
    """(chosen [n, top], weights [n, top]): softmax scores; the choice adds the
    correction, the weights do not; weights sum to one."""
    s = torch.softmax(h.to(torch.float32) @ w[prefix + ".router"].to(torch.float32).T, dim=-1)
    chosen = torch.topk(s + w[prefix + ".correction"].to(torch.float32), top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)


def mixture(h, w, prefix: str, mlp: dict):
    r = mlp["router"]
    chosen, weights = route(h, w, prefix, int(r["experts"]), int(r["top"]))
    out = torch.zeros_like(h)
    for e in range(int(r["experts"])):
        share = (weights * (chosen == e)).sum(dim=-1).to(h.dtype)  # 0 where e was not chosen
        rows = share.nonzero().flatten()
        if rows.numel():
            out[rows] += share[rows, None] * gated_expert(h[rows], w, f"{prefix}.e{e}")
    if mlp.get("shared"):
        out = out + gated_expert(h, w, prefix + ".shared")
    return out


def layer(x, positions, w, i: int, entry: dict, eps: float):
    p = f"l{i}"
    ln = lambda y, name: layer_norm(y, w[f"{p}.{name}"].to(y.dtype), w[f"{p}.{name}.b"].to(y.dtype), eps)  # noqa: E731
    h = ln(x, "norm1")
    if entry["type"] == "parallel":
        mixed = parallel_mixer(h, w, p + ".mix", entry["mixer"], eps)
    elif entry["type"] == "retention":
        mixed = retention_mixer(h, positions, w, p + ".mix", entry["mixer"], eps)
    else:
        raise ValueError(entry["type"])
    x = x + ln(mixed, "norm1b")
    if entry.get("mlp") is not None:
        x = x + ln(mixture(ln(x, "norm2"), w, p + ".mlp", entry["mlp"]), "norm2b")
    return x


def forward(cfg: dict, w: dict, tokens, keep_layers: bool = False):
    """Logits [tokens, vocab] of one sequence; with keep_layers also the stream that each
    layer hands on (after the depth average)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][tokens]
    x = layer_norm(x, w["embed.norm"].to(x.dtype), w["embed.norm.b"].to(x.dtype), eps)
    history, kept = [x], []
    for i, entry in enumerate(cfg["layers"]):
        history.append(layer(x, positions, w, i, entry, eps))
        coef = w[f"l{i}.dwa"].to(x.dtype)
        x = sum(coef[j] * history[j] for j in range(i + 2))
        kept.append(x)
    x = layer_norm(x, w["final.norm"].to(x.dtype), w["final.norm.b"].to(x.dtype), eps)
    logits = (x @ w["head"].T) * float(cfg.get("logit_scale", 1.0))
    if cfg.get("logit_softcap"):
        cap = float(cfg["logit_softcap"])
        logits = cap * torch.tanh(logits / cap)
    return (logits, torch.stack(kept)) if keep_layers else logits


class PlainLigipel:
    """A model folder read once; `logits(ids)`, the stream after every layer, and greedy
    generation over it, in float64 unless told otherwise."""

    def __init__(self, model_dir, dtype=torch.float64):
        import json
        from pathlib import Path

        from safetensors.torch import load_file

        self.cfg = json.loads((Path(model_dir) / "config.json").read_text())
        raw = load_file(str(Path(model_dir) / "model.safetensors"))
        self.weights = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in raw.items()}

    def logits(self, token_ids, rows=None) -> torch.Tensor:
        out = forward(self.cfg, self.weights, list(token_ids))
        return out if rows is None else out[torch.tensor(list(rows), dtype=torch.long)]

    def layers(self, token_ids) -> torch.Tensor:
        return forward(self.cfg, self.weights, list(token_ids), keep_layers=True)[1]

    def greedy(self, prompt, max_new_tokens: int) -> list[int]:
        seq, out = list(prompt), []
        for _ in range(max_new_tokens):
            tok = int(torch.argmax(self.logits(seq)[-1]))
            out.append(tok)
            seq.append(tok)
        return out
