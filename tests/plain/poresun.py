"""A plain, slow form of the Poresun decoder, one function per mechanism, written
from the design's equations with torch on the CPU.  It shares nothing with the
package: it takes the raw config dictionary and a dictionary of tensors by their
names in the weight file, runs one whole sequence at a time, keeps no cache, and
returns logits for every position (in the precision of the tensors it is given).

Notation: W[.] are matrices stored [out, in]; x is the stream [tokens, width];
positions count from 0; i is a query's position, j a key's.
"""

from __future__ import annotations

import math

import torch

QUICK_GELU_SLOPE = 1.702  # the dense feed-forward's gate is g * sigmoid(1.702 g)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps), the eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def visible(n: int, window: int | None = None) -> torch.Tensor:
    """vis[i, j]: j <= i, and with a window also i - j < window."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    vis = j <= i
    if window is not None:
        vis = vis & (i - j < window)
    return vis


def distance_bucket(distance: int, rows: int, reach: int) -> int:
    """Row of the bias table for a distance i - j >= 0: the first half of the rows one
    distance each, the other half spread evenly over the logarithm of the distance up to
    `reach`, the last row for everything beyond."""
    half = rows // 2
    if distance < half:
        return distance
    steps = math.floor(math.log(distance / half) / math.log(reach / half) * (rows - half))
    return min(rows - 1, half + steps)


def distance_bias(n: int, table: torch.Tensor, reach: int) -> torch.Tensor:
    """bias[h, i, j] = table[bucket(i - j), h] for j <= i (0 elsewhere)."""
    rows, heads = table.shape
    by_distance = torch.stack([table[distance_bucket(d, rows, reach)] for d in range(n)])  # [n, heads]
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    d = (i - j).clamp(min=0)
    return by_distance[d].permute(2, 0, 1)


def query_temperature(positions: torch.Tensor, coef: float, every: int, dtype) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1) per position."""
    steps = torch.div(positions + 1, every, rounding_mode="floor")
    return (1.0 + coef * torch.log(steps.to(torch.float64) + 1.0)).to(dtype)


def softmax_rows(scores: torch.Tensor, vis: torch.Tensor) -> torch.Tensor:
    return torch.softmax(scores.masked_fill(~vis, float("-inf")), dim=-1)


def grouped_keys_values(h, w, prefix: str, m: dict, eps: float, weighted: bool):
    """Keys [n, G, D] as the layer's cache holds them (after their norm) and values [n, G, V]."""
    n = h.shape[0]
    G, D, V = m["kv_heads"], m["dim"], m["vdim"]
    k = unit_rms((h @ w[prefix + ".k"].T).view(n, G, D), eps)
    if weighted:
        k = k * w[prefix + ".k.norm"]
    v = (h @ w[prefix + ".v"].T).view(n, G, V)
    return k, v


def biased_attention(h, positions, w, prefix: str, m: dict, eps: float, weighted: bool, keys_values=None):
    """Grouped-query attention without rotation.  Queries and keys are brought to unit root
    mean square per head (`weighted`: then times a weight of the head's size that all heads
    share); queries may be scaled by a slowly growing function of the position; the scaled
    score may be capped; a learned bias by distance is added after that; causal, with or
    without a window.  `keys_values`: another layer's (keys, values) to read instead of
    projecting one's own.  Returns (output, (keys, values))."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ w[prefix + ".q"].T).view(n, H, D), eps)
    if weighted:
        q = q * w[prefix + ".q.norm"]
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(positions, float(qt["coef"]), int(qt["every"]), q.dtype)[:, None, None]
    if keys_values is None:
        keys_values = grouped_keys_values(h, w, prefix, m, eps, weighted)
    k, v = keys_values
    cap = m.get("softcap")
    mask = m.get("mask")
    vis = visible(n, int(mask["size"]) if mask else None)
    bias = distance_bias(n, w[prefix + ".rel"].to(h.dtype), int(m["bias_max"]))
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        if cap:
            s = float(cap) * torch.tanh(s / float(cap))
        s = s + bias[head]
        out[:, head] = softmax_rows(s, vis) @ v[:, g]
    return out.reshape(n, H * V) @ w[prefix + ".o"].T, keys_values


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """Turns the pairs (2i, 2i + 1), i < dims / 2, of the last axis by position *
    base^(-2i / dims); what lies beyond `dims` passes unchanged.  x is [tokens, ..., size]."""
    rates = base ** (-torch.arange(0, dims, 2, dtype=torch.float64) / dims)
    angle = positions.to(torch.float64)[:, None] * rates  # [tokens, dims / 2]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (dims // 2,)
    cos, sin = torch.cos(angle).to(x.dtype).view(shape), torch.sin(angle).to(x.dtype).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_attention(h, positions, w, prefix: str, m: dict, eps: float):
    """Queries through a normed latent; keys and values through another, of which one normed
    part is every head's source of keys and values and a second, unnormed part is a rotated
    key that all heads share; causal; the heads' outputs are gated by sigmoid(W_g h)."""
    n = h.shape[0]
    H, D, R, V, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    c_q = unit_rms(h @ w[prefix + ".dq"].T, eps) * w[prefix + ".dq.norm"]
    q = (c_q @ w[prefix + ".uq"].T).view(n, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:], positions, float(rot["base"]), int(rot["dims"]))
    down = h @ w[prefix + ".dkv"].T
    c = unit_rms(down[:, :rank], eps) * w[prefix + ".dkv.norm"]
    k_rot = rotate_pairs(down[:, rank:], positions, float(rot["base"]), int(rot["dims"]))  # [n, R]
    k_plain = (c @ w[prefix + ".uk"].T).view(n, H, D)
    v = (c @ w[prefix + ".uv"].T).view(n, H, V)
    vis = visible(n)
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * float(m["scale"])
        out[:, head] = softmax_rows(s, vis) @ v[:, head]
    gate = torch.sigmoid(h @ w[prefix + ".g"].T)
    return (out.reshape(n, H * V) * gate) @ w[prefix + ".o"].T


def dense_ff(h, w, prefix: str, m: dict):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    limit = float(m["limit"])
    g = (h @ w[prefix + ".gate"].T).clamp(max=limit)
    u = (h @ w[prefix + ".up"].T).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(QUICK_GELU_SLOPE * g) * (u + 1.0)) @ w[prefix + ".down"].T


def squared_relu_expert(h, w, prefix: str):
    return torch.relu(h @ w[prefix + ".up"].T) ** 2 @ w[prefix + ".down"].T


def route(h, w, prefix: str, top: int):
    """(chosen [n, top], weights [n, top]): the experts with the largest logits W_router h + b,
    and the softmax over those logits alone."""
    logits = h.to(torch.float32) @ w[prefix + ".router"].to(torch.float32).T + w[prefix + ".router.b"].to(torch.float32)
    best, chosen = torch.topk(logits, top, dim=-1)
    return chosen, torch.softmax(best, dim=-1)


def mixture_ff(h, w, prefix: str, m: dict):
    """Every token's weighted sum of its chosen experts, plus the shared expert times
    sigmoid(W_sg h) (one number per token)."""
    experts, top = int(m["router"]["experts"]), int(m["router"]["top"])
    chosen, weights = route(h, w, prefix, top)
    out = torch.zeros_like(h)
    for e in range(experts):
        for slot in range(top):
            rows = (chosen[:, slot] == e).nonzero().flatten()
            if rows.numel():
                out[rows] += weights[rows, slot, None].to(h.dtype) * squared_relu_expert(h[rows], w, f"{prefix}.e{e}")
    if m.get("shared"):
        gate = torch.sigmoid(h @ w[prefix + ".shared.sg"].T)  # [n, 1]
        out = out + gate * squared_relu_expert(h, w, prefix + ".shared")
    return out


def feed_forward(h, w, prefix: str, m: dict):
    if m["kind"] == "dense":
        return dense_ff(h, w, prefix, m)
    if m["kind"] == "moe":
        return mixture_ff(h, w, prefix, m)
    raise ValueError(f"unknown feed-forward kind {m['kind']!r}")


def normed_sum(x, y, scale_vector, alpha: float, weight, eps: float):
    """norm(alpha x + scale_vector * y): the norm stands after the sum."""
    return unit_rms(alpha * x + scale_vector * y, eps) * weight


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [tokens, vocab] of one sequence; with return_layers also the stream after every layer."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    n = tokens.shape[0]
    positions = torch.arange(n)
    eps, alpha = float(cfg["norm"]["eps"]), float(cfg["postln_alpha"])
    x = w["embed"][tokens] * float(cfg["embedding"]["scale"])
    kept = {}  # keys and values by layer, for layers that read another's
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        if layer["type"] == "latent_attention":
            y = latent_attention(x, positions, w, p + ".mix", m, eps)
        elif layer["type"] in ("attention", "attention_2"):
            source = m.get("kv_from")
            y, kept[i] = biased_attention(x, positions, w, p + ".mix", m, eps, weighted=layer["type"] == "attention_2",
                                          keys_values=None if source is None else kept[int(source)])
        else:
            raise ValueError(f"unknown mixer type {layer['type']!r}")
        x = normed_sum(x, y, w[p + ".ls1"], alpha, w[p + ".norm1"], eps)
        if layer.get("mlp"):
            x = normed_sum(x, feed_forward(x, w, p + ".mlp", layer["mlp"]), w[p + ".ls2"], alpha, w[p + ".norm2"], eps)
        elif p + ".norm2" in w:  # a file that holds a second norm for a layer without a feed-forward
            x = normed_sum(x, torch.zeros_like(x), 1.0, alpha, w[p + ".norm2"], eps)
        streams.append(x)
    logits = (unit_rms(x, eps) * w["final.norm"]) @ w["embed"].T
    return (logits, torch.stack(streams)) if return_layers else logits


class PlainPoresun:
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
        return forward(self.cfg, self.weights, list(token_ids), return_layers=True)[1]

    def greedy(self, prompt, max_new_tokens: int) -> list[int]:
        seq, out = list(prompt), []
        for _ in range(max_new_tokens):
            tok = int(torch.argmax(self.logits(seq)[-1]))
            out.append(tok)
            seq.append(tok)
        return out
