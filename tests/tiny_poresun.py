"""Tiny Poresun configurations for tests.  They differ from each other in every size and
option: the three mixers in several orders and more than once; grouped, ungrouped and single
key/value heads; values smaller than, equal to and larger than keys; head sizes that are and
are not multiples of 32; windows of 1, 5, 16, 37 and 1,000 positions (smaller than a page,
exactly a page, across page edges, larger than any test sequence); bias tables of 2 to 40 rows
(odd counts too) that reach 3 to 500 positions, shorter and longer than the windows; caps from
2 to 50; query temperatures that step every position to every 300; layers that read the keys
and values of an earlier layer, of a windowed one too and more than one reader of one cache;
latent attention rotated whole, partly and not at all, with latents wider and narrower than
the heads; dense feed-forwards with limits of 0.5 to 7; 2 to 9 experts of which 1 to all are
chosen, with and without a shared expert, shared experts wider and narrower than the routed
ones; layers without a feed-forward; stream factors and embedding scales on either side of 1;
widths that are multiples of nothing."""

from __future__ import annotations

import tempfile
from pathlib import Path


def _attn(kind, heads, kv_heads, dim, vdim, rows, reach, scale=None, size=None, cap=None, temp=None, kv_from=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim**-0.5 if scale is None else scale,
           "bias_max": reach, "bias_rows": rows}
    if size is not None:
        out["mask"] = {"size": size}
    if cap is not None:
        out["softcap"] = cap
    if temp is not None:
        out["q_temp"] = {"coef": temp[0], "every": temp[1]}
    if kv_from is not None:
        out["kv_from"] = kv_from
    return {"type": kind, "mixer": out}


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, dims=None, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": (dim + rot_dim) ** -0.5 if scale is None else scale,
                      "rot": {"base": base, "dims": rot_dim if dims is None else dims}}}


def _dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def _with(layer, mlp):
    return {**layer, "mlp": mlp}


POR_A = {
    "architecture": "Poresun", "vocab": 211, "width": 70, "norm": {"eps": 1e-6}, "postln_alpha": 1.2,
    "embedding": {"scale": 3.0},
    "layers": [
        _with(_attn("attention_2", 4, 2, 32, 16, 12, 40, temp=(0.4, 7)), _moe(5, 2, 24, shared=40)),
        _with(_attn("attention", 4, 4, 16, 48, 7, 30, size=5, cap=8.0), _dense(80, 2.0)),
        _with(_attn("attention_2", 6, 2, 32, 16, 20, 100, temp=(0.9, 1), kv_from=0), None),
        _with(_latent(3, 24, 8, 20, 40, 32, base=500.0), _moe(9, 1, 20, shared=8)),
        _with(_attn("attention_2", 2, 2, 32, 16, 2, 3, kv_from=0), _moe(3, 3, 16)),
    ],
}

POR_B = {
    "architecture": "Poresun", "vocab": 97, "width": 100, "norm": {"eps": 1e-4}, "postln_alpha": 0.8,
    "embedding": {"scale": 0.5},
    "layers": [
        _with(_latent(5, 12, 6, 30, 20, 50, base=90.0, dims=2), _dense(40, 0.5)),
        _with(_attn("attention", 6, 1, 8, 5, 9, 25, size=1, cap=2.0), _moe(6, 4, 12, shared=25)),
        _with(_attn("attention", 3, 3, 40, 40, 40, 500, size=37, cap=50.0), None),
        # a causal layer that reads a windowed layer's keys and values: that cache keeps everything
        _with(_attn("attention_2", 3, 3, 40, 40, 16, 60, temp=(0.2, 300), kv_from=2), _moe(2, 2, 44)),
        _with(_latent(1, 40, 4, 12, 8, 16, dims=0), _moe(4, 1, 30, shared=30)),
    ],
}

POR_C = {
    "architecture": "Poresun", "vocab": 300, "width": 128, "norm": {"eps": 2e-5}, "postln_alpha": 1.6,
    "embedding": {"scale": 4.0},
    "layers": [
        _with(_attn("attention", 8, 2, 64, 64, 32, 200, size=1000, cap=30.0, scale=0.2), _moe(8, 2, 48, shared=80)),
        _with(_attn("attention_2", 8, 1, 32, 32, 18, 64, temp=(0.3, 64)), _dense(256, 7.0)),
        _with(_latent(4, 32, 32, 64, 64, 96, base=1.0e5), _moe(8, 8, 32, shared=32)),
        _with(_attn("attention", 4, 4, 32, 32, 8, 20, size=16, cap=15.0), _moe(4, 1, 128)),
    ],
}

CONFIGS = {"A": POR_A, "B": POR_B, "C": POR_C}
SEEDS = {"A": 7, "B": 17, "C": 31}
PAGE_SIZES = {"A": 16, "B": 4, "C": 32}


def make_model_dir(name: str, root=None, dtype: str = "float32", mode: str = "unit") -> Path:
    """Writes the tiny model `name` with seeded random weights (stored in `dtype`) into
    `root` (or a fresh temporary folder) and returns the folder."""
    from shrike_amd.weights import write_model_folder

    if root is None:
        root = tempfile.mkdtemp(prefix="shrike_tiny_")
    path = Path(root) / f"poresun_{name}_{dtype}_{mode}"
    if not (path / "model.safetensors").is_file():
        write_model_folder(dict(CONFIGS[name]), path, seed=SEEDS[name], dtype=dtype, mode=mode)
    return path
