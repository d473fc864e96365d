"""Tiny Ligipel configurations for tests.  They differ from each other in every size and
option: the two mixers in several orders and more than once, grouped, ungrouped and single
key/value heads, values smaller than, equal to and larger than keys, head sizes that are and
are not multiples of 32, windows of 1, 7, 40 and 1,000 positions (smaller than a page, across
page edges, larger than any test sequence) and none, scans with 1 to 5 taps and 3 to 70
states a channel, retention whole, partly and not rotated with head sizes on either side of a
lane's 16 rows, 3 to 9 experts of which 1 to all are chosen, with and without a shared expert,
layers without a feed-forward, logits with and without scale and cap, widths that are
multiples of nothing."""

from __future__ import annotations

import tempfile
from pathlib import Path


def _attn(heads, kv_heads, dim, vdim, size, scale=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim**-0.5 if scale is None else scale}
    if size is not None:
        out["mask"] = {"size": size}
    return out


def _scan(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def _parallel(left, right):
    return {"type": "parallel", "mixer": {"left": left, "right": right}}


def _retention(heads, dim, vdim, decay, base=None, dims=None):
    out = {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}
    if dims:
        out["rot"] = {"base": base, "dims": dims}
    return {"type": "retention", "mixer": out}


def _moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def _with(layer, mlp):
    return {**layer, "mlp": mlp}


LIG_A = {
    "architecture": "Ligipel", "vocab": 211, "width": 64, "norm": {"eps": 1e-6}, "logit_scale": 0.7, "logit_softcap": 12.0,
    "layers": [
        _with(_parallel(_attn(4, 2, 32, 16, 7), _scan(96, 12, 5, 4)), _moe(5, 2, 24, shared=40)),
        _with(_retention(2, 16, 20, [0.9, 0.97], base=500.0, dims=16), _moe(3, 3, 16)),
        _with(_parallel(_attn(2, 2, 16, 48, 40), _scan(40, 3, 2, 2)), None),
        _with(_parallel(_attn(3, 1, 24, 24, 1000), _scan(72, 33, 9, 3)), _moe(9, 1, 20, shared=8)),
    ],
}

LIG_B = {
    "architecture": "Ligipel", "vocab": 97, "width": 100, "norm": {"eps": 1e-4},
    "layers": [
        _with(_retention(3, 40, 16, [0.5, 0.99, 1.0], base=90.0, dims=6), _moe(4, 2, 30)),
        _with(_parallel(_attn(6, 1, 8, 5, 1), _scan(50, 70, 7, 1)), _moe(6, 4, 12, shared=25)),
        _with(_retention(1, 12, 50, [0.8]), None),
        _with(_parallel(_attn(1, 1, 40, 40, None), _scan(30, 16, 30, 5)), _moe(3, 2, 44)),
    ],
}

LIG_C = {
    "architecture": "Ligipel", "vocab": 300, "width": 128, "norm": {"eps": 2e-5}, "logit_scale": 1.5,
    "layers": [
        _with(_parallel(_attn(4, 4, 64, 128, 300, scale=0.2), _scan(256, 16, 8, 4)), _moe(8, 2, 48, shared=80)),
        _with(_parallel(_attn(8, 2, 32, 32, 33), _scan(128, 8, 4, 3)), _moe(4, 1, 128)),
        _with(_retention(2, 64, 64, [0.98, 0.999], base=1.0e5, dims=32), _moe(8, 8, 32, shared=32)),
    ],
}

# retention only: a model without any paged cache
LIG_D = {
    "architecture": "Ligipel", "vocab": 120, "width": 48, "norm": {"eps": 1e-5}, "logit_softcap": 20.0,
    "layers": [
        _with(_retention(4, 8, 8, [0.75, 0.9, 0.96, 0.995], base=300.0, dims=8), _moe(4, 2, 16, shared=24)),
        _with(_retention(2, 24, 12, [0.99, 0.6], base=7.0, dims=2), None),
    ],
}

# side-by-side mixers only; as many key/value heads as heads; a window of exactly a page
LIG_E = {
    "architecture": "Ligipel", "vocab": 160, "width": 72, "norm": {"eps": 1e-5}, "logit_scale": 2.0,
    "layers": [
        _with(_parallel(_attn(3, 3, 40, 24, 16), _scan(64, 4, 3, 2)), _moe(3, 3, 24)),
        _with(_parallel(_attn(5, 5, 8, 16, 17), _scan(80, 20, 6, 4)), _moe(7, 2, 8, shared=16)),
    ],
}

CONFIGS = {"A": LIG_A, "B": LIG_B, "C": LIG_C, "D": LIG_D, "E": LIG_E}
SEEDS = {"A": 5, "B": 13, "C": 29, "D": 41, "E": 53}
PAGE_SIZES = {"A": 16, "B": 4, "C": 32, "D": 16, "E": 16}


def make_model_dir(name: str, root=None, dtype: str = "float32", mode: str = "unit") -> Path:
    """Writes the tiny model `name` with seeded random weights (stored in `dtype`) into
    `root` (or a fresh temporary folder) and returns the folder."""
    from shrike_amd.weights import write_model_folder

    if root is None:
        root = tempfile.mkdtemp(prefix="shrike_tiny_")
    path = Path(root) / f"ligipel_{name}_{dtype}_{mode}"
    if not (path / "model.safetensors").is_file():
        write_model_folder(dict(CONFIGS[name]), path, seed=SEEDS[name], dtype=dtype, mode=mode)
    return path
