"""What pins the plain form of Poresun (tests/plain/poresun.py) without any library's model
code, and the configuration reader: each mechanism against numbers worked out by hand or
against a second writing, the whole model's causality, the order of layers, the tensor names
and what the caches keep."""

import math

import pytest
import torch

from .plain import poresun as P
from .tiny_poresun import CONFIGS, POR_A, POR_B

torch.manual_seed(0)
F64 = torch.float64


def test_unit_rms_has_eps_inside_the_root():
    x = torch.tensor([[3.0, 4.0]], dtype=F64)
    assert torch.allclose(P.unit_rms(x, 0.5), x / math.sqrt(12.5 + 0.5))
    assert torch.allclose(P.unit_rms(torch.zeros(1, 4, dtype=F64), 1e-6), torch.zeros(1, 4, dtype=F64))


def test_buckets_by_hand():
    # 8 rows that reach 50 positions: distances 0..3 a row each, then rows 4..7 over ln(d / 4) / ln(12.5)
    got = [P.distance_bucket(d, 8, 50) for d in (0, 1, 3, 4, 7, 8, 15, 16, 31, 32, 49, 50, 51, 1000)]
    assert got == [0, 1, 3, 4, 4, 5, 6, 6, 7, 7, 7, 7, 7, 7]
    # an odd count: half is 3, four rows for the logarithm
    assert [P.distance_bucket(d, 7, 30) for d in (2, 3, 5, 6, 10, 11, 17, 29, 30)] == [2, 3, 3, 4, 5, 5, 6, 6, 6]
    # rows never fall as the distance grows, and the last one is reached at `reach` at the latest
    for rows, reach in ((2, 3), (16, 64), (24, 300), (40, 500), (9, 25)):
        seq = [P.distance_bucket(d, rows, reach) for d in range(reach + 5)]
        assert seq == sorted(seq) and seq[reach] == rows - 1 and seq[0] == 0


@pytest.mark.parametrize("rows, reach", [(2, 3), (7, 30), (12, 40), (14, 90), (24, 300), (40, 500), (9, 25)])
def test_the_engines_table_of_buckets_is_the_plain_one(rows, reach):
    from shrike_amd.parts.attention import distance_buckets

    assert distance_buckets(rows, reach) == [P.distance_bucket(d, rows, reach) for d in range(reach + 1)]


def test_windows_written_out():
    vis = P.visible(5, 2)
    assert vis.int().tolist() == [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [0, 1, 1, 0, 0], [0, 0, 1, 1, 0], [0, 0, 0, 1, 1]]
    assert P.visible(4).int().tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [1, 1, 1, 0], [1, 1, 1, 1]]
    assert P.visible(3, 1).int().tolist() == [[1, 0, 0], [0, 1, 0], [0, 0, 1]]


def test_query_temperature_steps():
    t = P.query_temperature(torch.arange(10), 0.5, 4, F64)
    want = [1.0] * 3 + [1 + 0.5 * math.log(2)] * 4 + [1 + 0.5 * math.log(3)] * 3
    assert torch.allclose(t, torch.tensor(want, dtype=F64))


def _attention_weights(m, rel, n=6, weighted=False, extra=None):
    width = 8
    w = {"p.q": torch.randn(m["heads"] * m["dim"], width, dtype=F64), "p.k": torch.randn(m["kv_heads"] * m["dim"], width, dtype=F64),
         "p.v": torch.randn(m["kv_heads"] * m["vdim"], width, dtype=F64),
         "p.o": torch.eye(m["heads"] * m["vdim"], dtype=F64), "p.rel": rel}
    if weighted:
        w["p.q.norm"], w["p.k.norm"] = torch.rand(m["dim"], dtype=F64) + 0.5, torch.rand(m["dim"], dtype=F64) + 0.5
    w.update(extra or {})
    return w, torch.randn(n, width, dtype=F64)


def test_attention_position_by_position():
    """One head: every score written out with the cap before the bias, the window and the softmax."""
    m = {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.7, "softcap": 1.5, "bias_max": 5, "mask": {"size": 3}}
    rel = torch.tensor([[0.3], [-1.0], [2.0], [0.5]], dtype=F64)  # rows for distances 0, 1, then 2, 3..
    w, h = _attention_weights(m, rel)
    out, _ = P.biased_attention(h, torch.arange(6), w, "p", m, 1e-5, weighted=False)
    q = h @ w["p.q"].T
    k = h @ w["p.k"].T
    v = h @ w["p.v"].T
    q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + 1e-5)
    k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + 1e-5)
    for i in range(6):
        scores, values = [], []
        for j in range(max(0, i - 2), i + 1):
            s = 1.5 * math.tanh(float(q[i] @ k[j]) * 0.7 / 1.5)
            d = i - j
            row = d if d < 2 else min(3, 2 + math.floor(math.log(d / 2) / math.log(5 / 2) * 2))
            scores.append(s + float(rel[row, 0]))
            values.append(v[j])
        p = torch.softmax(torch.tensor(scores, dtype=F64), 0)
        assert torch.allclose(out[i], sum(pj * vj for pj, vj in zip(p, values)), atol=1e-12)


def test_weighted_norms_temperature_and_groups():
    """attention_2's particulars: the norm's weight is shared by the heads, the temperature
    multiplies the normed queries, query head h reads key/value head h // (H / G)."""
    m = {"heads": 4, "kv_heads": 2, "dim": 4, "vdim": 2, "scale": 0.5, "bias_max": 6, "q_temp": {"coef": 0.8, "every": 2}}
    rel = torch.randn(4, 4, dtype=F64)
    w, h = _attention_weights(m, rel, weighted=True)
    out, (keys, values) = P.biased_attention(h, torch.arange(6), w, "p", m, 1e-6, weighted=True)
    q = (h @ w["p.q"].T).view(6, 4, 4)
    q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + 1e-6) * w["p.q.norm"]
    q = q * (1 + 0.8 * torch.log(torch.div(torch.arange(6) + 1, 2, rounding_mode="floor").to(F64) + 1))[:, None, None]
    i = 5
    for head in range(4):
        g = head // 2
        s = torch.stack([q[i, head] @ keys[j, g] * 0.5 + rel[P.distance_bucket(i - j, 4, 6), head] for j in range(6)])
        assert torch.allclose(out[i].view(4, 2)[head], torch.softmax(s, 0) @ values[:, g], atol=1e-12)
    # keys as the cache holds them: normed and weighted
    k = (h @ w["p.k"].T).view(6, 2, 4)
    assert torch.allclose(keys, k / torch.sqrt((k * k).mean(-1, keepdim=True) + 1e-6) * w["p.k.norm"])


def test_a_layer_that_reads_anothers_keys_and_values():
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.5, "bias_max": 6}
    w, h = _attention_weights(m, torch.randn(4, 2, dtype=F64), weighted=True)
    _, kept = P.biased_attention(h, torch.arange(6), w, "p", m, 1e-6, weighted=True)
    other = torch.randn(6, 8, dtype=F64)
    reader = {k: v for k, v in w.items() if k not in ("p.k", "p.v", "p.k.norm")}
    out, _ = P.biased_attention(other, torch.arange(6), reader, "p", m, 1e-6, weighted=True, keys_values=kept)
    own, _ = P.biased_attention(other, torch.arange(6), w, "p", m, 1e-6, weighted=True)
    assert not torch.allclose(out, own)
    # with the same input the two are one
    again, _ = P.biased_attention(h, torch.arange(6), reader, "p", m, 1e-6, weighted=True, keys_values=kept)
    assert torch.allclose(again, P.biased_attention(h, torch.arange(6), w, "p", m, 1e-6, weighted=True)[0])


def test_rotation_is_a_complex_turn_of_neighbours():
    x = torch.randn(5, 3, 8, dtype=F64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    out = P.rotate_pairs(x, pos, 50.0, 6)
    z = torch.view_as_complex(x[..., :6].reshape(5, 3, 3, 2).contiguous())
    rates = torch.tensor([50.0 ** (-2 * i / 6) for i in range(3)], dtype=F64)
    turned = z * torch.polar(torch.ones(5, 3, dtype=F64), pos.to(F64)[:, None] * rates)[:, None, :]
    assert torch.allclose(torch.view_as_real(turned).reshape(5, 3, 6), out[..., :6], atol=1e-12)
    assert torch.equal(out[..., 6:], x[..., 6:]) and torch.equal(out[0], x[0])
    assert torch.equal(P.rotate_pairs(x, pos, 50.0, 0), x)


def test_latent_attention_folded_the_other_way():
    """The same mixer with the heads' key matrices applied to the queries instead of the latent,
    and the value matrices after the weighted sum of latents."""
    m = {"heads": 2, "dim": 4, "rot_dim": 4, "vdim": 3, "q_rank": 5, "kv_rank": 6, "scale": 0.3, "rot": {"base": 100.0, "dims": 2}}
    width, n = 8, 7
    w = {"p.dq": torch.randn(5, width, dtype=F64), "p.dq.norm": torch.rand(5, dtype=F64) + 0.5,
         "p.uq": torch.randn(16, 5, dtype=F64), "p.dkv": torch.randn(10, width, dtype=F64),
         "p.dkv.norm": torch.rand(6, dtype=F64) + 0.5, "p.uk": torch.randn(8, 6, dtype=F64),
         "p.uv": torch.randn(6, 6, dtype=F64), "p.g": torch.randn(6, width, dtype=F64), "p.o": torch.eye(6, dtype=F64)}
    h = torch.randn(n, width, dtype=F64)
    pos = torch.arange(n)
    out = P.latent_attention(h, pos, w, "p", m, 1e-6)
    c_q = P.unit_rms(h @ w["p.dq"].T, 1e-6) * w["p.dq.norm"]
    q = (c_q @ w["p.uq"].T).view(n, 2, 8)
    down = h @ w["p.dkv"].T
    c = P.unit_rms(down[:, :6], 1e-6) * w["p.dkv.norm"]
    k_rot = P.rotate_pairs(down[:, 6:], pos, 100.0, 2)
    gate = torch.sigmoid(h @ w["p.g"].T).view(n, 2, 3)
    for head in range(2):
        folded = q[:, head, :4] @ w["p.uk"].view(2, 4, 6)[head]  # [n, kv_rank]
        s = (folded @ c.T + P.rotate_pairs(q[:, head, 4:], pos, 100.0, 2) @ k_rot.T) * 0.3
        p = torch.softmax(s.masked_fill(~P.visible(n), float("-inf")), -1)
        o = (p @ c) @ w["p.uv"].view(2, 3, 6)[head].T
        assert torch.allclose(out.view(n, 2, 3)[:, head], o * gate[:, head], atol=1e-10)


def test_dense_feed_forward_by_hand():
    w = {"p.gate": torch.tensor([[1.0], [1.0], [1.0]], dtype=F64), "p.up": torch.tensor([[1.0], [-1.0], [0.1]], dtype=F64),
         "p.down": torch.eye(3, dtype=F64)}
    y = P.dense_ff(torch.tensor([[5.0]], dtype=F64), w, "p", {"limit": 2.0})[0]
    g = 2.0 * (1 / (1 + math.exp(-1.702 * 2.0)))  # the gate is bounded from above before its activation
    assert torch.allclose(y, torch.tensor([g * 3.0, g * -1.0, g * 1.5], dtype=F64))
    y = P.dense_ff(torch.tensor([[-5.0]], dtype=F64), w, "p", {"limit": 2.0})[0]
    g = -5.0 * (1 / (1 + math.exp(1.702 * 5.0)))  # and not from below
    assert torch.allclose(y, torch.tensor([g * -1.0, g * 3.0, g * 0.5], dtype=F64))


def test_router_and_mixture_by_hand():
    width = 4
    w = {"p.router": torch.eye(4, dtype=F64)[:3], "p.router.b": torch.tensor([0.0, 0.0, 2.5], dtype=F64),
         "p.shared.sg": torch.tensor([[0.0, 0.0, 0.0, 1.0]], dtype=F64),
         "p.shared.up": torch.randn(5, width, dtype=F64), "p.shared.down": torch.randn(width, 5, dtype=F64)}
    for e in range(3):
        w[f"p.e{e}.up"], w[f"p.e{e}.down"] = torch.randn(6, width, dtype=F64), torch.randn(width, 6, dtype=F64)
    h = torch.tensor([[3.0, 1.0, 0.0, 0.7], [0.0, 1.0, -2.0, -0.3]], dtype=F64)
    chosen, weights = P.route(h, w, "p", 2)
    assert chosen.tolist() == [[0, 2], [1, 2]]  # logits (3, 1, 2.5) and (0, 1, 0.5): the bias moves the choice
    assert torch.allclose(weights[0].double(), torch.softmax(torch.tensor([3.0, 2.5], dtype=F64), 0), atol=1e-6)
    m = {"kind": "moe", "router": {"experts": 3, "top": 2}, "expert": {"ff": 6}, "shared": {"ff": 5}}
    out = P.mixture_ff(h, w, "p", m)
    for t in range(2):
        want = sum(weights[t, s].double() * (torch.relu(w[f"p.e{int(chosen[t, s])}.up"] @ h[t]) ** 2) @ w[f"p.e{int(chosen[t, s])}.down"].T
                   for s in range(2))
        want = want + torch.sigmoid(h[t, 3]) * ((torch.relu(w["p.shared.up"] @ h[t]) ** 2) @ w["p.shared.down"].T)
        assert torch.allclose(out[t], want, atol=1e-6)


def _weights_for(cfg, seed=0):
    from shrike_amd.config.registry import get_architecture
    from shrike_amd.models import DecoderModel
    from shrike_amd.weights.random_init import random_tensor

    arch = get_architecture("Poresun")
    model = DecoderModel(arch.build_spec(arch.config_cls.from_dict(cfg)))
    return {p.name: random_tensor(p, seed, F64, mode="unit") for p in model.params() if not p.optional}, model


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_whole_model_is_causal_and_the_norm_stands_last(name):
    cfg = CONFIGS[name]
    w, _ = _weights_for(cfg)
    ids = [int(t) for t in torch.randint(0, cfg["vocab"], (40,))]
    logits, layers = P.forward(cfg, w, ids, return_layers=True)
    shorter = P.forward(cfg, w, ids[:23])
    assert torch.allclose(logits[:23], shorter, atol=1e-9)
    changed = P.forward(cfg, w, ids[:30] + [(ids[30] + 1) % cfg["vocab"]] + ids[31:])
    assert torch.allclose(changed[:30], logits[:30], atol=1e-9) and not torch.allclose(changed[30:], logits[30:])
    # what a layer leaves is a normed row: its root mean square is that of the norm's weight
    for i, x in enumerate(layers):
        last = "norm2" if cfg["layers"][i]["mlp"] is not None else "norm1"
        ratio = x / w[f"l{i}.{last}"]
        assert torch.allclose((ratio * ratio).mean(-1), torch.ones(40, dtype=F64), atol=1e-3)


def test_configuration_reader_and_layout():
    from shrike_amd.config.registry import ConfigError, get_architecture
    from shrike_amd.models.poresun import cache_windows

    arch = get_architecture("Poresun")
    cfg = arch.config_cls.from_dict(POR_A)
    assert arch.config_cls.from_dict(cfg.to_dict()) == cfg
    spec = arch.build_spec(cfg)
    assert [e.cache_of for e in spec.schedule] == [None, None, 0, None, 0]
    assert spec.blocks[2].mixer.shared_kv and not spec.blocks[0].mixer.shared_kv and spec.blocks[2].ffn is None
    assert spec.blocks[1].mixer.qk_norm == (1e-6, False) and spec.blocks[0].mixer.qk_norm == (1e-6, True)
    assert spec.tie_word_embeddings and spec.embedding.scale == 3.0 and spec.blocks[3].alpha == POR_A["postln_alpha"]
    _, model = _weights_for(POR_A)
    names = {p.name for p in model.params() if not p.optional}
    assert {"embed", "final.norm", "l0.mix.q.norm", "l0.mix.k.norm", "l0.mix.rel", "l0.ls1", "l0.ls2", "l1.mlp.gate",
            "l2.mix.q", "l2.mix.q.norm", "l2.mix.rel", "l3.mix.g", "l3.mix.dkv.norm", "l0.mlp.router.b", "l0.mlp.shared.sg",
            "l0.mlp.e4.up", "l3.mlp.e8.down"} <= names
    assert not {"l2.mix.k", "l2.mix.v", "l2.mix.k.norm", "l2.norm2", "l2.ls2", "l1.mix.q.norm", "l0.mlp.e0.gate",
                "l4.mlp.shared.up", "head"} & names
    # a causal layer that reads a windowed layer's cache: that cache keeps everything
    b = arch.config_cls.from_dict(POR_B)
    assert cache_windows(b) == {1: 1, 2: None}
    specs = arch.build_spec(b)
    assert specs.blocks[2].mixer.window == 37 and specs.blocks[2].mixer.cache_window is None
    from shrike_amd.models import DecoderModel

    kept = DecoderModel(specs).cache_specs()
    assert kept[2].window is None and kept[1].window == 1 and kept[3] is None
    for broken, text in (
        ({**POR_A, "layers": [{**POR_A["layers"][2]}]}, "earlier layer"),
        ({**POR_A, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]}, "unknown mixer"),
        ({**POR_A, "layers": [{**POR_A["layers"][0], "mlp": {"kind": "glu"}}]}, "unknown feed-forward"),
        ({k: v for k, v in POR_A.items() if k != "norm"}, "norm"),
    ):
        with pytest.raises(ConfigError, match=text):
            arch.config_cls.from_dict(broken)


def test_a_bias_tables_rows_are_the_files_own(tmp_path):
    """config.json need not count the bias table's rows: the tensor's shape gives them, the loader
    accepts any count for that size alone, and the engine's table by distance follows the file."""
    import json

    from shrike_amd.config.registry import load_model_config
    from shrike_amd.models import DecoderModel
    from shrike_amd.weights import write_model_folder
    from shrike_amd.weights.loader import WeightError, _index, check_names, shard_files

    folder = write_model_folder(dict(POR_A), tmp_path / "m", seed=3, dtype="float32")
    cfg = json.loads((folder / "config.json").read_text())
    for layer in cfg["layers"]:
        layer["mixer"].pop("bias_rows", None)
    (folder / "config.json").write_text(json.dumps(cfg))
    _, spec = load_model_config(folder)
    assert spec.blocks[0].mixer.bucket_bias == (None, 40)
    params = DecoderModel(spec).params()
    rel = next(p for p in params if p.name == "l0.mix.rel")
    assert rel.shape == (None, 4) and rel.drawn_shape() == (32, 4) and rel.matches((12, 4)) and not rel.matches((12, 5))
    check_names(_index(shard_files(folder)), params)  # 12, 7, 20 and 2 rows: all taken as they are
    # the plain form reads the same folder
    logits = P.PlainPoresun(folder).logits([1, 2, 3, 4, 5, 6, 7, 8, 9])
    assert torch.isfinite(logits).all()
    # another size of the same tensor is still an error
    wrong = [p if p.name != "l0.mix.rel" else type(p)(p.name, (None, 5), p.init, p.keep_float32) for p in params]
    with pytest.raises(WeightError, match="l0.mix.rel"):
        check_names(_index(shard_files(folder)), wrong)
