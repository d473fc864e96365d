"""What pins the plain form of Ligipel (tests/plain/ligipel.py), and the configuration
reader, without a GPU: each mechanism against a second, independent way of writing it."""

import copy
import math

import pytest
import torch

import shrike_amd.models  # noqa: F401  (registers the architectures)
from shrike_amd.config import registry  # (names through the module: another test reloads it)
from shrike_amd.models import DecoderModel
from shrike_amd.parts import StateSpec

from .plain import ligipel as plain
from .tiny_ligipel import CONFIGS

D = torch.float64


def test_config_reads_back_and_picks_the_parts():
    arch = registry.get_architecture("Ligipel")
    for name, raw in CONFIGS.items():
        cfg = arch.config_cls.from_dict(raw)
        assert arch.config_cls.from_dict(cfg.to_dict()) == cfg, name
        spec = arch.build_spec(cfg)
        want = {"parallel": "parallel_mixers", "retention": "retention"}
        assert [b.mixer.kind for b in spec.blocks] == [want[layer["type"]] for layer in raw["layers"]]
        assert [b.ffn is None for b in spec.blocks] == [layer["mlp"] is None for layer in raw["layers"]]
        for block, layer in zip(spec.blocks, raw["layers"]):
            if layer["type"] == "parallel":
                left, right = (m for _, m in block.mixer.branches)
                m = layer["mixer"]
                assert (left.num_heads, left.num_kv_heads, left.head_dim, left.value_dim, left.scale) == (
                    m["left"]["heads"], m["left"]["kv_heads"], m["left"]["dim"], m["left"]["vdim"], m["left"]["scale"])
                assert left.window == (m["left"]["mask"]["size"] if "mask" in m["left"] else None)
                assert (right.inner, right.state, right.dt_rank, right.conv) == tuple(
                    m["right"][k] for k in ("inner", "state", "dt_rank", "conv"))
            else:
                assert tuple(block.mixer.decay) == tuple(layer["mixer"]["decay"])
            if layer["mlp"] is not None:
                assert (block.ffn.experts, block.ffn.top, block.ffn.expert_size) == (
                    layer["mlp"]["router"]["experts"], layer["mlp"]["router"]["top"], layer["mlp"]["expert"]["ff"])
                assert block.ffn.shared_size == (layer["mlp"]["shared"]["ff"] if "shared" in layer["mlp"] else None)
        model = DecoderModel(spec)
        needs = model.cache_specs()
        assert len(needs) == len(raw["layers"])
        for layer, need in zip(raw["layers"], needs):
            if layer["type"] == "retention":
                m = layer["mixer"]
                assert isinstance(need, StateSpec) and need.shape == (m["heads"] * m["dim"] * m["vdim"],)


def test_the_tensor_names_are_the_designs():
    arch = registry.get_architecture("Ligipel")
    raw = CONFIGS["A"]
    model = DecoderModel(arch.build_spec(arch.config_cls.from_dict(raw)))
    names = {p.name: tuple(p.shape) for p in model.params()}
    w, left, right = raw["width"], raw["layers"][0]["mixer"]["left"], raw["layers"][0]["mixer"]["right"]
    for name, shape in {
        "embed": (raw["vocab"], w), "embed.norm": (w,), "embed.norm.b": (w,), "head": (raw["vocab"], w),
        "final.norm": (w,), "final.norm.b": (w,), "l0.norm1": (w,), "l0.norm1b.b": (w,), "l0.norm2b": (w,),
        "l0.mix.left.q": (left["heads"] * left["dim"], w), "l0.mix.left.v": (left["kv_heads"] * left["vdim"], w),
        "l0.mix.left.o": (w, left["heads"] * left["vdim"]), "l0.mix.left.r1": (left["heads"],),
        "l0.mix.left.talk": (left["heads"], left["heads"]), "l0.mix.left.out": (w,), "l0.mix.right.out": (w,),
        "l0.mix.right.in": (2 * right["inner"], w), "l0.mix.right.conv": (right["inner"], right["conv"]),
        "l0.mix.right.conv.b": (right["inner"],), "l0.mix.right.x": (right["dt_rank"] + 2 * right["state"], right["inner"]),
        "l0.mix.right.dt": (right["inner"], right["dt_rank"]), "l0.mix.right.dt.b": (right["inner"],),
        "l0.mix.right.A_log": (right["inner"], right["state"]), "l0.mix.right.D": (right["inner"],),
        "l0.mlp.e4.down": (w, 24), "l0.mlp.router": (5, w), "l0.mlp.correction": (5,), "l0.mlp.shared.gate": (40, w),
        "l1.mix.g": (2 * 20, w), "l1.mix.k": (2 * 16, w), "l0.dwa": (2,), "l3.dwa": (5,),
    }.items():
        assert names.get(name) == shape, (name, names.get(name))
    assert not any(n.startswith("l2.mlp") for n in names) and "l1.mlp.shared.up" not in names


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown mixer type"),
    (lambda c: c["layers"][0]["mixer"]["left"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["right"].pop("dt_rank"), "dt_rank"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "decays"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=5), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "feed-forward kind"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_config_errors_name_the_key(change, message):
    raw = copy.deepcopy(CONFIGS["A"])
    change(raw)
    with pytest.raises(registry.ConfigError, match=message):
        registry.get_architecture("Ligipel").config_cls.from_dict(raw)


# ------------------------------------------------------------------ the plain form, mechanism by mechanism

def test_layer_norm_and_unit_rms_by_hand():
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=D)
    w, b = torch.tensor([1.0, 2.0, 0.5, -1.0], dtype=D), torch.tensor([0.1, 0.0, -0.1, 1.0], dtype=D)
    var = ((1 - 3) ** 2 + (2 - 3) ** 2 + 0 + (6 - 3) ** 2) / 4
    want = torch.tensor([[-2.0, -1.0, 0.0, 3.0]], dtype=D) / math.sqrt(var + 0.5) * w + b
    assert torch.allclose(plain.layer_norm(x, w, b, 0.5), want)
    assert torch.allclose(plain.unit_rms(x, 0.5), x / math.sqrt((1 + 4 + 9 + 36) / 4 + 0.5))
    z = torch.linspace(-4, 4, 41, dtype=D)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))


def test_the_sink_is_a_key_of_score_zero_with_no_value():
    torch.manual_seed(0)
    n, H, G, dim, vdim = 9, 4, 2, 6, 5
    q, k, v = torch.randn(n, H, dim, dtype=D), torch.randn(n, G, dim, dtype=D), torch.randn(n, G, vdim, dtype=D)
    r1, r2 = torch.rand(H, dtype=D), torch.rand(H, dtype=D) + 0.5
    talk = torch.randn(H, H, dtype=D)
    window, scale = 4, 0.4
    got = plain.mixed_head_attention(q, k, v, scale, window, r1, r2, talk)
    # written out position by position with an explicit extra term
    want = torch.zeros(n, H, vdim, dtype=D)
    for i in range(n):
        lo = max(0, i - window + 1)
        p = torch.zeros(H, i + 1, dtype=D)
        for h in range(H):
            s = torch.stack([q[i, h] @ k[j, h // 2] * scale - r1[h] * math.log(1 + float(r2[h]) * (i - j))
                             for j in range(lo, i + 1)])
            full = torch.softmax(torch.cat([s, torch.zeros(1, dtype=D)]), dim=0)  # the sink is the last entry
            p[h, lo:] = full[:-1]
        mixed = talk @ p
        for h in range(H):
            want[i, h] = mixed[h] @ v[: i + 1, h // 2]
    assert torch.allclose(got, want, atol=1e-12)
    # no mixing: the identity in its place
    assert torch.allclose(plain.mixed_head_attention(q, k, v, scale, window, r1, r2, None),
                          plain.mixed_head_attention(q, k, v, scale, window, r1, r2, torch.eye(H, dtype=D)))


def test_causal_convolution_by_hand():
    x = torch.tensor([[1.0], [2.0], [4.0], [8.0]], dtype=D)
    taps = torch.tensor([[100.0, 10.0, 1.0]], dtype=D)  # the last column meets the current token
    got = plain.causal_conv(x, taps, torch.tensor([0.5], dtype=D))
    assert got.flatten().tolist() == [1.5, 12.5, 124.5, 248.5]


def test_the_scan_carries_its_state_and_equals_the_unrolled_sum():
    torch.manual_seed(1)
    n, inner, N = 11, 3, 4
    x, dt = torch.randn(n, inner, dtype=D), torch.rand(n, inner, dtype=D)
    A = -torch.rand(inner, N, dtype=D)
    B, C, skip = torch.randn(n, N, dtype=D), torch.randn(n, N, dtype=D), torch.randn(inner, dtype=D)
    y, S = plain.scan(x, dt, A, B, C, skip)
    # y_t = sum_{s <= t} exp(A * sum_{s < r <= t} dt_r) dt_s x_s B_s . C_t + D x_t
    want = torch.zeros(n, inner, dtype=D)
    for t in range(n):
        for s in range(t + 1):
            decay = torch.exp(A * dt[s + 1: t + 1].sum(dim=0)[:, None])
            want[t] += (decay * (dt[s] * x[s])[:, None] * B[s][None, :]) @ C[t]
        want[t] += skip * x[t]
    assert torch.allclose(y, want, atol=1e-12)
    y1, S1 = plain.scan(x[:4], dt[:4], A, B[:4], C[:4], skip)
    y2, S2 = plain.scan(x[4:], dt[4:], A, B[4:], C[4:], skip, S1)
    assert torch.allclose(torch.cat([y1, y2]), y) and torch.allclose(S2, S)


def test_rotation_turns_pairs_half_a_head_apart():
    x = torch.zeros(1, 1, 6, dtype=D)
    x[0, 0] = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    got = plain.rotate_half(x, torch.tensor([3]), 4, 100.0)[0, 0]
    a0, a1 = 3.0, 3.0 * 100.0 ** (-2 / 4)
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(got, torch.tensor(want, dtype=D))
    assert torch.equal(plain.rotate_half(x, torch.tensor([0]), 4, 100.0), x)


def test_retention_equals_decayed_linear_attention():
    torch.manual_seed(2)
    n, H, dim, vdim = 10, 2, 3, 4
    q, k, v = torch.randn(n, H, dim, dtype=D), torch.randn(n, H, dim, dtype=D), torch.randn(n, H, vdim, dtype=D)
    decay = [0.9, 1.0]
    o, S = plain.retention(q, k, v, decay)
    want = torch.zeros(n, H, vdim, dtype=D)
    for t in range(n):
        for s in range(t + 1):
            for h in range(H):
                want[t, h] += decay[h] ** (t - s) * (q[t, h] @ k[s, h]) * v[s, h]
    assert torch.allclose(o, want, atol=1e-12)
    o1, S1 = plain.retention(q[:3], k[:3], v[:3], decay)
    o2, S2 = plain.retention(q[3:], k[3:], v[3:], decay, S1)
    assert torch.allclose(torch.cat([o1, o2]), o) and torch.allclose(S2, S)


def test_router_by_hand():
    w = {"m.router": torch.eye(4, dtype=D), "m.correction": torch.tensor([0.0, 0.0, 10.0, 0.0], dtype=D)}
    h = torch.tensor([[3.0, 2.0, 0.0, 1.0]], dtype=D)
    chosen, weights = plain.route(h, w, "m", 4, 2)
    s = torch.softmax(h[0].float(), dim=0)
    assert chosen.tolist() == [[2, 0]]  # the correction brings expert 2 in; its weight is its own score
    assert torch.allclose(weights[0], torch.stack([s[2], s[0]]) / (s[2] + s[0]))


def test_mixture_is_the_weighted_sum_of_the_chosen_experts():
    torch.manual_seed(3)
    width, ff, E, top, n = 6, 5, 4, 2, 7
    w = {"m.router": torch.randn(E, width, dtype=D), "m.correction": torch.randn(E, dtype=D)}
    for e in list(range(E)) + ["shared"]:
        p = f"m.e{e}" if e != "shared" else "m.shared"
        w[p + ".gate"], w[p + ".up"], w[p + ".down"] = (torch.randn(ff, width, dtype=D), torch.randn(ff, width, dtype=D),
                                                        torch.randn(width, ff, dtype=D))
    h = torch.randn(n, width, dtype=D)
    mlp = {"router": {"experts": E, "top": top}, "expert": {"ff": ff}, "shared": {"ff": ff}}
    got = plain.mixture(h, w, "m", mlp)
    chosen, weights = plain.route(h, w, "m", E, top)
    for t in range(n):
        want = plain.gated_expert(h[t:t + 1], w, "m.shared")[0]
        for j in range(top):
            want = want + weights[t, j] * plain.gated_expert(h[t:t + 1], w, f"m.e{int(chosen[t, j])}")[0]
        assert torch.allclose(got[t], want, atol=1e-12)


@pytest.mark.parametrize("name", ["A", "B"])
def test_the_whole_model_is_causal_and_its_first_token_stands_alone(name, tmp_path):
    from .tiny_ligipel import make_model_dir

    model = plain.PlainLigipel(make_model_dir(name, tmp_path))
    ids = [3, 50, 7, 7, 90, 12, 64, 1, 33, 8, 21, 5]
    full = model.logits(ids)
    assert torch.allclose(model.logits(ids[:5]), full[:5], atol=1e-6)
    assert torch.allclose(model.logits(ids[:1]), full[:1], atol=1e-6)
    other = model.logits(ids[:6] + [9] + ids[7:])
    assert torch.allclose(other[:6], full[:6], atol=1e-6) and not torch.allclose(other[6:], full[6:], atol=1e-3)
    cap = model.cfg.get("logit_softcap")
    if cap:
        assert float(full.abs().max()) < cap
