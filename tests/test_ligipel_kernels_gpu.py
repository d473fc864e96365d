"""The kernels that the Ligipel decoder brought, each alone against a plain computation
(tests/plain/ligipel.py): the layer norm around the float32 stream and the normed addend;
the weighted sum over the layers' results; the logits' scale and cap; attention with a
distance bias, a sink and mixed heads, with one key made to stand out far back, at page
borders and just inside and just outside the window, in prompt portions and single tokens,
shared among workgroups or not; the short convolution, the step sizes and the selective
scan in pieces against the whole, in slots that are used again; the rotation of float32
rows; the retention scan in pieces; the router's choice (the correction moves the choice
and not the weights, ties go to the lower index) and the experts' products."""

import math

import pytest
import torch

from .plain import ligipel as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 3e-5, torch.bfloat16: 1.6e-2}


@pytest.fixture(scope="module")
def ops():
    from shrike_amd.kernels import ops

    return ops


def dev(t, dtype=None):
    return t.to("cuda", dtype).contiguous() if dtype else t.to("cuda").contiguous()


def i32(x):
    return torch.as_tensor(x, dtype=torch.int32).to("cuda")


def close(got, want, dtype, what="", tol=None):
    want = want.double().cpu()
    err = float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= (tol or TOL[dtype]), f"{what} rel err {err:.3e} > {tol or TOL[dtype]}"


def step_arrays(starts, lens):
    """positions, token_seq, cu_q of a step whose sequence s brings lens[s] tokens from starts[s]."""
    positions = torch.cat([torch.arange(s, s + l) for s, l in zip(starts, lens)])
    token_seq = torch.cat([torch.full((l,), i) for i, l in enumerate(lens)])
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)))
    return i32(positions), i32(token_seq), i32(cu)


# ------------------------------------------------------------------ norms and the stream

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n, hidden", [(1, 8), (5, 100), (33, 256), (3, 1030)])
def test_layer_norm_of_the_stream_and_of_the_addend(ops, dtype, n, hidden):
    torch.manual_seed(n * hidden)
    x = torch.randn(n, hidden, dtype=torch.float64) * 3 + 1.5  # a mean that is not zero
    delta = (torch.randn(n, hidden) * 2 - 0.7).to(dtype)
    w, b, dw, db = (torch.randn(hidden, dtype=torch.float32) for _ in range(4))
    eps, deps = 1e-5, 3e-3
    # the norm alone
    out = torch.empty(n, hidden, dtype=dtype, device="cuda")
    resid = dev(x, torch.float32)
    ops.add_layernorm(resid, None, None, dev(w), dev(b), eps, out=out)
    close(out, plain.layer_norm(resid.double().cpu(), w.double(), b.double(), eps), dtype, "norm")
    # the stream gains a normed addend, then is normed for the next sublayer
    ops.add_layernorm(resid, dev(delta), (dev(dw), dev(db), deps), dev(w), dev(b), eps, out=out)
    want = x.float().double() + plain.layer_norm(delta.double(), dw.double(), db.double(), deps)
    close(resid, want, torch.float32, "stream", tol=1e-5)
    close(out, plain.layer_norm(want, w.double(), b.double(), eps), dtype, "normed sum")


def test_layer_norm_of_chosen_rows(ops):
    torch.manual_seed(3)
    x = torch.randn(9, 48)
    w, b = torch.randn(48), torch.randn(48)
    rows = [7, 0, 7, 3]
    out = torch.empty(len(rows), 48, dtype=torch.float32, device="cuda")
    ops.add_layernorm(dev(x), None, None, dev(w), dev(b), 1e-6, out=out, rows=i32(rows), write_resid=False)
    close(out, plain.layer_norm(x[rows].double(), w.double(), b.double(), 1e-6), torch.float32)


@pytest.mark.parametrize("count", [1, 2, 5])
def test_weighted_sum_over_the_layers_results(ops, count):
    torch.manual_seed(count)
    n, hidden = 6, 70
    history = torch.randn(count + 2, n, hidden)
    coef = torch.randn(count + 1)
    out = torch.empty(n, hidden, device="cuda")
    ops.mix_history(dev(history), dev(coef), count, out)
    want = sum(coef[j].double() * history[j].double() for j in range(count))
    close(out, want, torch.float32)
    # the last entry first gains a normed addend
    delta = torch.randn(n, hidden).to(torch.bfloat16)
    dw, db = torch.randn(hidden), torch.randn(hidden)
    h = dev(history)
    ops.mix_history(h, dev(coef), count, out, delta=dev(delta), dnorm=(dev(dw), dev(db), 1e-5))
    last = history[count - 1].double() + plain.layer_norm(delta.double(), dw.double(), db.double(), 1e-5)
    close(h[count - 1], last, torch.float32, "entry", tol=1e-5)
    close(out, want - coef[count - 1].double() * history[count - 1].double() + coef[count - 1].double() * last,
          torch.float32, "sum", tol=1e-5)


@pytest.mark.parametrize("scale, cap", [(0.5, 30.0), (1.0, None), (2.5, 0.75)])
def test_logits_scale_and_cap(ops, scale, cap):
    torch.manual_seed(0)
    x = torch.randn(4, 333) * 20
    got = dev(x)
    ops.scale_softcap(got, scale, cap)
    want = x.double() * scale
    close(got, want if cap is None else cap * torch.tanh(want / cap), torch.float32)


# ------------------------------------------------------------------ attention with mixed heads

def fill_pools(ops, k, v, table, page_size, pages, dtype):
    """Pools that hold one sequence's keys [n, G, D] and values [n, G, V] in the pages of `table`."""
    n, G, D = k.shape
    V = v.shape[2]
    slab = ops.key_slab(D)
    k_pool = torch.full(ops.key_pool_shape(pages, G, page_size, D), 1e4)  # pages of others: large, never read
    v_pool = torch.full((pages, G, V, page_size), -1e4)
    for j in range(n):
        page, at = table[j // page_size], j % page_size
        k_pool[page, :, :, at, :] = k[j].view(G, D // slab, slab)
        v_pool[page, :, :, at] = v[j]
    return dev(k_pool, dtype), dev(v_pool, dtype)


def talking_case(H, G, D, V, n, seed, window):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n, H, D, generator=g)
    k = torch.randn(n, G, D, generator=g)
    v = torch.randn(n, G, V, generator=g)
    r1 = torch.rand(H, generator=g) * 0.8
    r2 = torch.rand(H, generator=g) * 2 + 0.1
    talk = torch.eye(H) * 0.7 + torch.randn(H, H, generator=g) * 0.3
    return q, k, v, r1, r2, talk


def run_talking(ops, q, k, v, r1, r2, talk, window, scale, dtype, page_size, cuts, sink=0.0, nshare=1):
    """The kernel over one sequence cut into steps of cuts[i] tokens; the keys and values of
    all positions are in the cache beforehand (a query reads none after itself)."""
    n, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    pages = -(-n // page_size) + 3
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(n)).tolist()
    table = perm[: -(-n // page_size)]
    k_pool, v_pool = fill_pools(ops, k.to(dtype).float(), v.to(dtype).float(), table, page_size, pages, dtype)
    tables = i32([table])
    got = torch.empty(n, H * V, dtype=dtype, device="cuda")
    at = 0
    for c in cuts:
        positions, token_seq, _ = step_arrays([at], [c])
        scratch = torch.empty(ops.attention_talking_scratch_floats(c, H, V, nshare), device="cuda")
        out = torch.empty(c, H * V, dtype=dtype, device="cuda")
        ops.attention_talking(dev(q[at:at + c].reshape(c, H * D), dtype), out, H, G, D, V, positions, token_seq, tables,
                              k_pool, v_pool, page_size, window, scale, scratch, r1=None if r1 is None else dev(r1),
                              r2=None if r2 is None else dev(r2), talk=None if talk is None else dev(talk), sink=sink,
                              nshare=nshare)
        got[at:at + c] = out
        at += c
    assert at == n
    return got


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, V, n, window, page_size", [
    (4, 2, 32, 16, 50, 7, 16),      # a window smaller than a page
    (3, 1, 24, 40, 70, 33, 4),      # heads that are no power of two, a head size that is no multiple of 32
    (2, 2, 64, 64, 150, None, 16),  # no window: more than two tiles of keys
    (6, 3, 16, 8, 90, 64, 8),       # a window of exactly a tile
    (1, 1, 8, 8, 20, 1, 16),        # a window of one: a token sees itself and the sink
])
def test_mixed_head_attention_against_the_plain_form(ops, dtype, H, G, D, V, n, window, page_size):
    q, k, v, r1, r2, talk = talking_case(H, G, D, V, n, 11 + n, window)
    scale = 0.3
    rd = lambda t: t.to(dtype).double()  # noqa: E731
    want = plain.mixed_head_attention(rd(q), rd(k), rd(v), scale, window, r1.double(), r2.double(), talk.double())
    whole = run_talking(ops, q, k, v, r1, r2, talk, window, scale, dtype, page_size, [n])
    close(whole, want.reshape(n, H * V), dtype, "whole")
    # portions down to two tokens, then single tokens: the same bits in float32
    cuts = [5, 2, 17, 2, 3] + [1] * (n - 29) if n > 29 else [3, 2] + [1] * (n - 5)
    pieces = run_talking(ops, q, k, v, r1, r2, talk, window, scale, dtype, page_size, cuts)
    close(pieces, want.reshape(n, H * V), dtype, "pieces")
    if dtype == torch.float32:
        assert torch.equal(pieces, whole)
    # single tokens whose keys are shared among workgroups
    shared = run_talking(ops, q, k, v, r1, r2, talk, window, scale, dtype, page_size, [n - 3, 1, 1, 1], nshare=3)
    close(shared, want.reshape(n, H * V), dtype, "shared")


def test_each_option_of_the_attention_alone(ops):
    """No bias, no sink, no mixing; then one of them at a time: what is left out is not computed."""
    H, G, D, V, n = 4, 2, 16, 16, 40
    q, k, v, r1, r2, talk = talking_case(H, G, D, V, n, 5, None)
    d = lambda t: t.double()  # noqa: E731
    for bias, sink, mix in [(False, False, False), (True, False, False), (False, True, False), (False, False, True)]:
        want = plain.mixed_head_attention(d(q), d(k), d(v), 0.25, 12, d(r1) if bias else None, d(r2) if bias else None,
                                          d(talk) if mix else None, sink=sink)
        got = run_talking(ops, q, k, v, r1 if bias else None, r2 if bias else None, talk if mix else None, 12, 0.25,
                          torch.float32, 8, [n], sink=0.0 if sink else None)
        close(got, want.reshape(n, H * V), torch.float32, f"bias={bias} sink={sink} mix={mix}")


@pytest.mark.parametrize("cuts", ["whole", "decode"])
def test_a_key_that_stands_out_shows_where_the_window_ends(ops, cuts):
    """One key is made so large that its weight is nearly one wherever it is seen, and its
    value is a marker: the marker shows in the output of exactly the positions whose window
    holds the key, at a page border, a tile's border and far back."""
    H, G, D, V, page_size = 2, 1, 16, 4, 16
    n = 420
    for target, window in [(15, 16), (16, 33), (63, 64), (64, 65), (3, 400), (130, 141), (200, 1)]:
        g = torch.Generator().manual_seed(target)
        q = torch.randn(n, H, D, generator=g) * 0.1
        k = torch.randn(n, G, D, generator=g) * 0.1
        v = torch.randn(n, G, V, generator=g) * 0.01
        q[:, :, 0] = 6.0
        k[target, 0, 0] = 6.0  # score 36 * scale against ~0 elsewhere
        v[target, 0] = torch.tensor([100.0, -100.0, 50.0, 25.0])
        r1, r2 = torch.tensor([0.5, 0.0]), torch.tensor([1.0, 3.0])
        talk = torch.tensor([[1.0, 0.0], [0.25, 0.75]])
        steps = [n] if cuts == "whole" else [target + 1] + [1] * (n - target - 1)
        got = run_talking(ops, q, k, v, r1, r2, talk, window, 1.0, torch.float32, page_size, steps).cpu()
        seen = got[:, 0].abs() > 30.0  # head 0, first value
        want = torch.zeros(n, dtype=torch.bool)
        want[target:min(n, target + window)] = True
        assert torch.equal(seen, want), f"target {target} window {window}: seen at {seen.nonzero().flatten().tolist()[:8]}.."
        d = lambda t: t.double()  # noqa: E731
        close(got, plain.mixed_head_attention(d(q), d(k), d(v), 1.0, window, d(r1), d(r2), d(talk)).reshape(n, H * V),
              torch.float32, f"target {target}")


def test_the_sink_takes_its_share(ops):
    """Scores far below zero: almost all of the softmax goes to the sink and the output is
    near nothing; without the sink the same scores give an average of the values."""
    H, G, D, V, n = 2, 2, 8, 8, 12
    q = torch.ones(n, H, D)
    k = -torch.ones(n, G, D)
    v = torch.ones(n, G, V)
    with_sink = run_talking(ops, q, k, v, None, None, None, None, 1.0, torch.float32, 4, [n], sink=0.0)
    without = run_talking(ops, q, k, v, None, None, None, None, 1.0, torch.float32, 4, [n], sink=None)
    assert float(with_sink.abs().max()) < (n * math.exp(-8.0)) * 1.01
    close(without, torch.ones(n, H * V), torch.float32)
    # a single key of score 0 beside the sink of score 0: half each
    half = run_talking(ops, torch.zeros(1, H, D), k[:1], v[:1], None, None, None, None, 1.0, torch.float32, 4, [1])
    close(half, torch.full((1, H * V), 0.5), torch.float32)


def test_batch_of_unequal_requests_in_pages_that_others_used(ops):
    """Three sequences in one step (a portion, a single token far on, a first token) give what
    each gives alone."""
    H, G, D, V, page_size = 4, 2, 32, 32, 8
    lens, starts, steps = [60, 141, 1], [37, 140, 0], [23, 1, 1]
    pages = 40
    k_pool = torch.full(ops.key_pool_shape(pages, G, page_size, D), 50.0)
    v_pool = torch.full((pages, G, V, page_size), 50.0)
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(1)).tolist()
    tables, cases = [], []
    for s, n in enumerate(lens):
        q, k, v, r1, r2, talk = talking_case(H, G, D, V, n, 100, None)  # the same learned numbers for all
        g = torch.Generator().manual_seed(200 + s)
        q, k, v = torch.randn(n, H, D, generator=g), torch.randn(n, G, D, generator=g), torch.randn(n, G, V, generator=g)
        table = [perm.pop() for _ in range(-(-n // page_size))]
        for j in range(n):
            k_pool[table[j // page_size], :, :, j % page_size, :] = k[j].view(G, D // 32, 32)
            v_pool[table[j // page_size], :, :, j % page_size] = v[j]
        tables.append(table + [0] * (20 - len(table)))
        cases.append((q, k, v))
    positions, token_seq, _ = step_arrays(starts, steps)
    rows = torch.cat([cases[s][0][starts[s]:starts[s] + steps[s]].reshape(steps[s], H * D) for s in range(3)])
    out = torch.empty(rows.shape[0], H * V, device="cuda")
    scratch = torch.empty(ops.attention_talking_scratch_floats(rows.shape[0], H, V, 1), device="cuda")
    ops.attention_talking(dev(rows), out, H, G, D, V, positions, token_seq, i32(tables), dev(k_pool), dev(v_pool),
                          page_size, 50, 0.2, scratch, r1=dev(r1), r2=dev(r2), talk=dev(talk), sink=0.0)
    at = 0
    for s in range(3):
        q, k, v = (t.double() for t in cases[s])
        want = plain.mixed_head_attention(q, k, v, 0.2, 50, r1.double(), r2.double(), talk.double())
        close(out[at:at + steps[s]], want[starts[s]:starts[s] + steps[s]].reshape(steps[s], H * V), torch.float32, f"seq {s}")
        at += steps[s]


# ------------------------------------------------------------------ the selective scan

def scan_weights(inner, states, rank, taps, seed):
    g = torch.Generator().manual_seed(seed)
    return {
        "conv": torch.randn(inner, taps, generator=g) * 0.5, "conv.b": torch.randn(inner, generator=g) * 0.1,
        "dt": torch.randn(inner, rank, generator=g) * 0.3, "dt.b": torch.randn(inner, generator=g),
        "A_log": torch.randn(inner, states, generator=g) * 0.5, "D": torch.randn(inner, generator=g),
    }


def plain_scan_chain(u, z, low, w, rank, states):
    """conv + silu, step sizes, scan, gate: from the in-projection's halves and W_x's output."""
    x = plain.silu(plain.causal_conv(u, w["conv"].double(), w["conv.b"].double()))
    dt = torch.nn.functional.softplus(low[:, :rank] @ w["dt"].double().T + w["dt.b"].double())
    y, _ = plain.scan(x, dt, -torch.exp(w["A_log"].double()), low[:, rank:rank + states], low[:, rank + states:],
                      w["D"].double())
    return x, y * plain.silu(z)


def run_scan_chain(ops, uz, low_of, w, inner, states, rank, taps, dtype, state, plan):
    """plan: steps of [(sequence, slot, start, count)]; uz[s] holds a sequence's in-projection
    rows; low_of(x) gives W_x's float32 output for conv outputs x (the test's own product)."""
    got = {s: torch.zeros(uz[s].shape[0], inner, dtype=dtype, device="cuda") for s in uz}
    wd = {k: dev(v) for k, v in w.items()}
    wd["dt"] = dev(w["dt"].t())  # the step-size matrix goes in transposed
    for step in plan:
        starts, lens = [st for _, _, st, _ in step], [c for _, _, _, c in step]
        positions, token_seq, cu = step_arrays(starts, lens)
        slots = i32([slot for _, slot, _, _ in step])
        rows = dev(torch.cat([uz[s][st:st + c] for s, _, st, c in step]), dtype)
        n = rows.shape[0]
        x = torch.empty(n, inner, dtype=dtype, device="cuda")
        ops.conv_silu(rows, wd["conv"], wd["conv.b"], positions, token_seq, cu, slots, state, states, x)
        low = dev(low_of(x.double().cpu()), torch.float32)
        dt = torch.empty(n, inner, device="cuda")
        ops.dt_softplus(low, wd["dt"], wd["dt.b"], dt)
        out = torch.empty(n, inner, dtype=dtype, device="cuda")
        ops.selective_scan(dt, x, low, rank, rank + states, rows[:, inner:], wd["A_log"], wd["D"], states, taps, rows,
                           positions, cu, slots, state, out, len(step))
        at = 0
        for s, _, st, c in step:
            got[s][st:st + c] = out[at:at + c]
            at += c
    return got


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inner, states, rank, taps", [(40, 3, 2, 2), (96, 12, 5, 4), (50, 70, 7, 1), (72, 33, 9, 3),
                                                       (300, 16, 30, 5), (24, 300, 3, 2)])
def test_selective_scan_in_pieces_and_in_used_slots(ops, dtype, inner, states, rank, taps):
    torch.manual_seed(inner)
    w = scan_weights(inner, states, rank, taps, inner + states)
    wx = torch.randn(rank + 2 * states, inner, dtype=torch.float64) * inner**-0.5
    low_of = lambda x: (x @ wx.T).float().double()  # noqa: E731
    lens = {"a": 37, "b": 9, "c": 1, "d": 14}
    uz = {s: (torch.randn(n, 2 * inner) * 1.5).to(dtype).double() for s, n in lens.items()}
    floats = ops.selective_scan_state_floats(inner, states, taps)
    state = torch.full((3, floats), 7.0, device="cuda")  # what earlier holders left behind
    plan = [
        [("a", 0, 0, 5), ("b", 2, 0, 1)],                    # first tokens: a portion and a single one
        [("a", 0, 5, 1), ("b", 2, 1, 2), ("c", 1, 0, 1)],    # a, b go on; c is one token long
        [("a", 0, 6, 2)],                                    # b is left out of a step
        [("b", 2, 3, 6), ("a", 0, 8, 29), ("d", 1, 0, 3)],   # d takes c's slot
        [("d", 1, 3, 1)], [("d", 1, 4, 1)], [("d", 1, 5, 9)],
    ]
    got = run_scan_chain(ops, uz, low_of, w, inner, states, rank, taps, dtype, state, plan)
    for s in lens:
        u, z = uz[s][:, :inner], uz[s][:, inner:]
        # the oracle follows the kernel's roundings of the convolution's output
        x = plain.silu(plain.causal_conv(u, w["conv"].double(), w["conv.b"].double())).to(dtype).double()
        low = low_of(x)
        dt = torch.nn.functional.softplus(low[:, :rank] @ w["dt"].double().T + w["dt.b"].double())
        y, _ = plain.scan(x, dt, -torch.exp(w["A_log"].double()), low[:, rank:rank + states], low[:, rank + states:],
                          w["D"].double())
        close(got[s], y * plain.silu(z), dtype, f"sequence {s}", tol=5e-5 if dtype == torch.float32 else 2.5e-2)


def test_selective_scan_keeps_a_far_input(ops):
    """A channel whose decay is almost one keeps an input from 500 tokens back; one whose
    decay is fast has lost it.  Decoded token by token after a prompt."""
    inner, states, rank, taps, n = 4, 2, 1, 2, 520
    w = {"conv": torch.tensor([[0.0, 1.0]] * inner), "conv.b": torch.zeros(inner), "dt": torch.zeros(inner, rank),
         "dt.b": torch.full((inner,), 0.5413),  # softplus -> 1.0
         "A_log": torch.tensor([[-12.0, -12.0], [-12.0, -12.0], [1.0, 1.0], [1.0, 1.0]]), "D": torch.zeros(inner)}
    u = torch.zeros(n, 2 * inner, dtype=torch.float64)
    u[:, inner:] = 5.0     # gates wide open
    u[7, :inner] = 4.0     # the one input
    low_of = lambda x: torch.ones(x.shape[0], rank + 2 * states, dtype=torch.float64)  # noqa: E731
    state = torch.zeros(1, ops.selective_scan_state_floats(inner, states, taps), device="cuda")
    plan = [[("s", 0, 0, 20)]] + [[("s", 0, t, 1)] for t in range(20, n)]
    got = run_scan_chain(ops, {"s": u}, low_of, w, inner, states, rank, taps, torch.float32, state, plan)["s"].cpu()
    _, want = plain_scan_chain(u[:, :inner], u[:, inner:], low_of(u), w, rank, states)
    close(got, want, torch.float32)
    assert float(got[-1, 0]) > 1.0 and abs(float(got[-1, 2])) < 1e-6


# ------------------------------------------------------------------ retention

@pytest.mark.parametrize("heads, dim, rot, base", [(2, 16, 16, 500.0), (3, 40, 6, 90.0), (1, 12, 0, 1.0), (2, 64, 32, 1e6)])
def test_rotation_of_float32_rows(ops, heads, dim, rot, base):
    torch.manual_seed(dim)
    n, off, ld = 9, 5, 5 + heads * dim + 3
    x = torch.randn(n, ld)
    positions = torch.tensor([0, 1, 2, 77, 64, 4095, 30000, 3, 1000])
    inv = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32) if rot else None
    got = dev(x)
    ops.rotate_half_rows(got, off, heads, dim, rot, None if inv is None else dev(inv), i32(positions), 0.37)
    want = x.double().clone()
    want[:, off:off + heads * dim] = (plain.rotate_half(x[:, off:off + heads * dim].double().view(n, heads, dim),
                                                        positions, rot, base) * 0.37).reshape(n, heads * dim)
    # angles are 32-bit products of a position and a frequency: at position p they are p * 2^-24 off at most
    close(got[:5], want[:5], torch.float32, tol=2e-5)
    close(got, want, torch.float32, tol=30000 * 2.0**-23)
    assert torch.equal(got[:, :off].cpu(), x[:, :off]) and torch.equal(got[:, off + heads * dim:].cpu(), x[:, off + heads * dim:])


@pytest.mark.parametrize("heads, dim, v_dim", [(2, 16, 20), (3, 40, 16), (1, 12, 50), (2, 64, 64), (4, 128, 32),
                                               (1, 600, 8), (3, 8, 3)])
def test_retention_scan_in_pieces_and_in_used_slots(ops, heads, dim, v_dim):
    torch.manual_seed(dim + v_dim)
    decay = torch.tensor([1.0, 0.5, 0.97, 0.999][:heads])
    lens = {"a": 41, "b": 6, "c": 13}
    qk, vv = heads * dim, heads * v_dim
    ld = 2 * qk + vv + 7
    proj = {s: torch.randn(n, ld) for s, n in lens.items()}
    state = torch.full((2, ops.retention_state_floats(heads, dim, v_dim)), -3.0, device="cuda")
    plan = [[("a", 0, 0, 2), ("b", 1, 0, 6)], [("a", 0, 2, 1)], [("a", 0, 3, 30), ("c", 1, 0, 1)],
            [("c", 1, 1, 1), ("a", 0, 33, 1)], [("c", 1, 2, 11), ("a", 0, 34, 7)]]
    got = {s: torch.zeros(n, vv, device="cuda") for s, n in lens.items()}
    for step in plan:
        starts, counts = [st for _, _, st, _ in step], [c for _, _, _, c in step]
        positions, _, cu = step_arrays(starts, counts)
        rows = dev(torch.cat([proj[s][st:st + c] for s, _, st, c in step]))
        out = torch.empty(rows.shape[0], vv, device="cuda")
        ops.retention_scan(rows, 3, 3 + qk, 3 + 2 * qk, dev(decay), len(step), heads, dim, v_dim, positions, cu,
                           i32([slot for _, slot, _, _ in step]), state, out)
        at = 0
        for s, _, st, c in step:
            got[s][st:st + c] = out[at:at + c]
            at += c
    for s, n in lens.items():
        p = proj[s].double()
        want, _ = plain.retention(p[:, 3:3 + qk].view(n, heads, dim), p[:, 3 + qk:3 + 2 * qk].view(n, heads, dim),
                                  p[:, 3 + 2 * qk:3 + 2 * qk + vv].view(n, heads, v_dim), decay.tolist())
        close(got[s], want.reshape(n, vv), torch.float32, f"sequence {s}")


def test_retention_keeps_a_far_key(ops):
    """With decay 1 the first token's value comes back whole 600 tokens later (decoded one by
    one); with decay 0.5 it is gone."""
    heads, dim, v_dim, n = 2, 4, 3, 600
    proj = torch.zeros(n, 2 * heads * dim + heads * v_dim)
    proj[0, heads * dim:2 * heads * dim] = 1.0   # k_0
    proj[0, 2 * heads * dim:] = 2.0              # v_0
    proj[:, :heads * dim] = 0.25                 # every q: q . k_0 = 1
    state = torch.full((1, ops.retention_state_floats(heads, dim, v_dim)), 9.0, device="cuda")
    last = None
    for start, count in [(0, 3)] + [(t, 1) for t in range(3, n)]:
        positions, _, cu = step_arrays([start], [count])
        last = torch.empty(count, heads * v_dim, device="cuda")
        ops.retention_scan(dev(proj[start:start + count]), 0, heads * dim, 2 * heads * dim, dev(torch.tensor([1.0, 0.5])),
                           1, heads, dim, v_dim, positions, cu, i32([0]), state, last)
    assert torch.allclose(last[0, :v_dim].cpu(), torch.full((v_dim,), 2.0)) and float(last[0, v_dim:].abs().max()) < 1e-30


# ------------------------------------------------------------------ experts

@pytest.mark.parametrize("experts, top", [(3, 3), (5, 2), (9, 1), (8, 3), (70, 6)])
def test_router_choice_and_weights(ops, experts, top):
    torch.manual_seed(experts)
    n = 37
    logits = torch.randn(n, experts) * 2
    correction = torch.randn(experts) * 0.3
    chosen = torch.empty(n, top, dtype=torch.int32, device="cuda")
    weights = torch.empty(n, top, device="cuda")
    ops.moe_route(dev(logits), dev(correction), top, chosen, weights)
    s = torch.softmax(logits.double(), dim=-1)
    want = torch.topk(s + correction.double(), top, dim=-1).indices
    assert torch.equal(chosen.cpu().long().sort(dim=-1).values, want.sort(dim=-1).values)
    picked = torch.gather(s, 1, chosen.cpu().long())
    close(weights, picked / picked.sum(dim=-1, keepdim=True), torch.float32)


def test_the_correction_moves_the_choice_and_not_the_weights(ops):
    logits = torch.tensor([[2.0, 1.0, 0.0, -1.0]])
    chosen = torch.empty(1, 2, dtype=torch.int32, device="cuda")
    weights = torch.empty(1, 2, device="cuda")
    ops.moe_route(dev(logits), dev(torch.tensor([0.0, 0.0, 0.0, 5.0])), 2, chosen, weights)
    s = torch.softmax(logits[0].double(), dim=-1)
    assert chosen.cpu().tolist() == [[3, 0]]
    close(weights, torch.stack([s[3], s[0]])[None] / (s[3] + s[0]), torch.float32)
    # equal scores: the lower index
    ops.moe_route(dev(torch.zeros(1, 4)), None, 2, chosen, weights)
    assert chosen.cpu().tolist() == [[0, 1]]
    close(weights, torch.full((1, 2), 0.5), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n, width, ff, experts, top, shared", [(1, 64, 24, 5, 2, True), (7, 100, 30, 4, 4, False),
                                                                (40, 128, 64, 8, 1, True), (130, 72, 20, 9, 3, False),
                                                                (300, 256, 96, 6, 2, True)])
def test_experts_products_against_the_plain_form(ops, dtype, n, width, ff, experts, top, shared):
    torch.manual_seed(n + width)
    x = torch.randn(n, width).to(dtype)
    wg, wu = (torch.randn(experts, ff, width) * width**-0.5).to(dtype), (torch.randn(experts, ff, width) * width**-0.5).to(dtype)
    wd = (torch.randn(experts, width, ff) * ff**-0.5).to(dtype)
    chosen = torch.stack([torch.randperm(experts)[:top] for _ in range(n)]).to(torch.int32)
    weights = torch.rand(n, top)
    weights = weights / weights.sum(dim=-1, keepdim=True)
    add = torch.randn(n, width).to(dtype) if shared else None
    act = torch.empty(n * top, ff, dtype=dtype, device="cuda")
    out = torch.empty(n, width, dtype=dtype, device="cuda")
    ops.moe_experts(dev(x), dev(chosen), dev(weights), dev(wg), dev(wu), dev(wd), act, out, "silu",
                    add=None if add is None else dev(add))
    want = torch.zeros(n, width, dtype=torch.float64) if add is None else add.double().clone()
    xd = x.double()
    for t in range(n):
        for j in range(top):
            e = int(chosen[t, j])
            hidden = plain.silu(wg[e].double() @ xd[t]) * (wu[e].double() @ xd[t])
            if dtype == torch.bfloat16:
                hidden = hidden.to(dtype).double()  # the activations between the two products have the compute dtype
            want[t] += weights[t, j].double() * (wd[e].double() @ hidden)
    close(out, want, dtype, tol=None if dtype == torch.float32 else 2e-2)
    # a token's result does not depend on the rest of the step
    alone = torch.empty(1, width, dtype=dtype, device="cuda")
    t = n // 2
    ops.moe_experts(dev(x[t:t + 1]), dev(chosen[t:t + 1]), dev(weights[t:t + 1]), dev(wg), dev(wu), dev(wd), act, alone,
                    "silu", add=None if add is None else dev(add[t:t + 1]))
    if dtype == torch.float32:
        assert torch.equal(alone[0], out[t])
    else:
        close(alone[0], out[t], dtype)


# ------------------------------------------------------------------ the same on the matrix units (bfloat16)

def run_talking_mfma(ops, seqs, steps, H, G, D, V, r1, r2, talk, window, scale, page_size, sink=0.0, nsplit=1):
    """seqs: {name: (q, k, v)}; steps: lists of (name, start, count), single tokens first.  Every
    sequence's keys and values are in the cache beforehand."""
    dtype = torch.bfloat16
    names = list(seqs)
    pages = sum(-(-seqs[s][0].shape[0] // page_size) for s in names) + 5
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(pages)).tolist()
    slab = ops.key_slab(D)
    k_pool = torch.full(ops.key_pool_shape(pages, G, page_size, D), float("nan"))  # what no one wrote is not a number
    v_pool = torch.full((pages, G, V, page_size), float("nan"))
    table_of, width = {}, max(-(-seqs[s][0].shape[0] // page_size) for s in names)
    for s in names:
        q, k, v = seqs[s]
        table = [perm.pop() for _ in range(-(-q.shape[0] // page_size))]
        for j in range(q.shape[0]):
            k_pool[table[j // page_size], :, :, j % page_size, :] = k[j].view(G, D // slab, slab)
            v_pool[table[j // page_size], :, :, j % page_size] = v[j]
        table_of[s] = table + [-1] * (width - len(table))
    k_pool, v_pool = dev(k_pool, dtype), dev(v_pool, dtype)
    got = {s: torch.zeros(seqs[s][0].shape[0], H * V, dtype=dtype, device="cuda") for s in names}
    for step in steps:
        starts, lens = [st for _, st, _ in step], [c for _, _, c in step]
        positions, token_seq, cu = step_arrays(starts, lens)
        single = sum(1 for c in lens if c == 1)
        assert all(c == 1 for c in lens[:single]) and all(c > 1 for c in lens[single:])
        tile_seq, tile_q0 = [], []
        for idx in range(single, len(step)):
            for q0 in range(0, lens[idx], 16):
                tile_seq.append(idx)
                tile_q0.append(q0)
        rows = dev(torch.cat([seqs[s][0][st:st + c].reshape(c, H * D) for s, st, c in step]), dtype)
        n = rows.shape[0]
        out = torch.empty(n, H * V, dtype=dtype, device="cuda")
        scratch = torch.empty(ops.attention_talking_mfma_scratch_floats(n, H, G, V, single, nsplit), device="cuda")
        ops.attention_talking_mfma(rows, out, single, H, G, D, V, positions, token_seq, cu,
                                   i32(tile_seq) if tile_seq else None, i32(tile_q0) if tile_q0 else None, len(tile_seq),
                                   i32([table_of[s] for s, _, _ in step]), k_pool, v_pool, page_size, window, scale, scratch,
                                   r1=None if r1 is None else dev(r1), r2=None if r2 is None else dev(r2),
                                   talk=None if talk is None else dev(talk), sink=sink, nsplit=nsplit)
        at = 0
        for s, st, c in step:
            got[s][st:st + c] = out[at:at + c]
            at += c
    return got


@pytest.mark.parametrize("H, G, D, V, window, page_size", [
    (4, 2, 32, 16, 7, 16),       # a window smaller than a page; values smaller than keys
    (3, 1, 24, 40, 33, 8),       # a head size that is no multiple of 32, value blocks with a ragged end
    (2, 2, 64, 64, None, 16),    # no window
    (6, 3, 16, 8, 64, 8),
    (8, 8, 128, 128, 100, 16),   # as many key/value heads as heads: value heads in several passes
    (20, 1, 8, 24, 50, 32),      # more heads of a key/value head than a tile has rows
    (4, 2, 256, 256, 45, 16),
])
def test_mixed_head_attention_on_the_matrix_units(ops, H, G, D, V, window, page_size):
    dtype = torch.bfloat16
    assert ops.attention_talking_supports_mfma(D, V, page_size, H * D)
    lens = {"a": 150, "b": 37, "c": 1, "d": 70}
    seqs, want = {}, {}
    _, _, _, r1, r2, talk = talking_case(H, G, D, V, 1, 77, window)
    talk = talk.to(dtype).float()  # (the weight file holds bfloat16)
    for idx, (s, n) in enumerate(lens.items()):
        q, k, v, _, _, _ = talking_case(H, G, D, V, n, 300 + idx, window)
        seqs[s] = tuple(t.to(dtype).float() for t in (q, k, v))
        qd, kd, vd = (t.double() for t in seqs[s])
        want[s] = plain.mixed_head_attention(qd, kd, vd, 0.3, window, r1.double(), r2.double(), talk.double())
    steps = [
        [("c", 0, 1), ("a", 0, 40), ("b", 0, 2)],               # a first token alone, a portion, a two-token portion
        [("a", 40, 1), ("b", 2, 1)],                            # single tokens only
        [("b", 3, 1), ("a", 41, 17), ("d", 0, 33)],             # mixed; tiles with ragged ends
        [("a", 58, 1), ("d", 33, 1), ("b", 4, 33)],
        [("d", 34, 36), ("a", 59, 91)],                         # portions only, far into their sequences
    ]
    for nsplit in (1, 3):  # (single tokens' keys in one workgroup, or shared among three)
        got = run_talking_mfma(ops, seqs, steps, H, G, D, V, r1, r2, talk, window, 0.3, page_size, nsplit=nsplit)
        for s, n in lens.items():
            close(got[s], want[s].reshape(n, H * V), dtype, f"sequence {s}, {nsplit} shares", tol=2e-2)


@pytest.mark.parametrize("cuts", ["whole", "decode"])
def test_the_window_ends_where_it_should_on_the_matrix_units(ops, cuts):
    H, G, D, V, page_size, n = 2, 1, 16, 16, 16, 300
    for target, window in [(15, 16), (16, 33), (63, 64), (64, 65), (3, 290), (130, 141), (200, 1), (31, 32), (32, 1)]:
        g = torch.Generator().manual_seed(target)
        q = torch.randn(n, H, D, generator=g) * 0.1
        k = torch.randn(n, G, D, generator=g) * 0.1
        v = torch.randn(n, G, V, generator=g) * 0.01
        q[:, :, 0] = 6.0
        k[target, 0, 0] = 6.0
        v[target, 0, 0] = 100.0
        r1, r2 = torch.tensor([0.5, 0.0]), torch.tensor([1.0, 3.0])
        talk = torch.tensor([[1.0, 0.0], [0.25, 0.75]])
        steps = [[("s", 0, n)]] if cuts == "whole" else [[("s", 0, target + 1)]] + [[("s", t, 1)] for t in range(target + 1, n)]
        got = run_talking_mfma(ops, {"s": (q, k, v)}, steps, H, G, D, V, r1, r2, talk, window, 1.0, page_size,
                               nsplit=1 if cuts == "whole" else 4)["s"].float().cpu()
        seen = got[:, 0].abs() > 30.0
        want = torch.zeros(n, dtype=torch.bool)
        want[target:min(n, target + window)] = True
        assert torch.equal(seen, want), f"target {target} window {window}: seen at {seen.nonzero().flatten().tolist()[:8]}.."


@pytest.mark.parametrize("n, width, ff, experts, top, shared", [(4, 64, 24, 5, 2, True), (7, 104, 32, 4, 4, False),
                                                                (40, 128, 64, 8, 1, True), (130, 72, 40, 9, 3, False),
                                                                (300, 256, 96, 6, 2, True), (33, 64, 8, 70, 6, False),
                                                                (200, 104, 72, 3, 2, False), (1, 64, 24, 5, 2, True),
                                                                (520, 152, 200, 2, 2, True)])
def test_experts_products_per_expert_on_the_matrix_units(ops, n, width, ff, experts, top, shared):
    dtype = torch.bfloat16
    assert ops.moe_grouped(n, width, ff, dtype)
    torch.manual_seed(n + width)
    x = torch.randn(n, width).to(dtype)
    wg, wu = (torch.randn(experts, ff, width) * width**-0.5).to(dtype), (torch.randn(experts, ff, width) * width**-0.5).to(dtype)
    wd = (torch.randn(experts, width, ff) * ff**-0.5).to(dtype)
    chosen = torch.stack([torch.randperm(experts)[:top] for _ in range(n)]).to(torch.int32)
    chosen[: n // 3] = torch.arange(top, dtype=torch.int32)  # many tokens on the same experts: lists longer than a tile
    weights = torch.rand(n, top)
    weights = weights / weights.sum(dim=-1, keepdim=True)
    add = torch.randn(n, width).to(dtype) if shared else None
    outs = []
    for grouped in (False, True):
        act = torch.full((n * top, ff), float("nan"), dtype=dtype, device="cuda")
        out = torch.empty(n, width, dtype=dtype, device="cuda")
        scratch = torch.empty(ops.moe_grouped_scratch_bytes(n, width, experts, top), dtype=torch.uint8, device="cuda") \
            if grouped else None
        ops.moe_experts(dev(x), dev(chosen), dev(weights), dev(wg), dev(wu), dev(wd), act, out, "silu",
                        add=None if add is None else dev(add), scratch=scratch)
        outs.append(out.float().cpu())
    want = torch.zeros(n, width, dtype=torch.float64) if add is None else add.double().clone()
    xd = x.double()
    for t in range(n):
        for j in range(top):
            e = int(chosen[t, j])
            hidden = (plain.silu(wg[e].double() @ xd[t]) * (wu[e].double() @ xd[t])).to(dtype).double()
            want[t] += weights[t, j].double() * (wd[e].double() @ hidden)
    close(outs[1], want, dtype, "per expert", tol=2e-2)
    close(outs[1], outs[0], dtype, "against the pair-by-pair kernel", tol=2e-2)
