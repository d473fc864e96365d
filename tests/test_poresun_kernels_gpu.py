"""The kernels and options that the Poresun decoder brought, each alone against a plain
computation (tests/plain/poresun.py): the normed sum around the stream in every form of the
kernel; the gate's activations with a limit; the cache write with normed queries and keys,
with and without weights, and for rows that bring queries alone; attention with a bias
table by distance in the general kernel and on the matrix units, whole, in portions and in
single tokens, with one key made to stand out far back, at page borders and just inside and
just outside a window, and with a table whose rows alone tell distances apart; experts
without gates beside a gated shared expert."""

import math

import pytest
import torch

from .plain import poresun as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 2e-5, torch.bfloat16: 1.6e-2}


@pytest.fixture(scope="module")
def ops():
    from shrike_amd.kernels import ops

    return ops


def dev(t, dtype=None):
    return t.to("cuda", dtype).contiguous() if dtype else t.to("cuda").contiguous()


def i32(x):
    return torch.as_tensor(x, dtype=torch.int32).to("cuda")


def close(got, want, dtype, what=""):
    want = want.double().cpu()
    err = float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= TOL[dtype], f"{what} rel err {err:.3e} > {TOL[dtype]}"


def step_arrays(starts, lens):
    positions = torch.cat([torch.arange(s, s + l) for s, l in zip(starts, lens)])
    token_seq = torch.cat([torch.full((l,), i) for i, l in enumerate(lens)])
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)))
    return i32(positions), i32(token_seq), i32(cu)


def tables_for(ctx_lens, page_size, num_pages, seed=0):
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g).tolist()
    width = max(-(-n // page_size) for n in ctx_lens)
    rows = []
    for n in ctx_lens:
        need = -(-n // page_size)
        rows.append([perm.pop() for _ in range(need)] + [0] * (width - need))
    return torch.tensor(rows, dtype=torch.int32)


# ------------------------------------------------------------------ the normed sum

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n, hidden, splits, scaled", [(5, 64, 0, True), (3, 70, 0, True), (40, 1024, 3, True),
                                                       (2, 4096, 0, False), (7, 9000, 2, True), (1, 5, 1, False)])
def test_normed_sum(ops, dtype, n, hidden, splits, scaled):
    """x <- norm(alpha x + s * delta) * w in the kernel that holds a row in registers (widths in
    fours up to 8192, narrow and wide) and in the one that holds it in LDS; delta a tensor or the
    partial sums of a split product."""
    torch.manual_seed(4)
    alpha, eps = 2.5, 1e-5
    resid = torch.randn(n, hidden) * 3
    weight, ls = torch.rand(hidden) + 0.5, (torch.randn(hidden) if scaled else None)
    if splits:
        parts = torch.randn(splits, n, hidden)
        delta, total = ops.SplitSum(dev(parts)), parts.double().sum(0)
    else:
        d = (torch.randn(n, hidden) * 2).to(dtype)
        delta, total = dev(d), d.double()
    x = alpha * resid.double() + (ls.double() if scaled else 1.0) * total
    want = plain.unit_rms(x, eps) * weight.double()
    got = dev(resid.clone())
    cast = torch.empty(n, hidden, dtype=dtype, device="cuda")
    ops.postnorm(got, delta, alpha, None if ls is None else dev(ls), dev(weight), eps, cast=cast)
    close(got, want, torch.float32, "stream")
    assert torch.equal(cast.cpu(), got.cpu().to(dtype)), "the copy is the stream, rounded once"
    again = dev(resid.clone())
    ops.postnorm(again, delta, alpha, None if ls is None else dev(ls), dev(weight), eps, dtype=dtype)
    assert torch.equal(again, got)


@pytest.mark.parametrize("dtype", DTYPES)
def test_cast_activations_and_gates(ops, dtype):
    torch.manual_seed(5)
    x = (torch.randn(33, 130) * 3).to(dtype)
    out = torch.empty(33, 130, dtype=dtype, device="cuda")
    ops.activate(dev(x), out, "relu_squared")
    close(out, torch.relu(x.double()) ** 2, dtype)
    assert float(out.min()) == 0.0
    ops.activate(dev(x), out, "silu")
    close(out, x.double() * torch.sigmoid(x.double()), dtype)
    g = (torch.randn(33, 130) * 4).to(dtype)
    ops.gate_mul(dev(x), dev(g), out)
    close(out, x.double() * torch.sigmoid(g.double()), dtype)
    src = torch.randn(7, 50)
    ops.cast_rows(dev(src), out[:7, :50].contiguous())
    into = torch.empty(7, 50, dtype=dtype, device="cuda")
    ops.cast_rows(dev(src), into)
    assert torch.equal(into.cpu(), src.to(dtype))
    with pytest.raises(Exception, match="activation"):
        ops.activate(dev(x), out, "tanh")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("limit, shift", [(1.0, 1.0), (0.5, 0.0), (7.0, 1.0), (None, 1.0)])
def test_gate_with_a_limit(ops, dtype, limit, shift):
    """g sigmoid(1.702 g) (u + shift), the gate bounded from above only and the other factor from
    both sides; inputs on both sides of every bound."""
    torch.manual_seed(6)
    gu = (torch.randn(20, 2 * 48) * 3).to(dtype)
    out = torch.empty(20, 48, dtype=dtype, device="cuda")
    ops.act_mul(dev(gu), out, "quick_gelu", limit, shift)
    g, u = gu[:, :48].double(), gu[:, 48:].double()
    if limit:
        assert float(g.max()) > limit and float(u.max()) > limit and float(u.min()) < -limit
        g, u = g.clamp(max=limit), u.clamp(-limit, limit)
    close(out, g * torch.sigmoid(1.702 * g) * (u + shift), dtype)
    w = {"p.gate": torch.eye(48, dtype=torch.float64), "p.up": torch.eye(48, dtype=torch.float64) * 0.5,
         "p.down": torch.eye(48, dtype=torch.float64)}
    if limit and shift == 1.0:  # the plain form's feed-forward on the same numbers
        x = gu[:, :48].double()
        ops.act_mul(dev(torch.cat([x, 0.5 * x], 1).to(dtype)), out, "quick_gelu", limit, shift)
        close(out, plain.dense_ff(x, w, "p", {"limit": limit}), dtype)


@pytest.mark.parametrize("n", [1, 8, 40, 64, 300, 2100])
@pytest.mark.parametrize("limit, shift, activation", [(1.0, 1.0, "quick_gelu"), (None, 1.0, "quick_gelu"), (3.0, 0.0, "silu"),
                                                      (None, 0.0, "relu")])
def test_gated_product_applies_a_gate_with_constants(ops, n, limit, shift, activation):
    """The bfloat16 gate/up product whose epilogue bounds, activates, shifts and multiplies, in each
    of its kernels (few tokens, some dozens, hundreds, thousands), against product-then-activation."""
    torch.manual_seed(11)
    k, ff = 96, 200
    x = (torch.randn(n, k) * 2).to(torch.bfloat16)
    gate, up = (torch.randn(ff, k) * 0.3).to(torch.bfloat16), (torch.randn(ff, k) * 0.3).to(torch.bfloat16)
    wt = ops.interleave_gate_up(dev(gate), dev(up))
    args = None if limit is None and shift == 0.0 else torch.tensor([limit or 0.0, shift], device="cuda")
    out = torch.empty(n, ff, dtype=torch.bfloat16, device="cuda")
    ops.gemm_tiled_weight(dev(x), wt, ff, k, out, gated=activation, gate_args=args)
    g, u = x.double() @ gate.double().T, x.double() @ up.double().T
    if limit:
        assert float(g.max()) > limit and float(u.min()) < -limit
        g, u = g.clamp(max=limit), u.clamp(-limit, limit)
    act = {"quick_gelu": lambda z: z * torch.sigmoid(1.702 * z), "silu": lambda z: z * torch.sigmoid(z), "relu": torch.relu}[activation]
    close(out, act(g) * (u + shift), torch.bfloat16)


# ------------------------------------------------------------------ cache write with normed queries and keys

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page_size, weighted, every",
                         [(6, 2, 40, 72, 16, True, 100), (3, 3, 8, 5, 4, False, 0), (10, 2, 64, 64, 8, True, 1),
                          (2, 2, 128, 32, 16, False, 3)])
def test_cache_write_with_normed_queries_and_keys(ops, dtype, heads, kv_heads, dim, vdim, page_size, weighted, every):
    torch.manual_seed(7)
    eps, coef = 1e-5, 0.6
    starts, lens = [0, 2 * max(every, 1) - 1, 1000], [4, 1, 3]
    ctx = [s + l for s, l in zip(starts, lens)]
    n = sum(lens)
    tables = tables_for(ctx, page_size, 400, seed=dim)
    slab = 32 if dim % 32 == 0 else dim
    k_pool = torch.zeros((400, kv_heads, dim // slab, page_size, slab), dtype=dtype, device="cuda")
    v_pool = torch.zeros((400, kv_heads, vdim, page_size), dtype=dtype, device="cuda")
    qkv = (torch.randn(n, heads * dim + kv_heads * (dim + vdim)) * 3).to(dtype)
    qw = (torch.rand(dim) + 0.5) if weighted else None
    kw = (torch.rand(dim) + 0.5) if weighted else None
    positions, token_seq, _ = step_arrays(starts, lens)
    got = dev(qkv.clone())
    ops.qkv_store(got, heads, kv_heads, dim, vdim, positions, token_seq, dev(tables), k_pool, v_pool, page_size,
                  q_temperature=(coef, every) if every else None, qk_norm_eps=eps,
                  q_weight=None if qw is None else dev(qw), k_weight=None if kw is None else dev(kw))
    pos = positions.cpu().long()
    x = qkv.double()
    q = plain.unit_rms(x[:, : heads * dim].view(n, heads, dim), eps) * (qw.double() if weighted else 1.0)
    if every:
        q = q * plain.query_temperature(pos, coef, every, torch.float64)[:, None, None]
    close(got[:, : heads * dim].view(n, heads, dim), q, dtype, "queries")
    k = plain.unit_rms(x[:, heads * dim : (heads + kv_heads) * dim].view(n, kv_heads, dim), eps) * (kw.double() if weighted else 1.0)
    v = x[:, (heads + kv_heads) * dim :].view(n, kv_heads, vdim)
    for t in range(n):
        page, slot = int(tables[int(token_seq[t]), int(pos[t]) // page_size]), int(pos[t]) % page_size
        close(k_pool[page, :, :, slot, :].reshape(kv_heads, dim), k[t], dtype, "keys")
        assert torch.equal(v_pool[page, :, :, slot].cpu().double(), v[t]), "values are stored as projected"
    # rows that bring queries alone: the same queries, and nothing is written
    alone = dev(qkv[:, : heads * dim].clone())
    before = k_pool.clone()
    ops.qkv_store(alone, heads, kv_heads, dim, vdim, positions, token_seq, dev(tables), k_pool, v_pool, page_size,
                  q_temperature=(coef, every) if every else None, qk_norm_eps=eps,
                  q_weight=None if qw is None else dev(qw), has_kv=False, write_kv=False)
    assert torch.equal(alone, got[:, : heads * dim]) and torch.equal(before, k_pool)


# ------------------------------------------------------------------ attention with a bias by distance

def plain_biased(q, k, v, pos_q, scale, cap, bias_by_distance, window):
    """One head: q [n, d] at positions pos_q over keys/values [ctx, .]; bias_by_distance [ctx]."""
    out = torch.zeros(q.shape[0], v.shape[1], dtype=torch.float64)
    for r, p in enumerate(pos_q):
        lo = 0 if window is None else max(0, p - window + 1)
        s = (k[lo : p + 1] @ q[r]) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        d = p - torch.arange(lo, p + 1)
        s = s + bias_by_distance[d.clamp(max=bias_by_distance.shape[0] - 1)]
        out[r] = torch.softmax(s, 0) @ v[lo : p + 1]
    return out


def fill_pools(keys, values, tables, page_size, kv_heads, dim, vdim, dtype, pages):
    slab = 32 if dim % 32 == 0 else dim
    k_pool = torch.full((pages, kv_heads, dim // slab, page_size, slab), float("nan"), dtype=dtype, device="cuda")
    v_pool = torch.full((pages, kv_heads, vdim, page_size), float("nan"), dtype=dtype, device="cuda")
    for s, (kk, vv) in enumerate(zip(keys, values)):
        for first in range(0, kk.shape[0], page_size):
            page, m = int(tables[s, first // page_size]), min(page_size, kk.shape[0] - first)
            k_pool[page, :, :, :m, :] = kk[first : first + m].to("cuda").view(m, kv_heads, dim // slab, slab).permute(1, 2, 0, 3)
            v_pool[page, :, :, :m] = vv[first : first + m].to("cuda").permute(1, 2, 0)
    # the matrix-unit kernels multiply weights of 0 with what masked slots hold: no NaN there
    return torch.nan_to_num(k_pool, nan=1e4), torch.nan_to_num(v_pool, nan=1e4)


def run_attention(ops, q, heads, kv_heads, dim, vdim, positions, token_seq, cu, tables, ctx, lens, k_pool, v_pool, page_size,
                  window, scale, cap, table, on_matrix_units):
    """All rows through the general kernel, or single tokens through the decode kernel and
    portions through the shared-key kernel (single tokens come first in a step)."""
    n = q.shape[0]
    out = torch.full((n, heads * vdim), float("nan"), dtype=q.dtype, device="cuda")
    if not on_matrix_units:
        ops.attention(q, out, heads, kv_heads, dim, positions, token_seq, tables, k_pool, v_pool, page_size, window, scale,
                      v_dim=vdim, softcap=cap, dist_bias=table)
        return out
    singles = sum(1 for l in lens if l == 1)
    assert all(l == 1 for l in lens[:singles]) and all(l > 1 for l in lens[singles:])
    if singles:
        for nsplit in (1, 3):
            partial = torch.full((singles * heads * nsplit * (dim + 2),), float("nan"), device="cuda")
            ops.attention_decode(q, out, singles, heads, kv_heads, dim, positions, tables, k_pool, v_pool, page_size, window,
                                 scale, partial, nsplit, softcap=cap, dist_bias=table)
    tiles = ops.attention_prefill_shared_tiles(heads, kv_heads, dim)
    wg_seq, wg_q0 = [], []
    for s, l in enumerate(lens):
        if s >= singles:
            for q0 in range(0, l, 16 * tiles):
                wg_seq.append(s), wg_q0.append(q0)
    if wg_seq:
        ops.attention_prefill_shared(q, out, len(wg_seq), heads, kv_heads, dim, cu, i32(ctx), i32(wg_seq), i32(wg_q0), tables,
                                     k_pool, v_pool, page_size, window, scale, first_token=singles, softcap=cap,
                                     dist_bias=table)
    return out


CASES = [
    # heads, kv_heads, dim, vdim, page_size, window, cap, rows, reach
    (6, 2, 40, 72, 16, None, 45.0, 12, 40),
    (3, 3, 32, 32, 8, 37, 4.0, 7, 30),
    (6, 1, 24, 7, 4, 1, None, 2, 3),
    (10, 2, 64, 64, 16, 50, 12.0, 14, 90),
    (6, 2, 64, 64, 16, None, None, 24, 300),
    (4, 4, 128, 128, 32, 300, 30.0, 40, 500),
    (16, 1, 32, 32, 16, 16, 9.0, 9, 25),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page_size, window, cap, rows, reach", CASES)
@pytest.mark.parametrize("matrix_units", [False, True])
def test_attention_with_a_bias_table(ops, dtype, heads, kv_heads, dim, vdim, page_size, window, cap, rows, reach,
                                     matrix_units):
    """Two single tokens and two portions (one of two tokens, one that crosses pages) over up to
    700 keys.  For every sequence's last query one key is made to stand out (a score of 12
    before the cap): far back where there is no window, else the oldest key inside the window, and
    the query before it points as strongly at the first key behind its own window (which must not
    show); the key just behind the last query's window, single tokens included, is a stronger copy of
    the one it may see.  The table's entries
    are several units apart, so that a wrong row shows too."""
    from shrike_amd.parts.attention import distance_buckets

    if matrix_units and not (dtype == torch.bfloat16 and vdim == dim and ops.attention_supports_mfma(
            heads, kv_heads, dim, page_size, heads * dim) and ops.attention_prefill_shared_tiles(heads, kv_heads, dim)):
        pytest.skip("the kernels on the matrix units take bfloat16, values as large as keys and head sizes in 32s")
    torch.manual_seed(8)
    ctx, lens = [700, 333, 2, 420], [1, 1, 2, 39]
    starts = [c - l for c, l in zip(ctx, lens)]
    scale = dim**-0.5
    tables = tables_for(ctx, page_size, 400, seed=dim)
    keys = [torch.randn(c, kv_heads, dim) * 0.3 for c in ctx]
    values = [torch.randn(c, kv_heads, vdim) for c in ctx]
    n = sum(lens)
    q = torch.randn(n, heads, dim) * 0.3
    rel = torch.randn(rows, heads) * 3
    row = 0
    for s, (c, l) in enumerate(zip(ctx, lens)):
        last = row + l - 1
        special = 3 if window is None else c - window  # the last query's oldest visible key
        if window is not None and special >= 1 and c > 2:
            # the key just behind the last query's window would score half as much again: it must not show,
            # for a single token no more than in a portion
            keys[s][special - 1] = 1.5 * keys[s][special]
        if special >= 0 and c > 2:
            for h in range(heads):
                k = keys[s][special, h // (heads // kv_heads)]
                q[last, h] = k / k.norm() ** 2 * 12.0 / scale
                if l > 1 and window is not None and special >= 2:
                    # the query before it: the key just behind its own window, which must not show
                    k = keys[s][special - 2, h // (heads // kv_heads)]
                    q[last - 1, h] = k / k.norm() ** 2 * 12.0 / scale
        row += l
    q, keys, values = q.to(dtype), [k.to(dtype) for k in keys], [v.to(dtype) for v in values]
    k_pool, v_pool = fill_pools(keys, values, tables, page_size, kv_heads, dim, vdim, dtype, 400)
    by_distance = rel[torch.tensor(distance_buckets(rows, reach))]  # [reach + 1, heads], the kernels' form
    check = torch.stack([rel[plain.distance_bucket(d, rows, reach)] for d in range(701)])
    assert torch.equal(check[: reach + 1], by_distance) and torch.equal(check[reach:], by_distance[-1:].expand(701 - reach, -1))
    positions, token_seq, cu = step_arrays(starts, lens)
    out = run_attention(ops, dev(q.reshape(n, heads * dim)), heads, kv_heads, dim, vdim, positions, token_seq, cu, dev(tables),
                        ctx, lens, k_pool, v_pool, page_size, window, scale, cap, dev(by_distance.t()), matrix_units)
    want = torch.zeros(n, heads, vdim, dtype=torch.float64)
    row = 0
    for s, (c, l) in enumerate(zip(ctx, lens)):
        for h in range(heads):
            g = h // (heads // kv_heads)
            want[row : row + l, h] = plain_biased(q[row : row + l, h].double(), keys[s][:, g].double(), values[s][:, g].double(),
                                                  list(range(c - l, c)), scale, cap, check[:, h].double(), window)
        row += l
    close(out.view(n, heads, vdim), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_and_single_tokens_agree(ops, dtype):
    """The same sequence whole, in portions down to two tokens and token by token: float32 the
    same bits in the general kernel; on the matrix units within rounding."""
    torch.manual_seed(9)
    heads, kv_heads, dim, page_size, window, rows, reach = 4, 2, 32, 16, 21, 10, 60
    length = 75
    keys, values = [(torch.randn(length, kv_heads, dim)).to(dtype)], [torch.randn(length, kv_heads, dim).to(dtype)]
    tables = tables_for([length], page_size, 40)
    k_pool, v_pool = fill_pools(keys, values, tables, page_size, kv_heads, dim, dim, dtype, 40)
    from shrike_amd.parts.attention import distance_buckets

    table = dev((torch.randn(rows, heads) * 2)[torch.tensor(distance_buckets(rows, reach))].t())
    q = dev((torch.randn(length, heads * dim)).to(dtype))

    def run(cuts, units):
        rows_out, at = [], 0
        for c in cuts:
            positions, token_seq, cu = step_arrays([at], [c])
            rows_out.append(run_attention(ops, q[at : at + c].contiguous(), heads, kv_heads, dim, dim, positions, token_seq, cu,
                                          dev(tables), [at + c], [c], k_pool, v_pool, page_size, window, dim**-0.5, 6.0, table,
                                          units))
            at += c
        return torch.cat(rows_out)

    whole = run([length], False)
    cuts = [2, 30, 1, 1, 17, 2, 22]
    assert torch.equal(run(cuts, False), whole) and torch.equal(run([1] * length, False), whole)
    if dtype == torch.bfloat16:
        close(run(cuts, True), whole, dtype)
        close(run([1] * length, True), whole, dtype)


# ------------------------------------------------------------------ experts without gates

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n, width, ff, experts, top, shared", [(1, 64, 24, 5, 2, 40), (9, 100, 30, 3, 3, None),
                                                              (70, 128, 96, 8, 3, 96), (300, 64, 16, 4, 1, 8)])
def test_experts_without_gates_and_a_gated_shared_expert(ops, dtype, n, width, ff, experts, top, shared):
    """The square of ReLU through the gated kernels (the one matrix in both places), pair by pair
    and per expert on the matrix units; the shared expert's rows times sigmoid of a column."""
    torch.manual_seed(10)
    x = torch.randn(n, width).to(dtype)
    w_up = (torch.randn(experts, ff, width) * width**-0.5).to(dtype)
    w_down = (torch.randn(experts, width, ff) * ff**-0.5).to(dtype)
    logits = torch.randn(n, experts + 1)
    chosen = torch.empty(n, top, dtype=torch.int32, device="cuda")
    weights = torch.empty(n, top, device="cuda")
    dlogits = dev(logits)
    ops.moe_route(dlogits[:, :experts], None, top, chosen, weights)
    best, index = torch.topk(logits[:, :experts], top, dim=-1)
    assert torch.equal(chosen.cpu().long(), index)
    close(weights, torch.softmax(best.double(), -1), torch.float32, "the softmax over the chosen logits alone")
    add = torch.randn(n, width).to(dtype) if shared else None
    want = torch.zeros(n, width, dtype=torch.float64)
    for t in range(n):
        for k in range(top):
            e = int(index[t, k])
            act = (torch.relu(w_up[e].double() @ x[t].double()) ** 2).to(dtype).double()
            want[t] += float(torch.softmax(best[t].double(), -1)[k]) * (w_down[e].double() @ act)
        if shared:
            want[t] += torch.sigmoid(logits[t, experts].double()) * add[t].double()
    outs = []
    for grouped in (False, True):
        if grouped and not ops.moe_grouped(n, width, ff, dtype):
            continue
        out = torch.empty(n, width, dtype=dtype, device="cuda")
        act_buf = torch.empty(n * top, ff, dtype=dtype, device="cuda")
        scratch = torch.empty(ops.moe_grouped_scratch_bytes(n, width, experts, top), dtype=torch.uint8, device="cuda") if grouped else None
        up = dev(w_up)
        ops.moe_experts(dev(x), chosen, weights, up, up, dev(w_down), act_buf, out, "relu", add=None if add is None else dev(add),
                        scratch=scratch, add_gate=dlogits[:, experts] if shared else None)
        close(out, want, dtype, "grouped" if grouped else "pair by pair")
        outs.append(out)
    assert outs
