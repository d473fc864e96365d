"""Python faces of the HIP launchers: they take torch tensors (used purely as
device allocations), check dtypes and contiguity, and pass raw pointers and
the current HIP stream to libshrike_hip.  Nothing here computes anything."""

from __future__ import annotations

import torch

from .lib import KernelError, check, load

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index: int | None = None


def _stream() -> int:
    """Handle of the current HIP stream (the capture stream while a graph is recorded).
    The engine runs on one GPU: its index is asked for once."""
    global _device_index
    if _device_index is None:
        _device_index = torch.cuda.current_device()
    if _raw_stream is not None:  # a tenth of the cost of building a torch.cuda.Stream object
        return _raw_stream(_device_index)
    return torch.cuda.current_stream().cuda_stream


def current_stream() -> int:
    """Handle of the HIP stream that launches go to now."""
    return _stream()


def _dev(t: torch.Tensor, name: str, dtype=None) -> int:
    if not t.is_cuda:
        raise KernelError(f"{name}: expected a device tensor (there is no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    return t.data_ptr()


def _rows(t: torch.Tensor, name: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{name}: expected a 2-d tensor with unit inner stride")


class SplitSum:
    """The float32 partial sums [splits, n, m] of a product that was split
    along k, with the bias that is still to be added.  Kernels that read the
    product (add_rmsnorm, rope_kv_store) add the parts up in order."""

    __slots__ = ("parts", "bias")

    def __init__(self, parts: torch.Tensor, bias: torch.Tensor | None = None):
        self.parts = parts
        self.bias = bias

    @property
    def shape(self):
        return self.parts.shape[1:]


def _words(t: torch.Tensor, name: str) -> int:
    """Address of an int32 tensor that a kernel may touch: on the device, or page-locked."""
    if t.dtype != torch.int32 or not t.is_contiguous() or not (t.is_cuda or t.is_pinned()):
        raise KernelError(f"{name}: expected a contiguous int32 tensor on the device or in page-locked memory")
    return t.data_ptr()


def copy_words(src: torch.Tensor, dst: torch.Tensor, patch: torch.Tensor | None = None, patch_at: int = 0) -> None:
    """dst[:] = src[:] (int32, equal lengths) by a kernel, with dst[patch_at : patch_at +
    len(patch)] taken from `patch` instead.  Either tensor may be page-locked host memory."""
    n = src.numel()
    if dst.numel() != n:
        raise KernelError("copy_words: src and dst differ in length")
    patch_n = 0 if patch is None else patch.numel()
    if patch_at < 0 or patch_at + patch_n > n:
        raise KernelError("copy_words: the patch does not fit")
    check(load().shk_copy_words(_words(src, "src"), _words(dst, "dst"), n,
                                None if patch is None else _words(patch, "patch"), patch_at, patch_n, _stream()))


def gather_rows(src: torch.Tensor, index: torch.Tensor, dst: torch.Tensor) -> None:
    """dst[r] = src[index[r]] for 2-d tensors of a 4-byte dtype (src rows may be
    strided); index int32, on the device or page-locked, every entry below src's
    row count (the caller's promise: nothing on the device checks it)."""
    _rows(src, "gather_rows src")
    if (dst.dim() != 2 or not dst.is_contiguous() or dst.dtype != src.dtype or src.element_size() != 4
            or dst.shape[1] != src.shape[1] or index.numel() != dst.shape[0]):
        raise KernelError("gather_rows: dst must be contiguous [len(index), width] of src's 4-byte dtype")
    check(load().shk_gather_rows(_dev(src, "src"), src.stride(0), src.shape[0], _words(index, "index"),
                                 _dev(dst, "dst"), dst.shape[0], dst.shape[1], _stream()))


def zero_(t: torch.Tensor) -> None:
    """Fills a contiguous device tensor with zero bytes by a kernel of the library."""
    if not t.is_contiguous():
        raise KernelError("zero_: expected a contiguous tensor")
    check(load().shk_zero_bytes(_dev(t, "t"), t.numel() * t.element_size(), _stream()))


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[i] = float(table[ids[i]]) * scale; ids int32 [n], out float32 [n, hidden]."""
    n, hidden = out.shape
    if not (table.is_contiguous() and out.is_contiguous() and table.shape[1] == hidden):
        raise KernelError("embed: table/out must be contiguous with the same width")
    check(
        load().shk_embed(
            _dev(table, "table"), dtype_code(table.dtype), _dev(ids, "ids", torch.int32),
            _dev(out, "out", torch.float32), n, hidden, table.shape[0], float(scale), _stream(),
        )
    )


def _delta(delta, resid, dtype, who: str):
    """(address, splits) of a product's output that a row kernel adds to `resid`: a
    tensor of the compute dtype, or the partial sums of a SplitSum."""
    if isinstance(delta, SplitSum):
        if delta.bias is not None or tuple(delta.shape) != tuple(resid.shape):
            raise KernelError(f"{who}: partial sums must match resid's shape and carry no bias")
        if delta.parts.dtype != torch.float32 or not delta.parts.is_contiguous():
            raise KernelError(f"{who}: partial sums must be contiguous float32")
        return _dev(delta.parts, "delta"), delta.parts.shape[0]
    if delta.dtype != dtype or not delta.is_contiguous() or delta.shape != resid.shape:
        raise KernelError(f"{who}: a delta must match resid's shape and have the compute dtype")
    return _dev(delta, "delta"), 0


def add_rows(resid, other=None, vec=None) -> None:
    """resid[r] += other[r] + vec (float32; either may be None)."""
    n, hidden = resid.shape
    if not resid.is_contiguous() or (other is not None and (other.shape != resid.shape or not other.is_contiguous())):
        raise KernelError("add_rows: resid and other must be contiguous and of one shape")
    if vec is not None and (vec.numel() != hidden or not vec.is_contiguous()):
        raise KernelError(f"add_rows: vec has {vec.numel()} elements, hidden is {hidden}")
    check(load().shk_add_rows(_dev(resid, "resid", torch.float32),
                              None if other is None else _dev(other, "other", torch.float32),
                              None if vec is None else _dev(vec, "vec", torch.float32), n, hidden, _stream()))


def add_deltas(resid, d1, d2=None, cast=None, dtype=None) -> None:
    """resid += d1 + d2 (outputs of products: tensors of the compute dtype or SplitSums);
    cast, if given, receives the new resid in the compute dtype."""
    n, hidden = resid.shape
    dtype = cast.dtype if cast is not None else dtype
    if dtype is None:
        raise KernelError("add_deltas: give cast or dtype")
    if not resid.is_contiguous() or (cast is not None and (cast.shape != resid.shape or not cast.is_contiguous())):
        raise KernelError("add_deltas: resid and cast must be contiguous and of one shape")
    p1, s1 = _delta(d1, resid, dtype, "add_deltas")
    p2, s2 = (None, 0) if d2 is None else _delta(d2, resid, dtype, "add_deltas")
    check(load().shk_add_deltas(_dev(resid, "resid", torch.float32), p1, s1, p2, s2,
                                None if cast is None else _dev(cast, "cast"), dtype_code(dtype), n, hidden,
                                _stream()))


def add_normed_rmsnorm(resid, delta, dweight, deps: float, weight=None, eps: float = 0.0, out=None,
                       rows=None, write_resid=True, dtype=None) -> None:
    """x = resid + delta * rsqrt(mean(delta^2) + deps) * dweight (per row; stored back with
    write_resid); with `out`, out = x * rsqrt(mean(x^2) + eps) * weight too.  With `rows`
    (int32 [n]) only those rows, into out[0..n)."""
    hidden = resid.shape[1]
    dtype = out.dtype if out is not None else dtype
    if dtype is None:
        raise KernelError("add_normed_rmsnorm: give out or dtype")
    n = resid.shape[0] if rows is None else rows.shape[0]
    if not resid.is_contiguous() or (out is not None and (tuple(out.shape) != (n, hidden) or not out.is_contiguous())):
        raise KernelError("add_normed_rmsnorm: resid/out must be contiguous with the same width")
    if dweight.numel() != hidden or (weight is not None and weight.numel() != hidden):
        raise KernelError(f"add_normed_rmsnorm: weights must have {hidden} elements")
    p, splits = _delta(delta, resid, dtype, "add_normed_rmsnorm")
    check(load().shk_add_normed_rmsnorm(
        _dev(resid, "resid", torch.float32), p, splits, _dev(dweight, "dweight", torch.float32), float(deps),
        None if weight is None else _dev(weight, "weight", torch.float32), float(eps),
        None if out is None else _dev(out, "out"), dtype_code(dtype),
        None if rows is None else _dev(rows, "rows", torch.int32), n, hidden, int(bool(write_resid)),
        resid.shape[0], _stream()))


def act_mul_rows(a, table, ids, offset: int, out, activation: str) -> None:
    """out[r, j] = act(a[r, j]) * table[ids[r], offset + j]: a gate times a slice of the
    table row that the token chooses.  `a` is a tensor of out's dtype or the SplitSum of
    a product split along k."""
    n, width = out.shape
    if not out.is_contiguous():
        raise KernelError("act_mul_rows: out must be contiguous")
    splits = 0
    if isinstance(a, SplitSum):
        if a.bias is not None or tuple(a.shape) != (n, width) or a.parts.dtype != torch.float32 \
                or not a.parts.is_contiguous():
            raise KernelError("act_mul_rows: partial sums must be contiguous float32 [splits, n, width] without a bias")
        splits, a = a.parts.shape[0], a.parts
    elif a.shape != out.shape or not a.is_contiguous() or a.dtype != out.dtype:
        raise KernelError("act_mul_rows: a and out must be contiguous, of one shape and dtype")
    if table.dim() != 2 or not table.is_contiguous() or table.dtype != out.dtype:
        raise KernelError("act_mul_rows: table must be a contiguous matrix of out's dtype")
    if offset < 0 or offset + width > table.shape[1] or ids.shape[0] < n:
        raise KernelError("act_mul_rows: the slice does not fit the table, or too few ids")
    check(load().shk_act_mul_rows(_dev(a, "a"), splits, _dev(table, "table"), dtype_code(out.dtype),
                                  _dev(ids, "ids", torch.int32), table.shape[1], int(offset), table.shape[0],
                                  _dev(out, "out"), n, width, activation_code(activation), _stream()))


def add_rmsnorm(resid, delta, weight, eps: float, out, rows=None, write_resid=True) -> None:
    """resid (+= delta); out = rmsnorm(resid) * weight.  With `rows` (int32 [n])
    only those rows are normed, into out[0..n)."""
    n, hidden = out.shape
    if not (resid.is_contiguous() and out.is_contiguous() and resid.shape[1] == hidden):
        raise KernelError("add_rmsnorm: resid/out must be contiguous with the same width")
    splits = 0
    if isinstance(delta, SplitSum):
        if delta.bias is not None or tuple(delta.shape) != tuple(resid.shape):
            raise KernelError("add_rmsnorm: partial sums must match resid's shape and carry no bias")
        splits, delta = delta.parts.shape[0], delta.parts
        if delta.dtype != torch.float32 or not delta.is_contiguous():
            raise KernelError("add_rmsnorm: partial sums must be contiguous float32")
    elif delta is not None and (
        delta.dtype != out.dtype or not delta.is_contiguous() or delta.shape != resid.shape
    ):
        raise KernelError("add_rmsnorm: delta must match resid's shape and out's dtype")
    if weight.numel() != hidden:
        raise KernelError(f"add_rmsnorm: weight has {weight.numel()} elements, hidden is {hidden}")
    if rows is None and resid.shape[0] != n:
        raise KernelError("add_rmsnorm: out and resid differ in rows")
    check(
        load().shk_add_rmsnorm(
            _dev(resid, "resid", torch.float32),
            None if delta is None else _dev(delta, "delta"),
            _dev(weight, "weight", torch.float32), float(eps), _dev(out, "out"),
            dtype_code(out.dtype), None if rows is None else _dev(rows, "rows", torch.int32),
            n, hidden, int(bool(write_resid)), splits, resid.shape[0], _stream(),
        )
    )


# a gate's activation: SiLU, GELU in its tanh form, ReLU, g * sigmoid(1.702 g); the products with a fused
# activation, the experts' kernels and act_mul each say which of them they take
GATE_ACTIVATIONS = {"silu": 1, "gelu_tanh": 2, "relu": 3, "quick_gelu": 4}
# an activation of a plain product (activate): the above without a second factor, and the square of ReLU
PLAIN_ACTIVATIONS = {"silu": 1, "gelu_tanh": 2, "relu": 3, "relu_squared": 4}


def activation_code(gated) -> int:
    """0 for a product that is not gated; else the code of the gate's activation
    (True stands for "silu")."""
    if not gated:
        return 0
    name = "silu" if gated is True else gated
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise KernelError(f"gate activation must be one of {sorted(GATE_ACTIVATIONS)}, got {gated!r}") from None


def act_mul(gate_up: torch.Tensor, out: torch.Tensor, activation: str = "silu", limit: float | None = None,
            up_shift: float = 0.0) -> None:
    """out = act(g) * (u + up_shift) with g = gate_up[:, :I], u = gate_up[:, I:]; with `limit`,
    g <- min(g, limit) and u <- clamp(u, -limit, limit) first."""
    n, inter = out.shape
    if gate_up.shape != (n, 2 * inter) or not gate_up.is_contiguous() or not out.is_contiguous():
        raise KernelError("act_mul: gate_up must be contiguous [n, 2*inter]")
    if gate_up.dtype != out.dtype:
        raise KernelError("act_mul: dtypes differ")
    check(load().shk_act_mul(_dev(gate_up, "gate_up"), _dev(out, "out"), dtype_code(out.dtype),
                             n, inter, activation_code(activation), float(limit or 0.0), float(up_shift), _stream()))


def postnorm(resid, delta, alpha: float, lscale, weight, eps: float, cast=None, dtype=None) -> None:
    """resid <- rmsnorm(alpha * resid + lscale * delta) * weight, row by row in float32 (lscale float32
    [hidden] or None: ones; delta a tensor of the compute dtype, a SplitSum, or None: nothing is
    added); `cast`, if given, receives the new rows in the compute dtype."""
    n, hidden = resid.shape
    dtype = cast.dtype if cast is not None else dtype
    if dtype is None:
        raise KernelError("postnorm: give cast or dtype")
    if not resid.is_contiguous() or (cast is not None and (cast.shape != resid.shape or not cast.is_contiguous())):
        raise KernelError("postnorm: resid and cast must be contiguous and of one shape")
    if weight.numel() != hidden or (lscale is not None and lscale.numel() != hidden):
        raise KernelError(f"postnorm: weight and lscale must have {hidden} elements")
    p, splits = (None, 0) if delta is None else _delta(delta, resid, dtype, "postnorm")
    check(load().shk_postnorm(_dev(resid, "resid", torch.float32), p, splits, float(alpha),
                              None if lscale is None else _dev(lscale, "lscale", torch.float32),
                              _dev(weight, "weight", torch.float32), float(eps),
                              None if cast is None else _dev(cast, "cast"), dtype_code(dtype), n, hidden, _stream()))


def cast_rows(src, dst) -> None:
    """dst = src (float32) in dst's dtype."""
    if src.shape != dst.shape or not src.is_contiguous() or not dst.is_contiguous():
        raise KernelError("cast_rows: src and dst must be contiguous and of one shape")
    check(load().shk_cast_rows(_dev(src, "src", torch.float32), _dev(dst, "dst"), dtype_code(dst.dtype), src.numel(),
                               _stream()))


def activate(x, out, activation: str) -> None:
    """out = act(x) elementwise, act one of PLAIN_ACTIVATIONS."""
    if x.shape != out.shape or x.dtype != out.dtype or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError("activate: x and out must be contiguous and alike")
    if activation not in PLAIN_ACTIVATIONS:
        raise KernelError(f"activate: activation must be one of {sorted(PLAIN_ACTIVATIONS)}, got {activation!r}")
    check(load().shk_activate(_dev(x, "x"), _dev(out, "out"), dtype_code(x.dtype), x.numel(),
                              PLAIN_ACTIVATIONS[activation], _stream()))


def gate_mul(x, gate, out) -> None:
    """out = x * sigmoid(gate) elementwise."""
    if x.shape != out.shape or gate.shape != x.shape or x.dtype != out.dtype or gate.dtype != x.dtype \
            or not (x.is_contiguous() and gate.is_contiguous() and out.is_contiguous()):
        raise KernelError("gate_mul: x, gate and out must be contiguous and alike")
    check(load().shk_gate_mul(_dev(x, "x"), _dev(gate, "gate"), _dev(out, "out"), dtype_code(x.dtype), x.numel(),
                              _stream()))


def gemm(a, w, out, bias=None, accumulate=False) -> None:
    """out (+)= a @ w.T + bias;  a [n, k], w [m, k] contiguous, out [n, m]."""
    _rows(a, "gemm a")
    _rows(out, "gemm out")
    n, k = a.shape
    m = w.shape[0]
    if w.dim() != 2 or w.shape[1] != k or not w.is_contiguous():
        raise KernelError(f"gemm: w must be contiguous [m, {k}], got {tuple(w.shape)}")
    if out.shape != (n, m):
        raise KernelError(f"gemm: out must be [{n}, {m}], got {tuple(out.shape)}")
    if a.dtype != w.dtype:
        raise KernelError(f"gemm: a is {a.dtype} but w is {w.dtype}")
    if bias is not None and bias.numel() != m:
        raise KernelError(f"gemm: bias has {bias.numel()} elements, m is {m}")
    check(
        load().shk_gemm(
            _dev(a, "a"), _dev(w, "w"),
            None if bias is None else _dev(bias, "bias", torch.float32),
            _dev(out, "out"), n, m, k, a.stride(0), out.stride(0),
            dtype_code(a.dtype), dtype_code(out.dtype), int(bool(accumulate)), _stream(),
        )
    )


def tiled_numel(m: int, k: int) -> int:
    """bfloat16 elements of the tiled layout of an [m, k] matrix."""
    return -(-m // 16) * -(-k // 32) * 512


def retile_weight(w: torch.Tensor) -> torch.Tensor:
    """The MFMA operand layout of a row-major bfloat16 [m, k] matrix (a flat tensor)."""
    if w.dim() != 2 or not w.is_contiguous() or w.dtype != torch.bfloat16:
        raise KernelError("retile_weight: expected a contiguous bfloat16 matrix")
    m, k = w.shape
    wt = torch.empty(tiled_numel(m, k), dtype=torch.bfloat16, device=w.device)
    check(load().shk_retile_weight(_dev(w, "w"), m, k, _dev(wt, "wt"), _stream()))
    return wt


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The tiled layouts of two row-major [m, k] matrices interleaved by blocks of
    16 rows, for the gated product of gemm_tiled_weight."""
    if gate.shape != up.shape:
        raise KernelError("interleave_gate_up: gate and up differ in shape")
    m, k = gate.shape
    gt, ut = retile_weight(gate), retile_weight(up)
    wt = torch.empty(2 * tiled_numel(m, k), dtype=torch.bfloat16, device=gate.device)
    check(load().shk_interleave_gate_up(_dev(gt, "gate"), _dev(ut, "up"), m, k, _dev(wt, "wt"),
                                        _stream()))
    return wt


def gemm_splits(n: int, m: int, k: int) -> int:
    """Shares of k that fill the chip for an [n, k] x [m, k]^T product (1: do not split)."""
    return int(load().shk_gemm_bf16_splits(n, m, k))


def gemm_parts(n: int, m: int, k: int, gated: bool = False) -> int:
    """Launches that an [n, k] x [m, k]^T product is made of (2: rows whose tiles
    fill whole rounds of the compute units, then the rest)."""
    return int(load().shk_gemm_bf16_parts(n, m, k, int(gated)))


def mfma_alone(operands: torch.Tensor, workgroups: int, iters: int) -> float:
    """Runs the bfloat16 matrix instruction by itself on `operands` (at least
    32,768 bfloat16 values, held in registers) and returns the flop it did:
    for measuring what the matrix units give on operands of a given kind."""
    if operands.dtype != torch.bfloat16 or operands.numel() < 32768 or not operands.is_contiguous():
        raise KernelError("mfma_alone: operands must be 32,768 contiguous bfloat16 values or more")
    out = torch.empty(workgroups * 256, dtype=torch.float32, device=operands.device)
    check(load().shk_mfma_alone(_dev(operands, "operands"), _dev(out, "out", torch.float32), workgroups, iters,
                                _stream()))
    return 2.0 * 64 * 64 * 32 * 4 * workgroups * iters


def gemm_tiled_weight(a, wt, m: int, k: int, out, bias=None, accumulate=False, gated=False,
                      splits: int = 1, gate_args=None) -> None:
    """out (+)= a @ w.T + bias with wt = retile_weight(w): up to 64 rows of a
    stream the weights once; more rows run the LDS-staged MFMA kernel (tiles of
    128 x 128 to 256 x 256, chosen by how many the product has).
    splits > 1: out is float32 [splits, n, m] and receives partial sums.
    gated: False, or the gate's activation (one of GATE_ACTIVATIONS; True is "silu") for
    an interleaved gate/up weight.  gate_args: float32 [2] on the device, (limit, up_shift) of
    such a gate: act(min(g, limit)) * (clamp(u, -limit, limit) + up_shift), limit 0: no bounds."""
    _rows(a, "gemm a")
    n = a.shape[0]
    if a.shape[1] != k or a.dtype != torch.bfloat16:
        raise KernelError(f"gemm_tiled_weight: a must be bfloat16 [n, {k}], got {tuple(a.shape)}")
    if splits > 1:
        if tuple(out.shape) != (splits, n, m) or not out.is_contiguous() or out.dtype != torch.float32:
            raise KernelError(f"gemm_tiled_weight: partial sums must be contiguous float32 [{splits}, {n}, {m}]")
    else:
        _rows(out, "gemm out")
        if out.shape != (n, m):
            raise KernelError(f"gemm_tiled_weight: out must be [{n}, {m}], got {tuple(out.shape)}")
    if wt.numel() != (2 if gated else 1) * tiled_numel(m, k) or wt.dtype != torch.bfloat16:
        raise KernelError("gemm_tiled_weight: wt is not the tiled layout of an [m, k] matrix")
    if bias is not None and bias.numel() != m:
        raise KernelError(f"gemm_tiled_weight: bias has {bias.numel()} elements, m is {m}")
    if gate_args is not None:
        if not gated or bias is not None or gate_args.numel() != 2 or gate_args.dtype != torch.float32:
            raise KernelError("gemm_tiled_weight: gate_args are two float32 numbers of a gated product without bias")
        bias = gate_args  # (they travel in the bias's place)
    check(
        load().shk_gemm_bf16_tiled_weight(
            _dev(a, "a"), _dev(wt, "wt"),
            None if bias is None else _dev(bias, "bias", torch.float32),
            _dev(out, "out"), n, m, k, a.stride(0), out.stride(-2), dtype_code(out.dtype),
            int(bool(accumulate)), activation_code(gated), int(splits), _stream(),
        )
    )


def key_slab(head_dim: int) -> int:
    """Elements per slab of the cached keys: 32, or the whole row where head_dim
    is no multiple of 32 (csrc/common.h: key_slab)."""
    return 32 if head_dim % 32 == 0 else head_dim


def key_pool_shape(pages: int, kv_heads: int, page_size: int, head_dim: int) -> tuple:
    """Keys of a page and head lie in slabs: [pages, kv_heads, head_dim / slab, page_size, slab]."""
    slab = key_slab(head_dim)
    return (pages, kv_heads, head_dim // slab, page_size, slab)


def _check_pools(who, q, tables, k_pool, v_pool, kv_heads, head_dim, page_size, v_dim=None) -> None:
    """Keys in slabs (key_pool_shape); values transposed [pages, kv_heads, v_dim, page_size]
    (v_dim None: values as large as keys)."""
    pages = k_pool.shape[0]
    key_dim, head_dim = head_dim, (head_dim if v_dim is None else v_dim)
    if tuple(k_pool.shape) != key_pool_shape(pages, kv_heads, page_size, key_dim):
        raise KernelError(f"{who}: key pool must be {list(key_pool_shape('pages', kv_heads, page_size, key_dim))}, "
                          f"got {tuple(k_pool.shape)}")
    if tuple(v_pool.shape) != (pages, kv_heads, head_dim, page_size):
        raise KernelError(f"{who}: value pool must be [pages, {kv_heads}, {head_dim}, {page_size}], "
                          f"got {tuple(v_pool.shape)}")
    if k_pool.dtype != q.dtype or v_pool.dtype != q.dtype:
        raise KernelError(f"{who}: pools and queries differ in dtype")
    if not (k_pool.is_contiguous() and v_pool.is_contiguous() and tables.is_contiguous()):
        raise KernelError(f"{who}: pools and tables must be contiguous")
    if tables.dim() != 2:
        raise KernelError(f"{who}: tables must be [sequences, blocks]")


def rope_kv_store(qkv, heads, kv_heads, head_dim, rot_dim, inv_freq, positions, token_seq,
                  tables, k_pool, v_pool, page_size, write_kv=True, split_sum=None,
                  adjacent_pairs: bool = False, values_from_keys: bool = False) -> None:
    """Rotate q and k of qkv [n, (heads + 2 kv_heads) head_dim] in float32 and put
    k, v into their pages (keys in slabs, see key_pool_shape; values transposed
    [pages, kv_heads, head_dim, page_size]).  adjacent_pairs: element 2i turns with
    2i + 1 instead of i with i + rot_dim / 2.  values_from_keys: qkv has no value
    columns, [n, (heads + kv_heads) head_dim], and a token's values are its keys as
    they come in (before the rotation)."""
    n = qkv.shape[0]
    if not qkv.is_contiguous() or qkv.shape[1] != (heads + (1 if values_from_keys else 2) * kv_heads) * head_dim:
        raise KernelError("rope_kv_store: qkv must be contiguous [n, (heads + 2 kv_heads) head_dim] "
                          "(heads + kv_heads with values_from_keys)")
    # the kernel reads one position (and one sequence index) per row of qkv
    if positions.shape[0] < n or (write_kv and token_seq.shape[0] < n):
        raise KernelError(f"rope_kv_store: qkv has {n} rows but positions / token_seq are shorter")
    parts, splits, bias = None, 0, None
    if split_sum is not None:
        parts, bias = split_sum.parts, split_sum.bias
        splits = parts.shape[0]
        if tuple(parts.shape[1:]) != tuple(qkv.shape) or parts.dtype != torch.float32 or not parts.is_contiguous():
            raise KernelError("rope_kv_store: partial sums must be contiguous float32 [splits, n, width]")
    num_pages = 0
    if write_kv:
        _check_pools("rope_kv_store", qkv, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
        num_pages = k_pool.shape[0]
    check(
        load().shk_rope_kv_store(
            _dev(qkv, "qkv"), dtype_code(qkv.dtype), n, heads, kv_heads, head_dim, rot_dim,
            None if inv_freq is None else _dev(inv_freq, "inv_freq", torch.float32),
            _dev(positions, "positions", torch.int32),
            _dev(token_seq, "token_seq", torch.int32) if write_kv else None,
            _dev(tables, "tables", torch.int32) if write_kv else None,
            tables.shape[1] if write_kv else 0,
            _dev(k_pool, "k_pool") if write_kv else None,
            _dev(v_pool, "v_pool") if write_kv else None,
            page_size, num_pages, int(bool(write_kv)),
            None if parts is None else _dev(parts, "parts", torch.float32), splits,
            None if bias is None else _dev(bias, "bias", torch.float32),
            int(bool(adjacent_pairs)), int(bool(values_from_keys)), _stream(),
        )
    )


def attention(q, out, heads, kv_heads, head_dim, positions, token_seq, tables, k_pool, v_pool,
              page_size, window, scale, chunk=None, v_dim=None, softcap=None, sinks=None, dist_bias=None) -> None:
    """q: [n, >= heads*head_dim] rows (a view into qkv is fine); out [n, heads*v_dim].
    v_dim: size of a value (None: head_dim); softcap: scores become cap * tanh(score / cap);
    sinks: float32 [heads], one more term exp(sinks[h]) in each head's softmax denominator;
    dist_bias: float32 [heads, rows], dist_bias[h, min(i - j, rows - 1)] joins the (capped) score."""
    _rows(q, "attention q")
    n = q.shape[0]
    v_dim = head_dim if v_dim is None else int(v_dim)
    if out.shape != (n, heads * v_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("attention: out must be contiguous [n, heads*v_dim] of q's dtype")
    if sinks is not None and (sinks.numel() != heads or not sinks.is_contiguous()):
        raise KernelError(f"attention: sinks must hold one value per head ({heads})")
    _dist_bias(dist_bias, heads, "attention")
    _check_pools("attention", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size, v_dim)
    check(
        load().shk_attention(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), dtype_code(q.dtype), n, heads, kv_heads,
            head_dim, _dev(positions, "positions", torch.int32),
            _dev(token_seq, "token_seq", torch.int32), _dev(tables, "tables", torch.int32),
            tables.shape[1], tables.shape[0], _dev(k_pool, "k_pool"), _dev(v_pool, "v_pool"),
            page_size, k_pool.shape[0], int(window or 0), int(chunk or 0), float(scale), v_dim,
            float(softcap or 0.0), None if sinks is None else _dev(sinks, "sinks", torch.float32),
            None if dist_bias is None else _dev(dist_bias, "dist_bias", torch.float32),
            0 if dist_bias is None else dist_bias.shape[1], _stream(),
        )
    )


def _dist_bias_args(dist_bias, heads, who):
    """(address, rows) of a distance bias for a launcher; (None, 0) without one."""
    _dist_bias(dist_bias, heads, who)
    return (None, 0) if dist_bias is None else (_dev(dist_bias, "dist_bias", torch.float32), dist_bias.shape[1])


def _dist_bias(dist_bias, heads, who):
    if dist_bias is not None and (dist_bias.dim() != 2 or dist_bias.shape[0] != heads or dist_bias.shape[1] < 1
                                  or not dist_bias.is_contiguous() or dist_bias.dtype != torch.float32):
        raise KernelError(f"{who}: a distance bias must be contiguous float32 [heads ({heads}), rows]")


def qkv_store(qkv, heads, kv_heads, head_dim, v_dim, positions, token_seq, tables, k_pool, v_pool, page_size,
              q_temperature=None, v_norm_eps=None, write_kv=True, qk_norm_eps=None, q_weight=None, k_weight=None,
              has_kv=True) -> None:
    """Cache write without rotation for keys of head_dim and values of v_dim: qkv is [n, heads *
    head_dim + kv_heads * (head_dim + v_dim)].  q_temperature = (coef, every): the queries at
    position p are multiplied by 1 + coef * ln(floor((p + 1) / every) + 1) in place.
    v_norm_eps: each head's value is stored divided by sqrt(mean(v^2) + eps).
    qk_norm_eps: every head of the queries (in place, before the temperature) and of the keys is
    divided by sqrt(mean(x^2) + eps) and multiplied by q_weight / k_weight (float32 [head_dim], or
    None).  has_kv False: qkv is [n, heads * head_dim], queries alone; nothing is written."""
    n = qkv.shape[0]
    write_kv = bool(write_kv and has_kv)
    width = heads * head_dim + (kv_heads * (head_dim + v_dim) if has_kv else 0)
    if not qkv.is_contiguous() or qkv.shape[1] != width:
        raise KernelError("qkv_store: qkv must be contiguous [n, heads*head_dim + kv_heads*(head_dim + v_dim)] "
                          "(queries alone without has_kv)")
    for w in (q_weight, k_weight):
        if w is not None and (qk_norm_eps is None or w.numel() != head_dim or w.dtype != torch.float32
                              or not w.is_contiguous()):
            raise KernelError("qkv_store: norm weights are float32 [head_dim] and need qk_norm_eps")
    if positions.shape[0] < n or (write_kv and token_seq.shape[0] < n):
        raise KernelError(f"qkv_store: qkv has {n} rows but positions / token_seq are shorter")
    num_pages = 0
    if write_kv:
        _check_pools("qkv_store", qkv, tables, k_pool, v_pool, kv_heads, head_dim, page_size, v_dim)
        num_pages = k_pool.shape[0]
    coef, every = (0.0, 0) if q_temperature is None else (float(q_temperature[0]), int(q_temperature[1]))
    if q_temperature is not None and every < 1:
        raise KernelError(f"qkv_store: the query temperature's step must be positive, got {every}")
    check(load().shk_qkv_store(
        _dev(qkv, "qkv"), dtype_code(qkv.dtype), n, heads, kv_heads, head_dim, v_dim, coef, every,
        float(v_norm_eps or 0.0), float(qk_norm_eps or 0.0),
        None if q_weight is None else _dev(q_weight, "q_weight"), None if k_weight is None else _dev(k_weight, "k_weight"),
        int(bool(has_kv)), _dev(positions, "positions", torch.int32),
        _dev(token_seq, "token_seq", torch.int32) if write_kv else None,
        _dev(tables, "tables", torch.int32) if write_kv else None, tables.shape[1] if write_kv else 0,
        _dev(k_pool, "k_pool") if write_kv else None, _dev(v_pool, "v_pool") if write_kv else None,
        page_size, num_pages, int(bool(write_kv)), _stream()))


def latent_prepare(down, q_rank, kv_rank, rot_dim, q_weight, kv_weight, eps, inv_freq, positions, token_seq,
                   tables, q_latent, pool, page_size, write_kv=True) -> None:
    """From a token's joint down-projection [q latent | key/value latent | rotated key part]:
    the normed query latent into q_latent [n, q_rank]; the normed key/value latent and the
    rotated key part (neighbouring pairs) into the token's row of pool [pages, page_size,
    kv_rank + rot_dim]."""
    n = down.shape[0]
    if not down.is_contiguous() or down.shape[1] != q_rank + kv_rank + rot_dim:
        raise KernelError("latent_prepare: down must be contiguous [n, q_rank + kv_rank + rot_dim]")
    if tuple(q_latent.shape) != (n, q_rank) or not q_latent.is_contiguous() or q_latent.dtype != down.dtype:
        raise KernelError("latent_prepare: q_latent must be contiguous [n, q_rank] of down's dtype")
    if q_weight.numel() != q_rank or kv_weight.numel() != kv_rank:
        raise KernelError("latent_prepare: the norms' weights do not fit the latents")
    if rot_dim and (inv_freq is None or inv_freq.numel() < rot_dim // 2):
        raise KernelError("latent_prepare: too few rotation rates")
    if positions.shape[0] < n or (write_kv and token_seq.shape[0] < n):
        raise KernelError(f"latent_prepare: down has {n} rows but positions / token_seq are shorter")
    num_pages = 0
    if write_kv:
        if (pool.dim() != 3 or tuple(pool.shape[1:]) != (page_size, kv_rank + rot_dim) or not pool.is_contiguous()
                or pool.dtype != down.dtype or tables.dim() != 2 or not tables.is_contiguous()):
            raise KernelError(f"latent_prepare: the pool must be contiguous [pages, {page_size}, {kv_rank + rot_dim}] "
                              "of down's dtype, the tables [sequences, blocks]")
        num_pages = pool.shape[0]
    check(load().shk_latent_prepare(
        _dev(down, "down"), dtype_code(down.dtype), n, q_rank, kv_rank, rot_dim,
        _dev(q_weight, "q_weight", torch.float32), _dev(kv_weight, "kv_weight", torch.float32), float(eps),
        None if inv_freq is None else _dev(inv_freq, "inv_freq", torch.float32),
        _dev(positions, "positions", torch.int32),
        _dev(token_seq, "token_seq", torch.int32) if write_kv else None,
        _dev(tables, "tables", torch.int32) if write_kv else None, tables.shape[1] if write_kv else 0,
        _dev(q_latent, "q_latent"), _dev(pool, "pool") if write_kv else None, page_size, num_pages,
        int(bool(write_kv)), _stream()))


def rotate_heads(src, src_head, src_off, dst, dst_head, dst_off, heads, rot_dim, inv_freq, positions) -> None:
    """dst[t, h*dst_head + dst_off + e] = rotation of src[t, h*src_head + src_off + e] for e < rot_dim:
    neighbouring pairs (2i, 2i + 1) turned by positions[t] * inv_freq[i]."""
    _rows(src, "rotate_heads src")
    _rows(dst, "rotate_heads dst")
    n = src.shape[0]
    if dst.shape[0] != n or src.dtype != dst.dtype or positions.shape[0] < n:
        raise KernelError("rotate_heads: src, dst and positions differ in rows or dtype")
    if src.shape[1] < heads * src_head or dst.shape[1] < heads * dst_head:
        raise KernelError("rotate_heads: the rows are shorter than heads * head size")
    if rot_dim and (inv_freq is None or inv_freq.numel() < rot_dim // 2):
        raise KernelError("rotate_heads: too few rotation rates")
    check(load().shk_rotate_heads(
        _dev(src, "src"), src.stride(0), src_head, src_off, _dev(dst, "dst"), dst.stride(0), dst_head, dst_off,
        dtype_code(src.dtype), n, heads, rot_dim,
        None if inv_freq is None else _dev(inv_freq, "inv_freq", torch.float32),
        _dev(positions, "positions", torch.int32), _stream()))


def latent_attention(q, out, heads, key_dim, v_dim, positions, token_seq, tables, pool, page_size, window,
                     scale, chunk=None) -> None:
    """q [n, heads * key_dim], out [n, heads * v_dim]; pool [pages, page_size, key_dim]: a row is a
    key, its first v_dim elements the value; every head reads the same rows."""
    n = q.shape[0]
    if tuple(q.shape) != (n, heads * key_dim) or not q.is_contiguous():
        raise KernelError("latent_attention: q must be contiguous [n, heads * key_dim]")
    if tuple(out.shape) != (n, heads * v_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("latent_attention: out must be contiguous [n, heads * v_dim] of q's dtype")
    if (pool.dim() != 3 or tuple(pool.shape[1:]) != (page_size, key_dim) or not pool.is_contiguous()
            or pool.dtype != q.dtype or tables.dim() != 2 or not tables.is_contiguous()):
        raise KernelError(f"latent_attention: the pool must be contiguous [pages, {page_size}, {key_dim}] of q's dtype")
    if positions.shape[0] < n or token_seq.shape[0] < n:
        raise KernelError("latent_attention: positions / token_seq are shorter than q")
    check(load().shk_latent_attention(
        _dev(q, "q"), _dev(out, "out"), dtype_code(q.dtype), n, heads, key_dim, v_dim,
        _dev(positions, "positions", torch.int32), _dev(token_seq, "token_seq", torch.int32),
        _dev(tables, "tables", torch.int32), tables.shape[1], _dev(pool, "pool"), page_size, pool.shape[0],
        int(window or 0), int(chunk or 0), float(scale), _stream()))


def latent_attention_supports_mfma(heads: int, key_dim: int, v_dim: int) -> bool:
    return bool(load().shk_latent_attention_supports_mfma(heads, key_dim, v_dim))


def latent_attention_mfma(q, out, heads, key_dim, v_dim, positions, token_seq, tables, pool, page_size, window,
                          scale, chunk=None, partial=None, nsplit: int = 1, tokens_per_group: int = 1) -> None:
    """latent_attention on the matrix units (bfloat16).  nsplit > 1 shares each token's rows among
    that many workgroups; partial: float32 scratch of n * heads * nsplit * (v_dim + 2).
    tokens_per_group: up to how many neighbouring tokens a workgroup may serve (prompt portions)."""
    n = q.shape[0]
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("latent_attention_mfma: bfloat16 only")
    if tuple(q.shape) != (n, heads * key_dim) or not q.is_contiguous() or tuple(out.shape) != (n, heads * v_dim) \
            or not out.is_contiguous():
        raise KernelError("latent_attention_mfma: q [n, heads * key_dim] and out [n, heads * v_dim], contiguous")
    if (pool.dim() != 3 or tuple(pool.shape[1:]) != (page_size, key_dim) or not pool.is_contiguous()
            or pool.dtype != q.dtype or tables.dim() != 2 or not tables.is_contiguous()):
        raise KernelError(f"latent_attention_mfma: the pool must be contiguous [pages, {page_size}, {key_dim}] bfloat16")
    if positions.shape[0] < n or token_seq.shape[0] < n:
        raise KernelError("latent_attention_mfma: positions / token_seq are shorter than q")
    if nsplit > 1 and (partial is None or partial.dtype != torch.float32
                       or partial.numel() < n * heads * nsplit * (v_dim + 2)):
        raise KernelError("latent_attention_mfma: key splits need a float32 partial buffer of "
                          f"{n * heads * nsplit * (v_dim + 2)} values")
    check(load().shk_latent_attention_bf16(
        _dev(q, "q"), _dev(out, "out"), n, heads, key_dim, v_dim, _dev(positions, "positions", torch.int32),
        _dev(token_seq, "token_seq", torch.int32), _dev(tables, "tables", torch.int32), tables.shape[1],
        _dev(pool, "pool"), page_size, pool.shape[0], int(window or 0), int(chunk or 0), float(scale),
        _dev(partial, "partial", torch.float32) if nsplit > 1 else None, int(nsplit), int(tokens_per_group),
        _stream()))


def gemm_batched(a, w, out, batch: int, a_step: int, out_step: int) -> None:
    """out[:, b*out_step : b*out_step + m] = a[:, b*a_step : b*a_step + k] @ w[b].T for b < batch;
    w [batch, m, k] contiguous; a and out 2-d with unit inner stride; all of one dtype."""
    _rows(a, "gemm_batched a")
    _rows(out, "gemm_batched out")
    n = a.shape[0]
    if w.dim() != 3 or w.shape[0] != batch or not w.is_contiguous() or w.dtype != a.dtype or out.dtype != a.dtype:
        raise KernelError("gemm_batched: w must be contiguous [batch, m, k] of a's dtype, as out is")
    m, k = w.shape[1], w.shape[2]
    if out.shape[0] != n or (batch - 1) * a_step + k > a.shape[1] or (batch - 1) * out_step + m > out.shape[1] \
            or out_step < m or a_step < 0:
        raise KernelError("gemm_batched: the batch's slices do not fit a or out")
    check(load().shk_gemm_batched(_dev(a, "a"), _dev(w, "w"), _dev(out, "out"), n, m, k, a.stride(0), out.stride(0),
                                  batch, a_step, m * k, out_step, dtype_code(a.dtype), _stream()))


def mlstm_state_floats(heads: int, dim: int, v_dim: int) -> int:
    """float32 values of one request's state in one mLSTM layer (mlstm_scan's own layout)."""
    return int(load().shk_mlstm_state_floats(heads, dim, v_dim))


def mlstm_scan(proj, q_off, k_off, v_off, i_off, f_off, i_bias, f_bias, cap, q_scale, num_seqs, heads, dim, v_dim,
               positions, cu_q, slots, state, out) -> None:
    """The mLSTM recurrence over the step's tokens.  proj float32 [n, ld] holds the projections
    at the given column offsets; state float32 [slots(+1), state floats]; out float32
    [n, heads * v_dim]."""
    _rows(proj, "mlstm_scan proj")
    n = proj.shape[0]
    if proj.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (n, heads * v_dim) \
            or not out.is_contiguous():
        raise KernelError("mlstm_scan: proj and out must be float32, out contiguous [n, heads * v_dim]")
    if state.dim() != 2 or state.dtype != torch.float32 or state.stride(1) != 1:
        raise KernelError("mlstm_scan: state must be float32 [slots, floats]")
    if cu_q.shape[0] < num_seqs + 1 or slots.shape[0] < num_seqs:
        raise KernelError("mlstm_scan: cu_q / slots are shorter than the step's sequences")
    if i_bias.numel() != heads or f_bias.numel() != heads:
        raise KernelError("mlstm_scan: one gate bias per head")
    check(load().shk_mlstm_scan(
        _dev(proj, "proj"), proj.stride(0), q_off, k_off, v_off, i_off, f_off,
        _dev(i_bias, "i_bias", torch.float32), _dev(f_bias, "f_bias", torch.float32), float(cap), float(q_scale),
        num_seqs, heads, dim, v_dim, _dev(positions, "positions", torch.int32), _dev(cu_q, "cu_q", torch.int32),
        _dev(slots, "slots", torch.int32), _dev(state, "state"), state.stride(0), _dev(out, "out"), _stream()))


def headnorm_gate(o, gate, weight, eps, out, heads, v_dim, gate_act: str = "sigmoid") -> None:
    """out[t, h] = o[t, h] / rms(o[t, h]) * weight[h] * g(gate[t, h]); o float32 [n, heads * v_dim],
    gate float32 rows (a view with a row stride is fine), out of the compute dtype.  weight
    None: none; gate_act "sigmoid" or "silu"."""
    _rows(gate, "headnorm_gate gate")
    n = o.shape[0]
    if o.dtype != torch.float32 or gate.dtype != torch.float32 or not o.is_contiguous() or not out.is_contiguous() \
            or tuple(o.shape) != (n, heads * v_dim) or tuple(out.shape) != (n, heads * v_dim) \
            or gate.shape[0] != n or gate.shape[1] < heads * v_dim \
            or (weight is not None and weight.numel() != heads * v_dim):
        raise KernelError("headnorm_gate: o, gate float32 [n, heads * v_dim], out alike in the compute dtype")
    if gate_act not in ("sigmoid", "silu"):
        raise KernelError(f"headnorm_gate: unknown gate {gate_act!r}")
    check(load().shk_headnorm_gate(_dev(o, "o"), _dev(gate, "gate"), gate.stride(0),
                                   None if weight is None else _dev(weight, "weight", torch.float32), float(eps),
                                   _dev(out, "out"), dtype_code(out.dtype), n, heads, v_dim,
                                   int(gate_act == "silu"), _stream()))


def _delta_any(delta, n, hidden, dtype, who: str):
    """(address, splits) of an addend [n, hidden]: a tensor of the compute dtype or a SplitSum."""
    if isinstance(delta, SplitSum):
        if delta.bias is not None or tuple(delta.shape) != (n, hidden) or delta.parts.dtype != torch.float32 \
                or not delta.parts.is_contiguous():
            raise KernelError(f"{who}: partial sums must be contiguous float32 [splits, n, hidden] without bias")
        return _dev(delta.parts, "delta"), delta.parts.shape[0]
    if delta.dtype != dtype or not delta.is_contiguous() or tuple(delta.shape) != (n, hidden):
        raise KernelError(f"{who}: an addend must be contiguous [n, hidden] of the compute dtype")
    return _dev(delta, "delta"), 0


def _f32vec(t, hidden, who):
    if t is None:
        return None
    if t.dtype != torch.float32 or t.numel() != hidden or not t.is_contiguous():
        raise KernelError(f"{who}: expected a contiguous float32 vector of {hidden}")
    return _dev(t, who)


def add_layernorm(resid, delta=None, dnorm=None, weight=None, bias=None, eps: float = 0.0, out=None, rows=None,
                  write_resid: bool = True, dtype=None) -> None:
    """Layer norm (weight, bias, variance as the mean squared deviation) around the float32
    stream.  resid [N, hidden] gains `delta` (a product's output, tensor or SplitSum), which with
    dnorm = (weight, bias, eps) is normed by itself first; `out` [n, hidden] (the compute dtype,
    or float32; it may be resid itself) receives the layer norm of the sum.  rows: int32 row
    indices, out[r] then belongs to resid[rows[r]]."""
    hidden = resid.shape[1]
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("add_layernorm: resid must be contiguous float32")
    n = resid.shape[0] if rows is None else rows.shape[0]
    if out is not None:
        dtype = out.dtype if out.dtype != torch.float32 or dtype is None else dtype
        if tuple(out.shape) != (n, hidden) or not out.is_contiguous():
            raise KernelError("add_layernorm: out must be contiguous [rows, hidden]")
    if dtype is None:
        dtype = delta.dtype if isinstance(delta, torch.Tensor) else torch.float32
    d_ptr, d_splits = (None, 0) if delta is None else _delta_any(delta, resid.shape[0], hidden, dtype, "add_layernorm")
    dw, db, deps = (None, None, 0.0) if dnorm is None else dnorm
    check(load().shk_add_layernorm(
        _dev(resid, "resid"), d_ptr, d_splits, _f32vec(dw, hidden, "dweight"), _f32vec(db, hidden, "dbias"),
        float(deps), _f32vec(weight, hidden, "weight"), _f32vec(bias, hidden, "bias"), float(eps),
        None if out is None else _dev(out, "out"), dtype_code(dtype),
        int(out is not None and out.dtype == torch.float32),
        None if rows is None else _dev(rows, "rows", torch.int32), n, hidden, int(bool(write_resid)),
        resid.shape[0], _stream()))


def mix_history(history, coef, count: int, out, delta=None, dnorm=None, dtype=None) -> None:
    """out = sum_j coef[j] * history[j], j < count (float32 [slots, n, hidden] -> [n, hidden]); with
    delta and dnorm = (weight, bias, eps), history[count - 1] first gains the normed addend."""
    if history.dim() != 3 or history.dtype != torch.float32 or not history.is_contiguous() or count > history.shape[0]:
        raise KernelError("mix_history: history must be contiguous float32 [slots >= count, n, hidden]")
    _, n, hidden = history.shape
    if tuple(out.shape) != (n, hidden) or out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("mix_history: out must be contiguous float32 [n, hidden]")
    if coef.dtype != torch.float32 or coef.numel() < count or not coef.is_contiguous():
        raise KernelError("mix_history: coef must hold count float32 values")
    if dtype is None:
        dtype = delta.dtype if isinstance(delta, torch.Tensor) else torch.float32
    d_ptr, d_splits = (None, 0) if delta is None else _delta_any(delta, n, hidden, dtype, "mix_history")
    dw, db, deps = (None, None, 0.0) if dnorm is None else dnorm
    check(load().shk_mix_history(_dev(history, "history"), history.stride(0), _dev(coef, "coef"), count,
                                 _dev(out, "out"), n, hidden, d_ptr, d_splits, _f32vec(dw, hidden, "dweight"),
                                 _f32vec(db, hidden, "dbias"), float(deps), dtype_code(dtype), _stream()))


def scale_softcap(x, scale: float, cap) -> None:
    """x <- cap * tanh(x * scale / cap) (cap None: x * scale), float32, in place."""
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("scale_softcap: expected a contiguous float32 tensor")
    check(load().shk_scale_softcap(_dev(x, "x"), x.numel(), float(scale), float(cap or 0.0), _stream()))


def attention_talking_scratch_floats(n: int, heads: int, v_dim: int, nshare: int) -> int:
    return int(load().shk_attention_talking_scratch_floats(n, heads, v_dim, nshare))


def attention_talking(q, out, heads, kv_heads, head_dim, v_dim, positions, token_seq, tables, k_pool, v_pool,
                      page_size, window, scale, scratch, chunk=None, r1=None, r2=None, talk=None, sink=None,
                      nshare: int = 1) -> None:
    """Attention with a distance bias r1 ln(1 + r2 distance) taken off the scores, a sink of
    score `sink` (None: none) in the denominator, and the softmax weights mixed across heads by
    talk [heads, heads] before they meet the values.  q rows [n, >= heads * head_dim]; out
    [n, heads * v_dim]; scratch float32 of attention_talking_scratch_floats(...)."""
    _rows(q, "attention_talking q")
    n = q.shape[0]
    if tuple(out.shape) != (n, heads * v_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("attention_talking: out must be contiguous [n, heads * v_dim] of q's dtype")
    for name, t, count in (("r1", r1, heads), ("r2", r2, heads), ("talk", talk, heads * heads)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != count or not t.is_contiguous()):
            raise KernelError(f"attention_talking: {name} must be contiguous float32 of {count} values")
    if scratch.dtype != torch.float32 or scratch.numel() < attention_talking_scratch_floats(n, heads, v_dim, nshare):
        raise KernelError("attention_talking: scratch is too small")
    _check_pools("attention_talking", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size, v_dim)
    check(load().shk_attention_talking(
        _dev(q, "q"), q.stride(0), _dev(out, "out"), dtype_code(q.dtype), n, heads, kv_heads, head_dim, v_dim,
        _dev(positions, "positions", torch.int32), _dev(token_seq, "token_seq", torch.int32),
        _dev(tables, "tables", torch.int32), tables.shape[1], _dev(k_pool, "k_pool"), _dev(v_pool, "v_pool"),
        page_size, k_pool.shape[0], int(window or 0), int(chunk or 0), float(scale),
        None if r1 is None else _dev(r1, "r1"), None if r2 is None else _dev(r2, "r2"),
        None if talk is None else _dev(talk, "talk"), int(sink is not None), float(sink or 0.0),
        _dev(scratch, "scratch"), int(nshare), _stream()))


def attention_talking_supports_mfma(head_dim: int, v_dim: int, page_size: int, q_stride: int) -> bool:
    return bool(load().shk_attention_talking_supports_mfma(head_dim, v_dim, page_size, q_stride))


def attention_talking_mfma_scratch_floats(n: int, heads: int, kv_heads: int, v_dim: int, num_single: int = 0,
                                          nsplit: int = 1) -> int:
    return int(load().shk_attention_talking_mfma_scratch_floats(n, num_single, heads, kv_heads, v_dim, nsplit))


def attention_talking_mfma(q, out, num_single, heads, kv_heads, head_dim, v_dim, positions, token_seq, cu_q, tile_seq,
                           tile_q0, num_tiles, tables, k_pool, v_pool, page_size, window, scale, scratch, chunk=None,
                           r1=None, r2=None, talk=None, sink=None, nsplit: int = 1) -> None:
    """attention_talking for bfloat16 on the matrix units.  The first num_single rows are single
    tokens of sequences 0 .. num_single - 1; the prompt portions after them are listed as
    num_tiles tiles of 16 queries (tile_seq, tile_q0: int32, q0 counted within the portion).
    nsplit > 1 shares every single token's keys among that many workgroups.
    scratch: float32 of attention_talking_mfma_scratch_floats(...)."""
    _rows(q, "attention_talking_mfma q")
    n = q.shape[0]
    if q.dtype != torch.bfloat16 or tuple(out.shape) != (n, heads * v_dim) or not out.is_contiguous() \
            or out.dtype != q.dtype:
        raise KernelError("attention_talking_mfma: bfloat16 q, out contiguous [n, heads * v_dim]")
    for name, t, count in (("r1", r1, heads), ("r2", r2, heads), ("talk", talk, heads * heads)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != count or not t.is_contiguous()):
            raise KernelError(f"attention_talking_mfma: {name} must be contiguous float32 of {count} values")
    if scratch.dtype != torch.float32 or scratch.numel() < attention_talking_mfma_scratch_floats(
            n, heads, kv_heads, v_dim, num_single, nsplit):
        raise KernelError("attention_talking_mfma: scratch is too small")
    if num_tiles and (tile_seq is None or tile_q0 is None or tile_seq.numel() < num_tiles or tile_q0.numel() < num_tiles):
        raise KernelError("attention_talking_mfma: the tile lists are shorter than num_tiles")
    _check_pools("attention_talking_mfma", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size, v_dim)
    check(load().shk_attention_talking_bf16(
        _dev(q, "q"), q.stride(0), _dev(out, "out"), n, num_single, num_tiles, heads, kv_heads, head_dim, v_dim,
        _dev(positions, "positions", torch.int32), _dev(token_seq, "token_seq", torch.int32),
        _dev(cu_q, "cu_q", torch.int32), None if not num_tiles else _dev(tile_seq, "tile_seq", torch.int32),
        None if not num_tiles else _dev(tile_q0, "tile_q0", torch.int32), _dev(tables, "tables", torch.int32),
        tables.shape[1], _dev(k_pool, "k_pool"), _dev(v_pool, "v_pool"), page_size, k_pool.shape[0], int(window or 0),
        int(chunk or 0), float(scale), None if r1 is None else _dev(r1, "r1"), None if r2 is None else _dev(r2, "r2"),
        None if talk is None else _dev(talk, "talk"), int(sink is not None), float(sink or 0.0),
        _dev(scratch, "scratch"), int(nsplit), _stream()))


def selective_scan_state_floats(inner: int, states: int, taps: int) -> int:
    return int(load().shk_selective_scan_state_floats(inner, states, taps))


def _state2d(state, who):
    if state.dim() != 2 or state.dtype != torch.float32 or state.stride(1) != 1:
        raise KernelError(f"{who}: state must be float32 [slots, floats]")


def conv_silu(x, taps, bias, positions, token_seq, cu_q, slots, state, states: int, y) -> None:
    """y = silu(causal convolution of x's channels over each sequence's inputs): x rows [n, >= inner]
    (a view is fine), taps float32 [inner, K] whose last column meets the current token, the
    slot's kept inputs for the positions before the step."""
    _rows(x, "conv_silu x")
    n, inner = y.shape
    if y.dtype != x.dtype or not y.is_contiguous() or x.shape[0] != n or x.shape[1] < inner:
        raise KernelError("conv_silu: y must be contiguous [n, inner] of x's dtype")
    if taps.dtype != torch.float32 or taps.dim() != 2 or taps.shape[0] != inner or not taps.is_contiguous() \
            or bias.dtype != torch.float32 or bias.numel() != inner:
        raise KernelError("conv_silu: taps float32 [inner, K], bias float32 [inner]")
    _state2d(state, "conv_silu")
    check(load().shk_conv_silu(_dev(x, "x"), x.stride(0), _dev(taps, "taps"), _dev(bias, "bias"), taps.shape[1], inner,
                               _dev(positions, "positions", torch.int32), _dev(token_seq, "token_seq", torch.int32),
                               _dev(cu_q, "cu_q", torch.int32), _dev(slots, "slots", torch.int32), _dev(state, "state"),
                               state.stride(0), states, _dev(y, "y"), dtype_code(y.dtype), n, _stream()))


def dt_softplus(low, w, b, dt) -> None:
    """dt = softplus(low[:, :rank] @ w + b) in float32, w [rank, inner] (the stored matrix transposed);
    low rows may be a view."""
    _rows(low, "dt_softplus low")
    n, inner = dt.shape
    rank = w.shape[0]
    if low.dtype != torch.float32 or dt.dtype != torch.float32 or w.dtype != torch.float32 or b.dtype != torch.float32 \
            or not dt.is_contiguous() or not w.is_contiguous() or tuple(w.shape) != (rank, inner) or b.numel() != inner \
            or low.shape[0] != n or low.shape[1] < rank:
        raise KernelError("dt_softplus: float32 low [n, >= rank], w [rank, inner], b [inner], dt [n, inner]")
    check(load().shk_dt_softplus(_dev(low, "low"), low.stride(0), _dev(w, "w"), _dev(b, "b"), rank, inner,
                                 _dev(dt, "dt"), n, _stream()))


def selective_scan(dt, x, bc, b_off, c_off, z, a_log, dskip, states, taps, raw, positions, cu_q, slots, state,
                   out, num_seqs) -> None:
    """The selective scan over the step's tokens; out = y * silu(z).  dt float32 [n, inner]; x, z,
    raw rows of the compute dtype (views are fine); bc float32 rows with B at b_off and C at c_off."""
    n, inner = dt.shape
    for name, t in (("z", z), ("raw", raw), ("bc", bc)):
        _rows(t, f"selective_scan {name}")
    if dt.dtype != torch.float32 or bc.dtype != torch.float32 or not dt.is_contiguous() or not x.is_contiguous() \
            or not out.is_contiguous() or tuple(x.shape) != (n, inner) or tuple(out.shape) != (n, inner) \
            or x.dtype != out.dtype or z.dtype != out.dtype or raw.dtype != out.dtype \
            or z.shape[1] < inner or raw.shape[1] < inner:
        raise KernelError("selective_scan: mismatched shapes or dtypes")
    if a_log.dtype != torch.float32 or tuple(a_log.shape) != (inner, states) or not a_log.is_contiguous() \
            or dskip.dtype != torch.float32 or dskip.numel() != inner:
        raise KernelError("selective_scan: a_log float32 [inner, states], dskip float32 [inner]")
    _state2d(state, "selective_scan")
    if cu_q.shape[0] < num_seqs + 1 or slots.shape[0] < num_seqs:
        raise KernelError("selective_scan: cu_q / slots are shorter than the step's sequences")
    check(load().shk_selective_scan(
        _dev(dt, "dt"), _dev(x, "x"), _dev(bc, "bc"), bc.stride(0), b_off, c_off, _dev(z, "z"), z.stride(0),
        _dev(a_log, "a_log"), _dev(dskip, "dskip"), inner, states, taps, _dev(raw, "raw"), raw.stride(0),
        _dev(positions, "positions", torch.int32), _dev(cu_q, "cu_q", torch.int32), _dev(slots, "slots", torch.int32),
        _dev(state, "state"), state.stride(0), _dev(out, "out"), dtype_code(out.dtype), num_seqs, _stream()))


def rotate_half_rows(x, off, heads, dim, rot_dim, inv_freq, positions, mult: float = 1.0) -> None:
    """Turns the pairs (i, i + rot_dim / 2) of every head at columns off + h * dim of float32 rows,
    in place, by positions[t] * inv_freq[i], and multiplies the head by mult."""
    _rows(x, "rotate_half_rows x")
    if x.dtype != torch.float32:
        raise KernelError("rotate_half_rows: float32 rows")
    if rot_dim and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() < rot_dim // 2):
        raise KernelError("rotate_half_rows: inv_freq must hold rot_dim / 2 float32 values")
    check(load().shk_rotate_half_rows(_dev(x, "x"), x.stride(0), off, heads, dim, rot_dim,
                                      None if not rot_dim else _dev(inv_freq, "inv_freq"),
                                      _dev(positions, "positions", torch.int32), float(mult), x.shape[0], _stream()))


def retention_state_floats(heads: int, dim: int, v_dim: int) -> int:
    return int(load().shk_retention_state_floats(heads, dim, v_dim))


def retention_scan(proj, q_off, k_off, v_off, decay, num_seqs, heads, dim, v_dim, positions, cu_q, slots, state,
                   out) -> None:
    """S_t = decay S_(t-1) + k v^T, o = S^T q per head over the step's tokens; proj float32 rows,
    out float32 [n, heads * v_dim]."""
    _rows(proj, "retention_scan proj")
    n = proj.shape[0]
    if proj.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (n, heads * v_dim) \
            or not out.is_contiguous():
        raise KernelError("retention_scan: proj and out must be float32, out contiguous [n, heads * v_dim]")
    if decay.dtype != torch.float32 or decay.numel() != heads:
        raise KernelError("retention_scan: one float32 decay per head")
    _state2d(state, "retention_scan")
    if cu_q.shape[0] < num_seqs + 1 or slots.shape[0] < num_seqs:
        raise KernelError("retention_scan: cu_q / slots are shorter than the step's sequences")
    check(load().shk_retention_scan(
        _dev(proj, "proj"), proj.stride(0), q_off, k_off, v_off, _dev(decay, "decay"), num_seqs, heads, dim, v_dim,
        _dev(positions, "positions", torch.int32), _dev(cu_q, "cu_q", torch.int32), _dev(slots, "slots", torch.int32),
        _dev(state, "state"), state.stride(0), _dev(out, "out"), _stream()))


def moe_route(logits, correction, top: int, chosen, weights) -> None:
    """softmax over float32 logits [n, experts]; the `top` largest of score + correction chosen
    (int32 [n, top]), weights their scores over the chosen ones' sum (float32 [n, top])."""
    _rows(logits, "moe_route logits")
    n, experts = logits.shape
    if logits.dtype != torch.float32 or chosen.dtype != torch.int32 or weights.dtype != torch.float32 \
            or tuple(chosen.shape) != (n, top) or tuple(weights.shape) != (n, top) \
            or not chosen.is_contiguous() or not weights.is_contiguous():
        raise KernelError("moe_route: logits float32 [n, experts], chosen int32 / weights float32 [n, top]")
    if correction is not None and (correction.dtype != torch.float32 or correction.numel() != experts):
        raise KernelError("moe_route: one float32 correction per expert")
    check(load().shk_moe_route(_dev(logits, "logits"), logits.stride(0),
                               None if correction is None else _dev(correction, "correction"), experts, top,
                               _dev(chosen, "chosen"), _dev(weights, "weights"), n, _stream()))


MOE_GROUPED_FROM = 1  # tokens of a step from which the experts' products run per expert on the matrix units


def moe_grouped(n: int, width: int, ff: int, dtype) -> bool:
    """Whether a step of n tokens runs its experts' products per expert on the matrix units:
    bfloat16 and rows in multiples of 8 elements."""
    return dtype == torch.bfloat16 and n >= MOE_GROUPED_FROM and width % 8 == 0 and ff % 8 == 0


def moe_grouped_scratch_bytes(n: int, width: int, experts: int, top: int) -> int:
    return int(load().shk_moe_grouped_scratch_bytes(n, width, experts, top))


def moe_experts(x, chosen, weights, w_gate, w_up, w_down, act_buf, out, activation: str = "silu", add=None,
                scratch=None, add_gate=None) -> None:
    """out = add + sum_k weights[:, k] * down_e(act(gate_e x) * up_e x), e = chosen[:, k]; matrices
    stacked [experts, ff, width] / [experts, width, ff] row-major in x's dtype.  scratch (uint8,
    moe_grouped_scratch_bytes): the products run per expert on the matrix units (see moe_grouped).
    add_gate: a float32 column (a view [n] with any stride): add[t] is multiplied by
    sigmoid(add_gate[t]).  Experts without a gate whose activation is the square of ReLU pass
    their one matrix as both w_gate and w_up with activation "relu"."""
    n, width = x.shape
    experts, ff, _ = w_gate.shape
    top = chosen.shape[1]
    tensors = (x, w_gate, w_up, w_down, act_buf, out) + (() if add is None else (add,))
    if any(t.dtype != x.dtype or not t.is_contiguous() for t in tensors):
        raise KernelError("moe_experts: tensors must be contiguous and of one dtype")
    if tuple(w_gate.shape) != (experts, ff, width) or tuple(w_up.shape) != (experts, ff, width) \
            or tuple(w_down.shape) != (experts, width, ff) or tuple(out.shape) != (n, width) \
            or act_buf.numel() < n * top * ff or (add is not None and tuple(add.shape) != (n, width)) \
            or tuple(weights.shape) != (n, top) or chosen.dtype != torch.int32 or weights.dtype != torch.float32:
        raise KernelError("moe_experts: mismatched shapes")
    gate_ptr, gate_ld = None, 0
    if add_gate is not None:
        if add is None or add_gate.dtype != torch.float32 or add_gate.dim() != 1 or add_gate.shape[0] != n:
            raise KernelError("moe_experts: add_gate is a float32 column of n numbers and needs `add`")
        gate_ptr, gate_ld = _dev(add_gate, "add_gate"), max(1, add_gate.stride(0))
    if scratch is not None:
        if not moe_grouped(n, width, ff, x.dtype) or scratch.dtype != torch.uint8 \
                or scratch.numel() < moe_grouped_scratch_bytes(n, width, experts, top):
            raise KernelError("moe_experts: scratch is for bfloat16 steps that moe_grouped() accepts, and must hold "
                              "moe_grouped_scratch_bytes() bytes")
        check(load().shk_moe_experts_grouped(
            _dev(x, "x"), _dev(chosen, "chosen"), _dev(weights, "weights"), _dev(w_gate, "w_gate"), _dev(w_up, "w_up"),
            _dev(w_down, "w_down"), None if add is None else _dev(add, "add"), gate_ptr, gate_ld,
            _dev(act_buf, "act_buf"), _dev(out, "out"), _dev(scratch, "scratch"), n, width, ff, experts, top, activation_code(activation),
            _stream()))
        return
    check(load().shk_moe_experts(_dev(x, "x"), _dev(chosen, "chosen"), _dev(weights, "weights"), _dev(w_gate, "w_gate"),
                                 _dev(w_up, "w_up"), _dev(w_down, "w_down"), None if add is None else _dev(add, "add"),
                                 gate_ptr, gate_ld, _dev(act_buf, "act_buf"), _dev(out, "out"), dtype_code(x.dtype), n, width, ff, experts,
                                 top, activation_code(activation), _stream()))


def xielu(x, out, a_pos: float, a_neg: float) -> None:
    """out = a_pos x^2 + x / 2 where x > 0, a_neg (exp(x) - 1 - x) + x / 2 elsewhere."""
    if x.shape != out.shape or x.dtype != out.dtype or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError("xielu: x and out must be contiguous and alike")
    check(load().shk_xielu(_dev(x, "x"), _dev(out, "out"), dtype_code(x.dtype), x.numel(), float(a_pos),
                           float(a_neg), _stream()))


def embed_pairs(table, pair_table, ids, positions, token_seq, cu_q, slots, last_token, out, buckets, mul_prev,
                mul_cur) -> None:
    """out[i] = table[ids[i]] + pair_table[hash(previous token, ids[i])] in float32; the token before a
    step's first one comes from last_token[slots[seq]] (int32 [slots(+1)]), which receives the
    step's last one."""
    n, hidden = out.shape
    if not (table.is_contiguous() and pair_table.is_contiguous() and out.is_contiguous()) \
            or table.shape[1] != hidden or tuple(pair_table.shape) != (buckets + 1, hidden) \
            or pair_table.dtype != table.dtype:
        raise KernelError("embed_pairs: table [vocab, hidden], pair_table [buckets + 1, hidden], out [n, hidden]")
    if last_token.dtype != torch.int32 or not last_token.is_contiguous():
        raise KernelError("embed_pairs: last_token must be contiguous int32")
    check(load().shk_embed_pairs(
        _dev(table, "table"), _dev(pair_table, "pair_table"), dtype_code(table.dtype),
        _dev(ids, "ids", torch.int32), _dev(positions, "positions", torch.int32),
        _dev(token_seq, "token_seq", torch.int32), _dev(cu_q, "cu_q", torch.int32),
        _dev(slots, "slots", torch.int32), _dev(last_token, "last_token"), _dev(out, "out", torch.float32),
        n, hidden, table.shape[0], int(buckets), int(mul_prev), int(mul_cur), _stream()))


def attention_supports_mfma(heads, kv_heads, head_dim, page_size, q_stride) -> bool:
    return bool(load().shk_attention_supports_mfma(heads, kv_heads, head_dim, page_size, q_stride))


def _sinks(sinks, heads, who):
    if sinks is None:
        return None
    if sinks.numel() != heads or not sinks.is_contiguous():
        raise KernelError(f"{who}: sinks must hold one value per head ({heads})")
    return _dev(sinks, "sinks", torch.float32)


def attention_decode(q, out, num_seqs, heads, kv_heads, head_dim, positions, tables, k_pool, v_pool,
                     page_size, window, scale, partial, nsplit, streaming=False, chunk=None, softcap=None,
                     sinks=None, dist_bias=None) -> None:
    """bfloat16 MFMA attention for the first num_seqs rows of q, one token per sequence.
    `streaming`: fetch keys and values with non-temporal loads (same result; faster when
    the launch reads tens of megabytes of them)."""
    _rows(q, "attention_decode q")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_decode: bfloat16 only")
    if q.shape[0] < num_seqs or tables.shape[0] < num_seqs or positions.shape[0] < num_seqs:
        raise KernelError("attention_decode: fewer rows than sequences")
    if out.shape[0] < num_seqs or out.shape[1] != heads * head_dim or not out.is_contiguous():
        raise KernelError("attention_decode: out must be contiguous [>= num_seqs, heads*head_dim]")
    _check_pools("attention_decode", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
    if partial.numel() < num_seqs * heads * nsplit * (head_dim + 2):
        raise KernelError("attention_decode: partial scratch is too small")
    check(
        load().shk_attention_decode_bf16(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), num_seqs, heads, kv_heads, head_dim,
            _dev(positions, "positions", torch.int32), _dev(tables, "tables", torch.int32),
            tables.shape[1], _dev(k_pool, "k_pool"), _dev(v_pool, "v_pool"), page_size,
            int(window or 0), int(chunk or 0), float(scale), _dev(partial, "partial", torch.float32), nsplit,
            int(bool(streaming)), float(softcap or 0.0), _sinks(sinks, heads, "attention_decode"),
            *_dist_bias_args(dist_bias, heads, "attention_decode"), _stream(),
        )
    )


def attention_prefill(q, out, num_tiles, heads, kv_heads, head_dim, cu_q, ctx_lens, tile_seq, tile_q0,
                      tables, k_pool, v_pool, page_size, window, scale, chunk=None) -> None:
    """bfloat16 MFMA attention for prompt portions, in tiles of 16 queries."""
    _rows(q, "attention_prefill q")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_prefill: bfloat16 only")
    if out.shape != (q.shape[0], heads * head_dim) or not out.is_contiguous():
        raise KernelError("attention_prefill: out must be contiguous [n, heads*head_dim]")
    if tile_seq.shape[0] < num_tiles or tile_q0.shape[0] < num_tiles:
        raise KernelError("attention_prefill: tile arrays are shorter than num_tiles")
    _check_pools("attention_prefill", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
    check(
        load().shk_attention_prefill_bf16(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), num_tiles, heads, kv_heads, head_dim,
            _dev(cu_q, "cu_q", torch.int32), _dev(ctx_lens, "ctx_lens", torch.int32),
            _dev(tile_seq, "tile_seq", torch.int32), _dev(tile_q0, "tile_q0", torch.int32),
            _dev(tables, "tables", torch.int32), tables.shape[1], _dev(k_pool, "k_pool"),
            _dev(v_pool, "v_pool"), page_size, int(window or 0), int(chunk or 0), float(scale), _stream(),
        )
    )


def attention_prefill_shared_tiles(heads, kv_heads, head_dim, small=False) -> int:
    """16-query tiles per workgroup of attention_prefill_shared (`small`: of its
    variant with half as many wavefronts); 0 if the shape is not served."""
    return int(load().shk_attention_prefill_shared_tiles(heads, kv_heads, head_dim, int(small)))


def attention_prefill_shared(q, out, num_wgs, heads, kv_heads, head_dim, cu_q, ctx_lens, wg_seq, wg_q0,
                             tables, k_pool, v_pool, page_size, window, scale, small=False,
                             partial=None, nsplit: int = 1, first_token: int = 0, chunk=None, softcap=None,
                             sinks=None, dist_bias=None) -> None:
    """bfloat16 MFMA attention for prompt portions; one workgroup per (run of query
    tiles, key/value head) shares each chunk of keys among its query heads.
    wg_seq / wg_q0 are in steps of 16 * attention_prefill_shared_tiles(..., small),
    launched in the list's order.  nsplit > 1 shares every entry's keys among
    that many workgroups, whose results pass through `partial` (float32, (rows
    of q from first_token on) * heads * nsplit * (head_dim + 2) values)."""
    _rows(q, "attention_prefill_shared q")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_prefill_shared: bfloat16 only")
    if out.shape != (q.shape[0], heads * head_dim) or not out.is_contiguous():
        raise KernelError("attention_prefill_shared: out must be contiguous [n, heads*head_dim]")
    if wg_seq.shape[0] < num_wgs or wg_q0.shape[0] < num_wgs:
        raise KernelError("attention_prefill_shared: workgroup arrays are shorter than num_wgs")
    _check_pools("attention_prefill_shared", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
    prompt_tokens = q.shape[0] - first_token
    if nsplit > 1:
        need = prompt_tokens * heads * nsplit * (head_dim + 2)
        if partial is None or partial.dtype != torch.float32 or partial.numel() < need or prompt_tokens <= 0:
            raise KernelError(f"attention_prefill_shared: {nsplit} key splits need a float32 partial buffer "
                              f"of {need} values for the {prompt_tokens} prompt tokens")
    check(
        load().shk_attention_prefill_shared_bf16(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), num_wgs, heads, kv_heads, head_dim,
            _dev(cu_q, "cu_q", torch.int32), _dev(ctx_lens, "ctx_lens", torch.int32),
            _dev(wg_seq, "wg_seq", torch.int32), _dev(wg_q0, "wg_q0", torch.int32),
            _dev(tables, "tables", torch.int32), tables.shape[1], _dev(k_pool, "k_pool"),
            _dev(v_pool, "v_pool"), page_size, int(window or 0), int(chunk or 0), float(scale), int(small),
            _dev(partial, "partial", torch.float32) if nsplit > 1 else None, int(nsplit), int(first_token),
            int(prompt_tokens), float(softcap or 0.0), _sinks(sinks, heads, "attention_prefill_shared"),
            *_dist_bias_args(dist_bias, heads, "attention_prefill_shared"), _stream(),
        )
    )


_ARGMAX_SCRATCH: dict = {}


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = lowest index of the maximum of logits[r]; logits float32 [rows, vocab]."""
    _rows(logits, "argmax logits")
    rows, vocab = logits.shape
    need = load().shk_argmax_scratch_floats(rows, vocab)
    scratch = None
    if need:
        key = (logits.device.type, logits.device.index)
        scratch = _ARGMAX_SCRATCH.get(key)
        if scratch is None or scratch.numel() < need:
            scratch = torch.empty(max(need, 1 << 16), dtype=torch.float32, device=logits.device)
            _ARGMAX_SCRATCH[key] = scratch
    check(load().shk_argmax(_dev(logits, "logits", torch.float32), _dev(out, "out", torch.int32),
                            rows, vocab, logits.stride(0),
                            None if scratch is None else scratch.data_ptr(), _stream()))


def sample_scratch_floats(rows: int, vocab: int) -> int:
    """float32 elements of scratch that sample() needs for logits [rows, vocab]."""
    return int(load().shk_sample_scratch_floats(rows, vocab))


def sample(logits, out, temperature, top_p, uniforms, scratch, nucleus: bool = True) -> None:
    """One token per row: argmax where temperature is 0, else a top-p draw with uniforms[r].
    nucleus=False promises that no row has a top_p below 1 (fewer passes)."""
    _rows(logits, "sample logits")
    rows, vocab = logits.shape
    if scratch.numel() < sample_scratch_floats(rows, vocab):
        raise KernelError(f"sample: scratch needs {sample_scratch_floats(rows, vocab)} float32 elements "
                          "(sample_scratch_floats)")
    check(
        load().shk_sample(
            _dev(logits, "logits", torch.float32), _dev(out, "out", torch.int32),
            _dev(temperature, "temperature", torch.float32), _dev(top_p, "top_p", torch.float32),
            _dev(uniforms, "uniforms", torch.float32), _dev(scratch, "scratch", torch.float32),
            scratch.numel(), rows, vocab, logits.stride(0), int(bool(nucleus)), _stream(),
        )
    )
