"""Causal grouped-query attention over the paged key/value cache."""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..kernels import ops
from .base import PAGE, Mixer, PagedSpec, PageTensor, ParamSpec, PositionEncoding, build_part, register_mixer

QUERY_TILE = 16  # queries per tile of the MFMA kernels for prompt portions
COMPUTE_UNITS = 256  # of an MI355X; compute_units() asks the device that is there
KEYS_PER_WORKGROUP = 256  # a decode workgroup's four wavefronts want at least this many keys
MAX_KEY_SPLITS = 64
# decode attention fetches keys and values with non-temporal loads from this many bytes
# of them per launch on (counted with the batch and the context rounded up to powers of two)
STREAMING_FROM_BYTES = 96 << 20
_UNITS: int | None = None


def compute_units() -> int:
    """Compute units of the GPU the process runs on (read once; COMPUTE_UNITS where no
    GPU is visible, so that launch plans can be computed and tested without one)."""
    global _UNITS
    if _UNITS is None:
        _UNITS = (torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
                  if torch.cuda.is_available() else COMPUTE_UNITS)
    return _UNITS


def kv_cache_spec(num_kv_heads: int, head_dim: int, window: int | None = None,
                  chunk: int | None = None, value_dim: int | None = None) -> PagedSpec:
    """The cache of grouped-query attention, laid out for this file's kernels: per
    page and key/value head the keys in slabs of 32 elements, [head_dim / 32,
    page_size, 32] (a wavefront's operand load for the matrix instruction then
    touches whole cache lines: 64 bytes from each of four consecutive keys; one
    slab of head_dim elements where head_dim is no multiple of 32), and the values
    transposed, [head_dim, page_size] (the keys of a page side by side for every
    element, which is the operand layout of V^T).  `value_dim`: the size of a value
    where it is not the keys' size."""
    slab = ops.key_slab(head_dim)
    return PagedSpec(
        tensors=(PageTensor("k", (num_kv_heads, head_dim // slab, PAGE, slab)),
                 PageTensor("v", (num_kv_heads, head_dim if value_dim is None else value_dim, PAGE))),
        window=window,
        chunk=chunk,
    )


def distance_buckets(rows: int, reach: int) -> list[int]:
    """Row of a [rows, heads] bias table for every distance 0 .. reach between a query and a key:
    with half = rows // 2, the distances below half have a row each; from there on the row is half
    + floor(ln(d / half) / ln(reach / half) * (rows - half)), the rest of the rows spread evenly over
    the logarithm of the distance up to `reach`; the last row serves that distance and all beyond."""
    import math

    half = rows // 2
    out = []
    for d in range(reach + 1):
        if d < half:
            out.append(d)
        elif half <= 0 or reach <= half:
            out.append(rows - 1)
        else:
            out.append(min(rows - 1, half + math.floor(math.log(d / half) / math.log(reach / half) * (rows - half))))
    return out


def _pow2(n: int, floor: int = 1) -> int:
    b = floor
    while b < n:
        b *= 2
    return b


def decode_splits(num_seqs: int, kv_heads: int, max_ctx: int) -> int:
    """Workgroups per (sequence, key/value head) of decode attention: enough to
    put one on every compute unit, each with at least KEYS_PER_WORKGROUP keys
    for its four wavefronts.  Both inputs are rounded up to powers of two first,
    so a step gives the same result whether it runs kernel by kernel or as a
    graph captured for a padded batch."""
    want = -(-compute_units() // (_pow2(num_seqs) * kv_heads))
    most = max(1, _pow2(max_ctx, KEYS_PER_WORKGROUP) // KEYS_PER_WORKGROUP)
    return max(1, min(want, most, MAX_KEY_SPLITS))


def decode_streams(num_seqs: int, kv_heads: int, head_dim: int, max_ctx: int, window: int | None = None) -> bool:
    """Whether a decode launch reads so many keys and values that non-temporal
    loads pay (measured with 4 key/value heads of 128: a tenth faster from 64
    sequences of 2,200 keys or 8 of 16,000, 2 % at 8 of 4,000, 1 to 4 % slower
    below).  The result is the same either way; batch and context are rounded up
    as in decode_splits(), so that a graph's steps all decide alike."""
    keys = _pow2(max_ctx, KEYS_PER_WORKGROUP)
    if window:
        keys = min(keys, window)
    return _pow2(num_seqs) * keys * kv_heads * head_dim * 4 >= STREAMING_FROM_BYTES


@dataclass
class AttentionPlan:
    """How one step's attention is launched for a (heads, kv heads, head size)."""

    mfma: bool = False
    nsplit: int = 1  # key splits of the single-token rows
    streaming: bool = False  # single-token rows: non-temporal loads of keys and values
    kernel: str = ""  # for prompt portions: "shared", "tiles" or "" (none in the step)
    small: bool = False  # "shared" with half as many wavefronts per workgroup
    portion_splits: int = 1  # "shared": workgroups that share an entry's keys
    first_token: int = 0  # index of the step's first prompt token
    count: int = 0  # workgroups ("shared") or tiles ("tiles")
    seq_name: str = ""  # names of the launch lists among the step's extras
    q0_name: str = ""


def portion_runs(q_lens, first_seq: int, run: int):
    """Prompt portions cut into runs of `run` queries: (sequence of each run, its
    first query within the portion)."""
    counts = -(-np.asarray(q_lens, dtype=np.int64) // run)
    seqs = np.repeat(np.arange(first_seq, first_seq + counts.size), counts)
    first = np.zeros(counts.size + 1, dtype=np.int64)
    np.cumsum(counts, out=first[1:])
    q0 = (np.arange(int(counts.sum())) - first[seqs - first_seq]) * run
    return seqs, q0


def portion_splits(workgroups: int, mean_keys: int) -> int:
    """Among how many workgroups each entry of a step's prompt portions shares
    its keys.  A few hundred queries far into a sequence (a long prompt cut by
    the token budget) make few workgroups with thousands of keys each; shared,
    they fill the chip.  Measured at 28 heads over 4, 512 queries (128
    workgroups): at position 1,536 64 us a layer unshared, 47 / 40 / 48 in 2 / 4
    / 8 shares; at 31,000 900 us against 464 / 337 / 345; from position 0 (264
    keys on average) 21 us against 25 in 2.  Hence as many shares as bring the
    launch to twice the compute units, each worth 256 keys or more on average."""
    if workgroups <= 0:
        return 1
    return max(1, min(2 * compute_units() // workgroups, mean_keys // KEYS_PER_WORKGROUP, MAX_KEY_SPLITS))


def heavy_first(work):
    """The order in which workgroups of unequal `work` are launched: the
    heaviest first (a causal prompt's last queries read every key, its first
    ones few), so that the light ones fill the compute units that the heavy
    ones leave last."""
    return np.argsort(-np.asarray(work, dtype=np.int64), kind="stable")


class PagedAttention(Mixer):
    """q/k/v projections (with or without bias), position encoding of q and k,
    cache write, attention over the sequence's pages, output projection
    (reference: shrike/models/qwen.py:111-125, shrike/engine/model_runner.py:63-151).
    Beyond the reference's model, by the spec: a window, a block-local mask
    (`chunk`), and values that are the keys before their rotation
    (`values_from_keys`: no value projection, the cache still holds both);
    without rotation also values of another size than keys, a query temperature,
    normed values, normed queries and keys (with or without weights), capped
    scores, sinks, a learned bias by distance from a table (laid out by distance
    when the weights are loaded), and layers without keys and values of their
    own that read another run's cache.

    The three projections are stacked into one [(H + 2 Hkv) D, h] matrix at
    load time; head j of q is rows j*D..(j+1)*D-1 of the q part, as in the
    reference's view (qwen.py:120-122).
    """

    @property
    def launches_follow_shape(self):
        # the plan of a step's launches is a function of the step's shape and goes into its
        # launch key (prepare); a position encoding of its own kind must say the same of itself
        return self.position is None or self.position.launches_follow_shape

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.position = (
            build_part("position", spec.position, width, name) if spec.position is not None else None
        )

    @property
    def value_dim(self) -> int:
        s = self.spec
        return s.head_dim if getattr(s, "value_dim", None) is None else int(s.value_dim)

    @property
    def plain_store(self) -> bool:
        """Whether the step goes through the cache-write kernel without rotation that
        takes values of another size than keys, the queries' temperature and the
        values' unit norm (attention itself then runs on the matrix-instruction kernels
        where they take the shape, values as large as keys included, else on the general
        kernel)."""
        s = self.spec
        return bool(self.value_dim != s.head_dim or getattr(s, "query_temperature", None)
                    or getattr(s, "value_norm_eps", None) or getattr(s, "softcap", None)
                    or getattr(s, "sinks", False) or self.talking or getattr(s, "qk_norm", None)
                    or getattr(s, "bucket_bias", None) or self.shared_kv)

    @property
    def shared_kv(self) -> bool:
        """Whether the layer has no keys and values of its own and reads another run's cache."""
        return bool(getattr(self.spec, "shared_kv", False))

    @property
    def talking(self) -> bool:
        """Whether the step's attention runs in the kernels that keep a token's heads together:
        a distance bias, a sink of fixed score, or weights mixed across heads."""
        s = self.spec
        return bool(getattr(s, "distance_bias", False) or getattr(s, "fixed_sink", None) is not None
                    or getattr(s, "talking_heads", False))

    def params(self):
        s, h = self.spec, self.width
        q, kv = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
        t = self._tensor
        out = [ParamSpec(t("q"), (q, h))]
        if not self.shared_kv:
            out.append(ParamSpec(t("k"), (kv, h)))
            if not s.values_from_keys:
                out.append(ParamSpec(t("v"), (s.num_kv_heads * self.value_dim, h)))
        out.append(ParamSpec(t("o"), (h, s.num_heads * self.value_dim)))
        qk_norm = getattr(s, "qk_norm", None)
        if qk_norm and qk_norm[1]:
            out.append(ParamSpec(t("q_norm"), (s.head_dim,), init="norm", keep_float32=True))
            if not self.shared_kv:
                out.append(ParamSpec(t("k_norm"), (s.head_dim,), init="norm", keep_float32=True))
        if getattr(s, "bucket_bias", None):
            # (rows None: the table has as many rows as the file's tensor; random weights then draw 32)
            rows = s.bucket_bias[0]
            out.append(ParamSpec(t("rel"), (None if rows is None else int(rows), s.num_heads), init="score_bias",
                                 keep_float32=True, free_size=32))
        if getattr(s, "sinks", False):
            out.append(ParamSpec(t("sink"), (s.num_heads,), init="bias", keep_float32=True))
        if getattr(s, "distance_bias", False):
            out += [ParamSpec(t("r1"), (s.num_heads,), init="positive", keep_float32=True),
                    ParamSpec(t("r2"), (s.num_heads,), init="positive", keep_float32=True)]
        if getattr(s, "talking_heads", False):
            out.append(ParamSpec(t("talk"), (s.num_heads, s.num_heads), init="near_identity", keep_float32=True))
        if s.qkv_bias:
            out += [ParamSpec(t(f"{r}_bias"), (q if r == "q" else kv,), init="bias", keep_float32=True)
                    for r in ("q", "k") + (() if s.values_from_keys else ("v",))]
        if s.out_bias:
            out.append(ParamSpec(t("o_bias"), (h,), init="bias", keep_float32=True))
        return out

    _DEFAULT_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                      "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias",
                      "o_bias": "o_proj.bias", "sink": "sinks", "r1": "r1", "r2": "r2", "talk": "talk",
                      "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "rel": "rel"}

    def _tensor(self, role: str) -> str:
        return self.tensor_name(role, self._DEFAULT_NAMES[role])

    def cache_spec(self):
        s = self.spec
        kept = getattr(s, "cache_window", "own")
        return kv_cache_spec(s.num_kv_heads, s.head_dim, s.window if kept == "own" else kept, s.chunk,
                             None if self.value_dim == s.head_dim else self.value_dim)

    def check(self, runtime):
        s = self.spec
        if self.plain_store:
            if self.position is not None or s.values_from_keys or s.qkv_bias:
                raise ValueError(f"{self.name}: values of another size than keys, a query temperature, normed "
                                 "values, capped scores and sinks are built for attention without rotation, "
                                 "without biases on q, k, v and with values of their own")
            if not 1 <= self.value_dim <= 256:
                raise ValueError(f"{self.name}: value_dim {self.value_dim} is outside 1..256")
            qt = getattr(s, "query_temperature", None)
            if qt is not None and (len(qt) != 2 or int(qt[1]) < 1):
                raise ValueError(f"{self.name}: query_temperature must be (coef, every) with every >= 1, got {qt}")
            if getattr(s, "softcap", None) is not None and not s.softcap > 0:
                raise ValueError(f"{self.name}: softcap must be positive, got {s.softcap}")
        qk_norm, buckets = getattr(s, "qk_norm", None), getattr(s, "bucket_bias", None)
        if qk_norm is not None and (len(qk_norm) != 2 or not float(qk_norm[0]) > 0):
            raise ValueError(f"{self.name}: qk_norm must be (eps > 0, weighted), got {qk_norm}")
        if buckets is not None and (len(buckets) != 2 or (buckets[0] is not None and int(buckets[0]) < 1)
                                    or int(buckets[1]) < 1):
            raise ValueError(f"{self.name}: bucket_bias must be (rows >= 1, reach >= 1), got {buckets}")
        if self.talking and (qk_norm or buckets or self.shared_kv):
            raise ValueError(f"{self.name}: a distance bias by formula, a fixed sink and mixed heads are built "
                             "without normed queries and keys, a bias table and a cache of another layer")
        kept = getattr(s, "cache_window", "own")
        if kept != "own" and kept is not None and (s.window is None or kept < s.window):
            raise ValueError(f"{self.name}: the cache keeps {kept} keys, fewer than the layer's own window")
        if self.talking and (getattr(s, "sinks", False) or getattr(s, "softcap", None)
                             or getattr(s, "query_temperature", None) or getattr(s, "value_norm_eps", None)):
            raise ValueError(f"{self.name}: a distance bias, a fixed sink and mixed heads are built without "
                             "learned sinks, capped scores, a query temperature and normed values")
        if s.num_heads % s.num_kv_heads:
            raise ValueError(
                f"{self.name}: {s.num_heads} query heads are not a multiple of "
                f"{s.num_kv_heads} key/value heads"
            )
        if not 1 <= s.head_dim <= 256:
            raise ValueError(f"{self.name}: head_dim {s.head_dim} is outside 1..256")
        if s.window is not None and s.window < 1:
            raise ValueError(f"{self.name}: window must be positive, got {s.window}")
        if s.chunk is not None and s.chunk < 1:
            raise ValueError(f"{self.name}: chunk must be positive, got {s.chunk}")
        if s.values_from_keys and self.position is not None and \
                type(self.position).rotary_table is PositionEncoding.rotary_table:
            raise ValueError(f"{self.name}: values that are the keys before their position encoding need "
                             "an encoding that the cache-write kernel applies")

    def load(self, tensors, runtime):
        s, t = self.spec, self._tensor
        roles = ("q",) if self.shared_kv else ("q", "k") if s.values_from_keys else ("q", "k", "v")
        self.w_qkv = runtime.weight(torch.cat([tensors[t(r)] for r in roles], dim=0))
        self.b_qkv = torch.cat([tensors[t(f"{r}_bias")] for r in roles]).contiguous() if s.qkv_bias else None
        self.w_o = runtime.weight(tensors[t("o")])
        self.b_o = tensors[t("o_bias")] if s.out_bias else None
        self.sinks = tensors[t("sink")].contiguous() if getattr(s, "sinks", False) else None
        bias = getattr(s, "distance_bias", False)
        self.r1 = tensors[t("r1")].contiguous() if bias else None
        self.r2 = tensors[t("r2")].contiguous() if bias else None
        self.talk = tensors[t("talk")].contiguous() if getattr(s, "talking_heads", False) else None
        qk_norm = getattr(s, "qk_norm", None)
        self.q_norm = self.k_norm = None
        if qk_norm and qk_norm[1]:
            self.q_norm = tensors[t("q_norm")].contiguous()
            self.k_norm = None if self.shared_kv else tensors[t("k_norm")].contiguous()
        self.dist_bias = None
        if getattr(s, "bucket_bias", None):
            # the table by distance, a row per head: the kernels look a distance up, not its bucket
            rows, reach = int(tensors[t("rel")].shape[0]), int(s.bucket_bias[1])
            index = torch.tensor(distance_buckets(rows, reach), dtype=torch.long, device=tensors[t("rel")].device)
            self.dist_bias = tensors[t("rel")].to(torch.float32)[index].t().contiguous()
        if self.position is not None:
            self.position.load(tensors, runtime)
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred
        self.dtype = runtime.dtype

    # ------------------------------------------------------------ launch plans

    @property
    def plan_key(self):
        s = self.spec
        return ("paged_attention", s.num_heads, s.num_kv_heads, s.head_dim, s.window, s.chunk, self.plain_store,
                self.talking, self.value_dim, self._qkv_width(), bool(getattr(s, "bucket_bias", None)),
                bool(getattr(s, "softcap", None)), bool(getattr(s, "sinks", False)))

    def prepare(self, shape) -> None:
        """Decides once per step and head geometry how attention is launched:
        the key splits of single-token rows, and for prompt portions the kernel
        and its list of workgroups, which goes up with the step's metadata."""
        key = self.plan_key
        if key in shape.notes:
            return  # a layer with the same geometry has prepared this step
        s = self.spec
        h, hkv, d = s.num_heads, s.num_kv_heads, s.head_dim
        plan = shape.notes[key] = AttentionPlan()
        if self.talking and self.dtype == torch.bfloat16 and ops.attention_talking_supports_mfma(
                d, self.value_dim, shape.page_size, self._qkv_width()):
            # on the matrix units: single tokens by key/value head, prompt portions in tiles of 16 queries
            plan.kernel = "talking_mfma"
            portions = shape.q_lens[shape.num_decode:]
            plan.count = 0
            if portions.size:
                seqs, q0 = portion_runs(portions, shape.num_decode, QUERY_TILE)
                keys = shape.starts[seqs] + q0  # (the heaviest tiles first)
                order = heavy_first(np.minimum(keys, s.window) if s.window else keys)
                seqs, q0 = seqs[order], q0[order]
                plan.count = int(seqs.size)
                tag = f"talking:{h}:{hkv}:{d}:{s.window or 0}:{s.chunk or 0}"
                plan.seq_name, plan.q0_name = f"attention_seq:{tag}", f"attention_q0:{tag}"
                shape.add(plan.seq_name, seqs)
                shape.add(plan.q0_name, q0)
            if shape.num_decode:
                # single tokens with many keys share them among workgroups: as many shares as bring the
                # launch to twice the compute units, each worth 128 keys or more
                reach = min(x for x in (s.window, s.chunk, shape.max_decode_ctx or 1) if x)
                launched = shape.num_decode * hkv * -(-hkv * -(-(h // hkv) // 16) // 4)
                plan.nsplit = max(1, min(2 * compute_units() // launched, reach // 128, 32))
            shape.launch_key.append((key, "talking_mfma", shape.num_decode, plan.count, plan.nsplit))
            return
        if self.talking:
            # a token's heads stay together in one workgroup; single tokens with many keys share
            # them among workgroups (bfloat16 only: float32 keeps one order of summation whatever
            # the step holds)
            reach = min(x for x in (s.window, s.chunk, _pow2(shape.max_decode_ctx or 1, KEYS_PER_WORKGROUP)) if x)
            if self.dtype == torch.bfloat16 and shape.num_decode == shape.num_seqs and shape.num_decode:
                plan.nsplit = max(1, min(compute_units() // _pow2(shape.num_decode), -(-reach // 256), 32))
            shape.launch_key.append((key, "talking", plan.nsplit))
            return
        plan.mfma = self.dtype == torch.bfloat16 and self.value_dim == d and ops.attention_supports_mfma(
            h, hkv, d, shape.page_size, self._qkv_width())
        # capped scores, sinks and a bias table are built into the decode kernel and the shared-key prompt
        # kernel; where the latter does not take the shape, the general kernel serves the step
        if plan.mfma and (getattr(s, "softcap", None) or getattr(s, "sinks", False) or getattr(s, "bucket_bias", None)) \
                and not ops.attention_prefill_shared_tiles(h, hkv, d):
            plan.mfma = False
        # the most keys that any query reads, where the mask bounds them
        reach = min(x for x in (s.window, s.chunk, 1 << 40) if x)
        if not plan.mfma:
            return  # the general kernel takes every token alike
        if shape.num_decode:
            plan.nsplit = decode_splits(shape.num_decode, hkv, min(shape.max_decode_ctx, reach))
            plan.streaming = decode_streams(shape.num_decode, hkv, d, shape.max_decode_ctx,
                                            reach if s.window or s.chunk else None)
            shape.launch_key.append((key, plan.nsplit, plan.streaming))
        portions = shape.q_lens[shape.num_decode:]
        if portions.size == 0:
            return
        tiles = ops.attention_prefill_shared_tiles(h, hkv, d)
        if tiles:
            plan.kernel = "shared"
            small_tiles = ops.attention_prefill_shared_tiles(h, hkv, d, small=True)
            if small_tiles:
                # Workgroups of half the size while all of them find room on the chip at
                # once (two on a compute unit): the step then takes as long as the
                # heaviest of them, which has half the queries.  Measured at 28 heads
                # over 4: 2,048 queries in 67 to 77 us against 92, 4,096 the same either way;
                # at 40 over 8: 1,024 in 37 against 48, 2,048 in 118 against 98.
                small_count = int((-(-portions // (QUERY_TILE * small_tiles))).sum())
                # (two workgroups of 8 wavefronts fit on a compute unit)
                if small_count * hkv <= 2 * compute_units():
                    plan.small, tiles = True, small_tiles
            seqs, q0 = portion_runs(portions, shape.num_decode, QUERY_TILE * tiles)
            # the keys an entry's last query reads: where its portion starts plus its queries
            keys = shape.starts[seqs] + q0 + QUERY_TILE * tiles
            if s.window or s.chunk:
                keys = np.minimum(keys, reach + QUERY_TILE * tiles)
            order = heavy_first(keys)
            seqs, q0 = seqs[order], q0[order]
            plan.portion_splits = portion_splits(int(seqs.size) * hkv, int(keys.mean()))
            plan.first_token = shape.num_decode
        else:
            plan.kernel = "tiles"
            seqs, q0 = portion_runs(portions, shape.num_decode, QUERY_TILE)
        plan.count = int(seqs.size)
        # what the launches of the portions depend on beyond the step's sizes
        shape.launch_key.append((key, plan.kernel, plan.small, plan.portion_splits, plan.first_token, plan.count))
        tag = ":".join(str(int(x or 0)) for x in key[1:])  # (one list per plan: the plan's key names it)
        plan.seq_name, plan.q0_name = f"attention_seq:{tag}", f"attention_q0:{tag}"
        shape.add(plan.seq_name, seqs)
        shape.add(plan.q0_name, q0)

    def attend(self, ctx, qkv, out, tables, cache) -> None:
        """Attention of every token of the step over its sequence's cache."""
        s = self.spec
        h, hkv, d = s.num_heads, s.num_kv_heads, s.head_dim
        plan = ctx.notes.get(self.plan_key)
        if plan is None:
            raise RuntimeError(f"{self.name}: the step was not prepared for this mixer "
                               "(the step function calls prepare() on every part)")
        q = qkv[:, : h * d]
        if plan.kernel == "talking_mfma":
            floats = ops.attention_talking_mfma_scratch_floats(q.shape[0], h, hkv, self.value_dim, ctx.num_decode,
                                                               plan.nsplit)
            scratch = ctx.buffer("attn_talking_sums", (floats,), torch.float32)
            ops.attention_talking_mfma(q, out, ctx.num_decode, h, hkv, d, self.value_dim, ctx.positions, ctx.token_seq,
                                       ctx.cu_q, ctx.extras[plan.seq_name] if plan.count else None,
                                       ctx.extras[plan.q0_name] if plan.count else None, plan.count, tables,
                                       cache.pools["k"], cache.pools["v"], cache.page_size, s.window, s.scale, scratch,
                                       chunk=s.chunk, r1=self.r1, r2=self.r2, talk=self.talk,
                                       sink=getattr(s, "fixed_sink", None), nsplit=plan.nsplit)
            return
        if self.talking:
            floats = ops.attention_talking_scratch_floats(q.shape[0], h, self.value_dim, plan.nsplit)
            scratch = ctx.buffer("attn_talking_scratch", (floats,), torch.float32)
            ops.attention_talking(q, out, h, hkv, d, self.value_dim, ctx.positions, ctx.token_seq, tables,
                                  cache.pools["k"], cache.pools["v"], cache.page_size, s.window, s.scale, scratch,
                                  chunk=s.chunk, r1=self.r1, r2=self.r2, talk=self.talk,
                                  sink=getattr(s, "fixed_sink", None), nshare=plan.nsplit)
            return
        if not plan.mfma:
            ops.attention(q, out, h, hkv, d, ctx.positions, ctx.token_seq, tables, cache.pools["k"],
                          cache.pools["v"], cache.page_size, s.window, s.scale, chunk=s.chunk,
                          v_dim=self.value_dim, softcap=getattr(s, "softcap", None), sinks=self.sinks,
                          dist_bias=self.dist_bias)
            return
        if ctx.num_decode:
            partial = ctx.buffer("attn_partial", (ctx.num_decode * h * plan.nsplit * (d + 2),),
                                 torch.float32)
            ops.attention_decode(q, out, ctx.num_decode, h, hkv, d, ctx.positions, tables,
                                 cache.pools["k"], cache.pools["v"], cache.page_size, s.window, s.scale,
                                 partial, plan.nsplit, plan.streaming, chunk=s.chunk,
                                 softcap=getattr(s, "softcap", None), sinks=self.sinks, dist_bias=self.dist_bias)
        if plan.kernel == "shared":
            partial = None
            if plan.portion_splits > 1:
                prompt_tokens = ctx.num_tokens - plan.first_token
                partial = ctx.buffer("attn_portion_partial",
                                     (prompt_tokens * h * plan.portion_splits * (d + 2),), torch.float32)
            ops.attention_prefill_shared(q, out, plan.count, h, hkv, d, ctx.cu_q, ctx.ctx_lens,
                                         ctx.extras[plan.seq_name], ctx.extras[plan.q0_name], tables,
                                         cache.pools["k"], cache.pools["v"], cache.page_size, s.window,
                                         s.scale, small=plan.small, partial=partial,
                                         nsplit=plan.portion_splits, first_token=plan.first_token,
                                         chunk=s.chunk, softcap=getattr(s, "softcap", None), sinks=self.sinks,
                                         dist_bias=self.dist_bias)
        elif plan.kernel == "tiles":
            ops.attention_prefill(q, out, plan.count, h, hkv, d, ctx.cu_q, ctx.ctx_lens,
                                  ctx.extras[plan.seq_name], ctx.extras[plan.q0_name], tables,
                                  cache.pools["k"], cache.pools["v"], cache.page_size, s.window, s.scale,
                                  chunk=s.chunk)

    def _qkv_width(self) -> int:
        s = self.spec
        if self.shared_kv:
            return s.num_heads * s.head_dim
        if s.values_from_keys:
            return (s.num_heads + s.num_kv_heads) * s.head_dim
        return (s.num_heads + s.num_kv_heads) * s.head_dim + s.num_kv_heads * self.value_dim

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        s = self.spec
        n = x.shape[0]
        qkv_width = self._qkv_width()
        if self.plain_store:
            qk_norm = getattr(s, "qk_norm", None)
            if self.shared_kv == cache.owned:
                raise RuntimeError(f"{self.name}: a layer without keys and values of its own must read another "
                                   "run's cache, and only such a layer may")
            qkv = ctx.buffer("attn_qkv", (n, qkv_width), ctx.dtype)
            self.linear(x, self.w_qkv, qkv)
            tables = ctx.block_tables[cache.group]
            ops.qkv_store(qkv, s.num_heads, s.num_kv_heads, s.head_dim, self.value_dim, ctx.positions,
                          ctx.token_seq, tables, cache.pools["k"], cache.pools["v"], cache.page_size,
                          q_temperature=getattr(s, "query_temperature", None),
                          v_norm_eps=getattr(s, "value_norm_eps", None), write_kv=cache.owned,
                          qk_norm_eps=qk_norm[0] if qk_norm else None, q_weight=self.q_norm, k_weight=self.k_norm,
                          has_kv=not self.shared_kv)
            attn = ctx.buffer("attn_out", (n, s.num_heads * self.value_dim), ctx.dtype)
            self.attend(ctx, qkv, attn, tables, cache)
            return self.linear_deferred(ctx, "attn_proj", attn, self.w_o, bias=self.b_o)
        table = self.position.rotary_table() if self.position is not None else None
        fused_position = self.position is None or table is not None
        split_sum = None
        if fused_position:
            # the cache-write kernel can take the projections as partial sums
            qkv = self.linear_deferred(ctx, "attn_qkv_sum", x, self.w_qkv, bias=self.b_qkv,
                                       reader="position")
            if isinstance(qkv, ops.SplitSum):
                split_sum, qkv = qkv, ctx.buffer("attn_qkv", (n, qkv_width), ctx.dtype)
        else:
            qkv = ctx.buffer("attn_qkv", (n, qkv_width), ctx.dtype)
            self.linear(x, self.w_qkv, qkv, bias=self.b_qkv)
            self.position.apply(ctx, qkv, s.num_heads, s.num_kv_heads, s.head_dim)
        inv_freq, rot_dim = table if table is not None else (None, 0)
        tables = ctx.block_tables[cache.group]
        ops.rope_kv_store(
            qkv, s.num_heads, s.num_kv_heads, s.head_dim, rot_dim, inv_freq, ctx.positions,
            ctx.token_seq, tables, cache.pools["k"], cache.pools["v"], cache.page_size,
            write_kv=cache.owned, split_sum=split_sum,
            adjacent_pairs=bool(table is not None and getattr(self.position, "adjacent_pairs", False)),
            values_from_keys=s.values_from_keys,
        )
        attn = ctx.buffer("attn_out", (n, s.num_heads * s.head_dim), ctx.dtype)
        self.attend(ctx, qkv, attn, tables, cache)
        # the norm that follows adds the output to the residual stream and can add up parts
        return self.linear_deferred(ctx, "attn_proj", attn, self.w_o, bias=self.b_o)


register_mixer("paged_attention", PagedAttention)
