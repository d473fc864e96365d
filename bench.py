"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--shape 7b]
    python bench.py --shape 14b --mixed 32      # a mixed step instead (a line of its own)

The model has the layer sizes of the Qwen2.5-7B shape (28 layers, hidden 3584,
28 query heads over 4 key/value heads of 128, intermediate 18944, vocabulary
152064) with random weights in bfloat16.  A "step" is one decode step of
the whole serving path (LLMEngine.step: schedule, forward from the paged cache,
sample, book-keeping) for `batch` requests that were each prefilled with 2,048
random tokens; decoding runs towards context 4,096 (`--context N` starts it at
N tokens instead).  One JSON line is printed: `value` is decoded tokens per
second; `prefill` is a 2,048-token prompt in one step; `roofline` prices the
decode step's unavoidable HBM reads (every weight once, the live requests'
cache) against 8 TB/s, and against the bandwidth that a plain device copy
reaches on this GPU (`achievable`); `prefill.achievable_frac` prices the prompt
against the rate of the engine's own 4096^3 product; `points` holds batch 1 and
64, the same batches at a context near 4,000, a 2,048-token prompt taken in
portions under the reference's 512-token budget, batch 8 at a context of 16,000,
and, with the layer sizes of two larger published models (`config.points_shapes`),
a step of 32 decodes beside a prompt portion (14B) and decode at batch 64 (32B);
`breakdown_us` is the decode step's time by kernel, from events around every
launch of a step that runs kernel by kernel.  The larger models' points are left
out when the run has already taken two minutes.
"""

from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Qwen2.5-7B shape
# layer sizes: the config.json files that the package ships as data
def _shape(name: str) -> dict:
    from shrike_amd.config.presets import load_preset

    return load_preset(f"qwen2.5-{name}")


SHAPE_NAMES = ("0.5b", "7b", "14b", "32b")
PROMPT_LEN = 2048
CONTEXT_END = 4096
PAGE_SIZE = 16
HBM_PEAK_GBS = 8000.0
BF16_PEAK_FLOPS = 2.5e15


def matmul_params(cfg) -> tuple[int, int]:
    """(elements of all per-layer matrices, elements of the output matrix)."""
    h, d = cfg.hidden_size, cfg.head_dim
    if getattr(cfg, "layer_elements", None) is not None:  # a design with other matrices per layer
        return cfg.layer_elements * cfg.num_hidden_layers, cfg.vocab_size * h
    per_layer = (
        (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h
        + cfg.num_attention_heads * d * h
        + 3 * h * cfg.intermediate_size
    )
    return per_layer * cfg.num_hidden_layers, cfg.vocab_size * h


def kv_bytes_per_token(cfg) -> int:
    if getattr(cfg, "kv_elements_per_token", None) is not None:  # a design whose layers cache other things
        return cfg.kv_elements_per_token * 2
    return cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * cfg.head_dim * 2


def prefill_flops(cfg, n: int) -> float:
    layers, head = matmul_params(cfg)
    linear = 2.0 * n * layers + 2.0 * head  # the output matrix runs on one row
    # causal attention: token p reads p + 1 keys, 2 products of head_dim each per head
    attn_layers = getattr(cfg, "attention_layers", cfg.num_hidden_layers)
    attn = 4.0 * cfg.head_dim * cfg.num_attention_heads * attn_layers * n * (n + 1) / 2
    return linear + attn


def run_offline(cfg, spec, requests: int, seed: int) -> dict:
    """The reference's offline throughput run (bench/bench_engine.py:47-63, lengths as
    bench/workload.py:15-22): `requests` short prompts, 32 to 256 new tokens each, greedy,
    all handed to generate() at once, the engine with its defaults (512-token budget,
    prefix caching on).  The prompts are random ids of 24 to 72 tokens instead of the
    reference's sentences."""
    import torch

    from shrike_amd import SamplingParams
    from shrike_amd.config import EngineConfig
    from shrike_amd.engine.llm_engine import LLMEngine
    from shrike_amd.engine.loading import random_model

    model, runtime = random_model(spec, seed=seed, dtype="bfloat16")
    rng = random.Random(seed)
    prompts = [[rng.randrange(cfg.vocab_size) for _ in range(rng.randint(24, 72))] for _ in range(requests)]
    sampling = [SamplingParams(max_new_tokens=rng.randint(32, 256), ignore_eos=True) for _ in range(requests)]
    defaults = EngineConfig(dtype="bfloat16", seed=seed)
    pages = requests * (-(-(72 + 256) // defaults.block_size) + 1)
    engine = LLMEngine(None, EngineConfig(dtype="bfloat16", seed=seed, num_kv_blocks=pages), model=model,
                       runtime=runtime)
    engine.generate(prompts[:4], SamplingParams(max_new_tokens=4, ignore_eos=True), chat=False)  # first launches
    torch.cuda.synchronize()
    steps_before = engine.metrics()["steps"]
    t0 = time.perf_counter()
    outputs = engine.generate(prompts, sampling, chat=False)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    tokens = sum(len(o) for o in outputs)
    assert [len(o) for o in outputs] == [s.max_new_tokens for s in sampling]
    m = engine.metrics()
    return {"tokens": tokens, "seconds": round(seconds, 4), "tok_s": round(tokens / seconds, 1),
            "steps": m["steps"] - steps_before, "preemptions": m["preemptions"],
            "prefix_cache_hit_rate": m["prefix_cache_hit_rate"], "max_running": defaults.max_running,
            "token_budget": defaults.max_tokens_per_step, "page_size": defaults.block_size}


def make_engine(cfg, spec, max_batch: int, seed: int, budget: int | None = None):
    import torch

    from shrike_amd.config import EngineConfig
    from shrike_amd.engine.llm_engine import LLMEngine
    from shrike_amd.engine.loading import random_model

    t0 = time.perf_counter()
    model, runtime = random_model(spec, seed=seed, dtype="bfloat16")
    torch.cuda.synchronize()
    print(f"[bench] random weights on the device in {time.perf_counter() - t0:.1f}s", file=sys.stderr)
    pages = max_batch * (CONTEXT_END // PAGE_SIZE + 2)
    config = EngineConfig(
        block_size=PAGE_SIZE, num_kv_blocks=pages,
        # a whole prompt, of any context this program asks for, beside every running request's token
        max_tokens_per_step=budget if budget is not None else CONTEXT_END + max_batch,
        max_running=max_batch, enable_prefix_caching=False, dtype="bfloat16", seed=seed,
    )
    return LLMEngine(None, config, model=model, runtime=runtime)


def run_decode(engine, cfg, batch: int, steps: int, warmup: int, seed: int,
               prompt_len: int = PROMPT_LEN, temperature: float = 0.0, top_p: float = 1.0) -> dict:
    """Prefill `batch` prompts of `prompt_len` tokens, then time `steps` decode steps."""
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed)
    # the first requests decode while the later ones' prompts are taken in, portion by portion
    prefill_steps = batch * -(-prompt_len // engine.scheduler.max_tokens_per_step)
    sampling = SamplingParams(max_new_tokens=prefill_steps + batch + warmup + steps + 8, ignore_eos=True,
                              temperature=temperature, top_p=top_p)
    for _ in range(batch):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(prompt_len)], sampling)
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        engine.step()
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    context_start = sum(r.num_computed_tokens for r in engine.scheduler.running) / batch
    t0 = time.perf_counter()
    produced = 0
    for _ in range(steps):
        produced += len(engine.step())
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    context_end = sum(r.num_computed_tokens for r in engine.scheduler.running) / batch
    assert produced == batch * steps, f"{produced} tokens from {steps} steps of {batch}"
    for req in list(engine.scheduler.running):
        engine.abort(req.req_id)
    layer_w, head_w = matmul_params(cfg)
    mean_ctx = (context_start + context_end) / 2 + 1
    # (a design with recurrent layers reads and writes each request's state once a step)
    step_bytes = (2.0 * (layer_w + head_w) + batch * mean_ctx * kv_bytes_per_token(cfg)
                  + batch * getattr(cfg, "state_bytes_per_seq", 0))
    ms = elapsed / steps * 1e3
    return {
        "tok_s": produced / elapsed, "ms_per_step": ms, "context_start": context_start,
        "context_end": context_end, "step_bytes": step_bytes,
        "gb_s": step_bytes / (ms * 1e-3) / 1e9,
    }


def run_chunked_prefill(engine, cfg, seed: int, budget: int = 512, prompt_len: int = PROMPT_LEN) -> float:
    """Milliseconds until a prompt of `prompt_len` tokens has its first token when the
    scheduler cuts it into portions of `budget` tokens (the reference's default: 512)."""
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed + 3)
    saved, engine.scheduler.max_tokens_per_step = engine.scheduler.max_tokens_per_step, budget
    best = None
    try:
        for _ in range(2):
            engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(prompt_len)],
                               SamplingParams(max_new_tokens=1, ignore_eos=True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            steps = 0
            while engine.has_work:
                engine.step()
                steps += 1
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            assert steps == -(-prompt_len // budget)
            best = dt if best is None else min(best, dt)
    finally:
        engine.scheduler.max_tokens_per_step = saved
    return best * 1e3


def other_shapes(args, started: float, limit: float = 120.0) -> tuple[dict, str]:
    """Points with the layer sizes of larger published models, each skipped once the
    whole run has taken `limit` seconds: a step of 32 decodes beside a portion of a
    2,048-token prompt under a 512-token budget (14B), decode at batch 64 (32B)."""
    import torch

    from shrike_amd.models.qwen2 import Qwen2Config, build_spec

    points, named = {}, []
    for shape, what in (("14b", "mixed"), ("32b", "decode")):
        if time.perf_counter() - started > limit:
            print(f"[bench] {shape} point skipped: the run has taken {time.perf_counter() - started:.0f}s", file=sys.stderr)
            continue
        cfg = Qwen2Config.from_dict(_shape(shape))
        spec = build_spec(cfg)
        named.append(f"{shape}: {cfg.num_hidden_layers} layers, hidden {cfg.hidden_size}, {cfg.num_attention_heads} heads "
                     f"over {cfg.num_key_value_heads} of {cfg.head_dim}, intermediate {cfg.intermediate_size}")
        if what == "mixed":
            engine = make_engine(cfg, spec, 33, args.seed, budget=512)
            mixed = run_mixed(engine, cfg, 32, 512, args.seed)
            points["mixed_14b_ms"] = mixed["mixed_step_ms"]
            points["decode_b32_14b_ms"] = mixed["decode_only_ms"]
            print(f"[bench] 14B sizes, 32 decodes + a portion under a 512-token budget: {mixed}", file=sys.stderr)
        else:
            engine = make_engine(cfg, spec, 64, args.seed)
            run = run_decode(engine, cfg, 64, min(args.steps, 40), args.warmup, args.seed + 64)
            points["decode_b64_32b"] = round(run["tok_s"], 1)
            points["decode_b64_32b_hbm_frac"] = round(run["gb_s"] / HBM_PEAK_GBS, 4)
            print(f"[bench] 32B sizes, batch 64: {run['tok_s']:.1f} tok/s, {run['ms_per_step']:.3f} ms/step, "
                  f"{run['gb_s']:.0f} GB/s", file=sys.stderr)
        del engine
        torch.cuda.empty_cache()
    return points, "; ".join(named)


def run_prefill(engine, cfg, seed: int, repeats: int = 3) -> dict:
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed + 1)
    best = None
    for _ in range(repeats):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(PROMPT_LEN)],
                           SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(outs) == 1 and outs[0].finished
        best = dt if best is None else min(best, dt)
    flops = prefill_flops(cfg, PROMPT_LEN)
    return {"value": round(PROMPT_LEN / best, 1), "tokens": PROMPT_LEN, "ms": round(best * 1e3, 3),
            "frac": round(flops / best / BF16_PEAK_FLOPS, 4)}


def measure_peaks(device="cuda:0") -> dict:
    """What this GPU reaches on the plainest work of each kind: bytes per second
    of a device-to-device copy of 2 GiB (read + write), of a read-only stream
    (the engine's one-row product with a 1 GiB matrix), and flop/s of the engine's own bfloat16 product
    at 4096 x 4096 x 4096."""
    import torch

    from shrike_amd.kernels import ops

    out = {}
    src = torch.empty(1 << 30, dtype=torch.bfloat16, device=device).normal_()
    dst = torch.empty_like(src)

    def timed(fn, repeats):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(repeats):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / repeats * 1e-3

    nbytes = src.numel() * 2
    out["copy_gbs"] = round(2 * nbytes / timed(lambda: dst.copy_(src), 5) / 1e9, 1)
    del src, dst
    # a read-only stream: the engine's own product of one row with a 1 GiB matrix
    rows, width = 131072, 4096
    big = ops.retile_weight(torch.empty(rows, width, dtype=torch.bfloat16, device=device).normal_())
    x = torch.randn(1, width, device=device).to(torch.bfloat16)
    y = torch.empty(1, rows, dtype=torch.bfloat16, device=device)
    out["read_gbs"] = round(rows * width * 2 / timed(lambda: ops.gemm_tiled_weight(x, big, rows, width, y), 5) / 1e9, 1)
    del big
    # the matrix units alone on random operands: the power limit's ceiling for every product
    operands = torch.randn(32768, device=device).to(torch.bfloat16)
    flop = ops.mfma_alone(operands, 2048, 2048)
    out["mfma_tflops"] = round(flop / timed(lambda: ops.mfma_alone(operands, 2048, 2048), 3) / 1e12, 1)
    n = 4096
    a = torch.randn(n, n, device=device).to(torch.bfloat16)
    wt = ops.retile_weight(torch.randn(n, n, device=device).to(torch.bfloat16))
    c = torch.empty(n, n, dtype=torch.bfloat16, device=device)
    out["gemm_tflops"] = round(2.0 * n**3 / timed(lambda: ops.gemm_tiled_weight(a, wt, n, n, c), 10) / 1e12, 1)
    return out


def kernel_breakdown(engine, steps: int = 3, before_step=None) -> dict:
    """Microseconds per step by kernel: the running requests' next steps run kernel by
    kernel (no graph) with an event before and after every launch.  `before_step()` is
    called ahead of every step (to add the prompt that the step is to take in)."""
    import torch

    from shrike_amd.kernels import ops

    names = ["embed", "add_rmsnorm", "act_mul", "gemm", "gemm_tiled_weight", "rope_kv_store", "attention",
             "attention_decode", "attention_prefill", "attention_prefill_shared", "argmax", "sample",
             "add_deltas", "add_normed_rmsnorm", "act_mul_rows", "add_rows", "embed_pairs", "qkv_store",
             "latent_prepare", "rotate_heads", "latent_attention", "latent_attention_mfma", "gemm_batched", "mlstm_scan", "headnorm_gate",
             "xielu", "layernorm", "add_layernorm", "attention_talking", "attention_talking_mfma", "conv_silu", "dt_softplus", "selective_scan",
             "rotate_half_rows", "retention_scan", "moe_route", "moe_experts", "mix_history", "scale_softcap",
             "postnorm", "cast_rows", "activate", "gate_mul"]
    names = [n for n in names if hasattr(ops, n)]
    spans: list[tuple[str, object, object]] = []
    saved = {n: getattr(ops, n) for n in names}

    def wrap(name, fn):
        def timed(*args, **kwargs):
            label = name
            if name == "gemm_tiled_weight":  # told apart by the matrix: [m, k]
                label = f"gemm {args[2]}x{args[3]}" + (" gated" if kwargs.get("gated") else "")
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            out = fn(*args, **kwargs)
            b.record()
            spans.append((label, a, b))
            return out
        return timed

    runner = engine.runner
    # no step may be in flight or planned from before: the next ones are to run kernel by kernel
    overlap, engine.config.overlap_steps = engine.config.overlap_steps, False
    engine.step()  # takes in the step that was launched ahead, if one was, and launches none
    graphs, runner.use_graphs = runner.use_graphs, False
    lists, runner.use_call_lists = runner.use_call_lists, False
    engine._planned = None
    try:
        for n, fn in saved.items():
            setattr(ops, n, wrap(n, fn))
        if before_step is not None:
            before_step()
        engine.step()  # buffers of the kernel-by-kernel path
        spans.clear()
        for _ in range(steps):
            if before_step is not None:
                before_step()
            # the device is held back while the host queues the step's launches and
            # events, so that an event pair brackets its kernel and not the host's pace
            torch.cuda.synchronize()
            torch.cuda._sleep(30_000_000)
            engine.step()
        torch.cuda.synchronize()
    finally:
        for n, fn in saved.items():
            setattr(ops, n, fn)
        runner.use_graphs = graphs
        runner.use_call_lists = lists
        engine.config.overlap_steps = overlap
        engine._planned = None
    total: dict[str, float] = {}
    for label, a, b in spans:
        total[label] = total.get(label, 0.0) + a.elapsed_time(b) * 1e3 / steps
    return {k: round(v, 1) for k, v in sorted(total.items(), key=lambda kv: -kv[1])}


def mofarax_like(qcfg, mask_size: int, side_dim: int):
    """A Mofarax configuration with the layer sizes of a Qwen2 one (same width, heads,
    head size, feed-forward width, vocabulary and number of layers; heads rotated whole;
    the loop runs all layers once, so that the two models run layer for layer), and an
    object that names its sizes as the formulas of this program expect them."""
    from types import SimpleNamespace

    from shrike_amd.models.mofarax import MofaraxAttention, MofaraxConfig, MofaraxLayer

    mixer = MofaraxAttention(heads=qcfg.num_attention_heads, kv_heads=qcfg.num_key_value_heads, dim=qcfg.head_dim,
                             vdim=qcfg.head_dim, scale=qcfg.head_dim**-0.5, mask_size=mask_size,
                             rot_base=qcfg.rope_theta, rot_dims=qcfg.head_dim)
    layers = tuple(MofaraxLayer(mixer, qcfg.intermediate_size) for _ in range(qcfg.num_hidden_layers))
    mcfg = MofaraxConfig(vocab=qcfg.vocab_size, width=qcfg.hidden_size, embedding_scale=8.0,
                         norm_eps=qcfg.rms_norm_eps, layers=layers, side_dim=side_dim,
                         loop=(0, qcfg.num_hidden_layers, 1))
    h, d = qcfg.hidden_size, qcfg.head_dim
    sizes = SimpleNamespace(
        hidden_size=h, head_dim=d, num_attention_heads=qcfg.num_attention_heads,
        num_key_value_heads=qcfg.num_key_value_heads, intermediate_size=qcfg.intermediate_size,
        num_hidden_layers=qcfg.num_hidden_layers, vocab_size=qcfg.vocab_size,
        # no value projection; the side input's two matrices
        layer_elements=(2 * qcfg.num_attention_heads + qcfg.num_key_value_heads) * d * h
        + 3 * h * qcfg.intermediate_size + 2 * side_dim * h)
    return mcfg, sizes


def minilorn_like(qcfg, window: int, pattern: str):
    """A Minilorn configuration with the layer sizes of a Qwen2 one (same width, feed-forward
    width, vocabulary and number of layers): attention layers with Qwen2's heads (values as
    large as keys); latent attention with as many heads, a query latent of 3/8 and a key/value
    latent of 1/8 of the width (rounded to 64) and half a head rotated; matrix memories of
    width / 512 heads with 256 query/key and 512 value elements; `pattern` says which mixer
    each layer has, letter by letter (a, l, m), repeated.  With it an object that names the
    sizes as the formulas of this program expect them."""
    from types import SimpleNamespace

    from shrike_amd.models.minilorn import (LatentAttention, MatrixMemory, MinilornConfig, MinilornLayer,
                                            SinkAttention)

    h, d, H = qcfg.hidden_size, qcfg.head_dim, qcfg.num_attention_heads
    up64 = lambda x: max(64, -(-int(x) // 64) * 64)  # noqa: E731
    mixers = {
        "a": ("attention", SinkAttention(heads=H, kv_heads=qcfg.num_key_value_heads, dim=d, vdim=d, scale=d**-0.5,
                                         softcap=30.0, q_temp=(0.25, 256))),
        "l": ("latent_attention", LatentAttention(heads=H, dim=d, rot_dim=d // 2, vdim=d, q_rank=up64(3 * h / 8),
                                                   kv_rank=up64(h / 8), scale=(1.5 * d) ** -0.5, rot_base=10000.0,
                                                   window=window, rot_dims=d // 2)),
        "m": ("mlstm", MatrixMemory(heads=max(1, h // 512), dim=256, vdim=512, gate_cap=15.0)),
    }
    kinds = [mixers[pattern[i % len(pattern)]] for i in range(qcfg.num_hidden_layers)]
    layers = tuple(MinilornLayer(kind, mixer, qcfg.intermediate_size) for kind, mixer in kinds)
    mcfg = MinilornConfig(vocab=qcfg.vocab_size, width=h, norm_eps=qcfg.rms_norm_eps, layers=layers,
                          bigram=(65521, 31, 17))
    la, mm = mixers["l"][1], mixers["m"][1]
    elements = {
        "attention": 2 * (H + qcfg.num_key_value_heads) * d * h,
        "latent_attention": (la.q_rank + la.kv_rank + la.rot_dim) * h + H * (d + la.rot_dim) * la.q_rank
        + 2 * H * d * la.kv_rank + H * d * h,
        "mlstm": (2 * mm.heads * mm.dim + 3 * mm.heads * mm.vdim + 2 * mm.heads) * h,
    }
    cached = {"attention": 2 * qcfg.num_key_value_heads * d, "latent_attention": la.kv_rank + la.rot_dim, "mlstm": 0}
    n = len(kinds)
    sizes = SimpleNamespace(
        hidden_size=h, head_dim=d, num_attention_heads=H, num_key_value_heads=qcfg.num_key_value_heads,
        intermediate_size=qcfg.intermediate_size, num_hidden_layers=n, vocab_size=qcfg.vocab_size,
        layer_elements=sum(elements[k] for k, _ in kinds) // n + 2 * h * qcfg.intermediate_size,
        kv_elements_per_token=sum(cached[k] for k, _ in kinds))
    return mcfg, sizes


def ligipel_like(qcfg, window: int, pattern: str, experts: int, top: int):
    """A Ligipel configuration with the layer sizes of a Qwen2 one (same width, vocabulary and
    number of layers).  `pattern` says which mixer each layer has, letter by letter, repeated:
    p, attention with Qwen2's heads (sliding window `window`) beside a selective scan of
    `width` channels with 16 states, 4 taps and a step-size rank of width / 16; r, retention
    with width / 256 heads of 128 query/key and 256 value elements.  Every layer has `experts`
    routed experts of which a token uses `top`, and a shared one half as wide as Qwen2's
    feed-forward; the chosen experts together are the other half.  With it an object that
    names the sizes as the formulas of this program expect them; its `at_batch(b)` sets the
    matrices' elements that a step of b tokens reads (the experts that b tokens are expected
    to touch when the router spreads them evenly)."""
    from types import SimpleNamespace

    from shrike_amd.models.ligipel import (BiasedAttention, DecayedRetention, LigipelConfig, LigipelLayer, Mixture,
                                           Scan, SideBySide)

    h, d, H, KV = qcfg.hidden_size, qcfg.head_dim, qcfg.num_attention_heads, qcfg.num_key_value_heads
    inter = qcfg.intermediate_size
    ff = max(64, inter // (2 * top) // 64 * 64)
    shared = inter // 2
    scan = Scan(inner=h, state=16, dt_rank=max(1, h // 16), conv=4)
    rheads = max(1, h // 256)
    mixers = {
        "p": ("parallel", SideBySide(left=BiasedAttention(heads=H, kv_heads=KV, dim=d, vdim=d, scale=d**-0.5,
                                                          window=window), right=scan)),
        "r": ("retention", DecayedRetention(heads=rheads, dim=128, vdim=256,
                                            decay=tuple(1.0 - 2.0 ** (-5 - i % 8) for i in range(rheads)),
                                            rot_base=10000.0, rot_dims=64)),
    }
    kinds = [mixers[pattern[i % len(pattern)]] for i in range(qcfg.num_hidden_layers)]
    mlp = Mixture(experts=experts, top=top, ff=ff, shared_ff=shared)
    lcfg = LigipelConfig(vocab=qcfg.vocab_size, width=h, norm_eps=qcfg.rms_norm_eps,
                         layers=tuple(LigipelLayer(kind, mixer, mlp) for kind, mixer in kinds),
                         logit_scale=1.0, logit_softcap=30.0)
    n = len(kinds)
    elements = {
        "parallel": 2 * (H + KV) * d * h + 3 * scan.inner * h + (scan.dt_rank + 2 * scan.state) * scan.inner
        + scan.inner * scan.dt_rank * 2,  # (the step-size matrix is float32)
        "retention": (2 * rheads * 128 + 3 * rheads * 256) * h,
    }
    states = {"parallel": scan.inner * (scan.state + scan.conv - 1), "retention": rheads * 128 * 256}
    mixer_elements = sum(elements[k] for k, _ in kinds) // n
    sizes = SimpleNamespace(
        hidden_size=h, head_dim=d, num_attention_heads=H, num_key_value_heads=KV, intermediate_size=inter,
        num_hidden_layers=n, vocab_size=qcfg.vocab_size, attention_layers=sum(k == "parallel" for k, _ in kinds),
        kv_elements_per_token=sum(2 * KV * d for k, _ in kinds if k == "parallel"),
        state_bytes_per_seq=2 * 4 * sum(states[k] for k, _ in kinds))

    def at_batch(b: int) -> None:
        touched = experts * (1.0 - (1.0 - top / experts) ** b)
        sizes.layer_elements = int(mixer_elements + experts * h + 3 * h * shared + touched * 3 * h * ff)

    sizes.at_batch = at_batch
    # a prompt: every token's own experts are work, whichever matrices hold them
    sizes.layer_elements = mixer_elements + experts * h + 3 * h * shared + top * 3 * h * ff
    return lcfg, sizes


def poresun_like(qcfg, window: int, pattern: str, experts: int, top: int):
    """A Poresun configuration with the layer sizes of a Qwen2 one (same width, vocabulary and
    number of layers).  `pattern` says which mixer each layer has, letter by letter, repeated:
    a, attention with Qwen2's heads, unweighted norms of queries and keys, a cap, a bias table
    of 32 rows that reaches 4,096 positions and a sliding window `window`; b, the causal
    attention with weighted norms, a query temperature and the same table; s, such a layer
    that reads the keys and values of the last b layer before it; l, latent attention with as
    many heads, a query latent of 3/8 and a key/value latent of 1/8 of the width (rounded to
    64, at most 512), half a head rotated, and the output gate.  The first layer of every repetition has the
    bounded gated feed-forward as wide as Qwen2's; the others `experts` routed experts without
    gates of which a token uses `top` (together half of Qwen2's feed-forward's multiply-adds)
    and a gated shared expert of the other half.  With it an object that names the sizes as the
    formulas of this program expect them (see ligipel_like)."""
    from types import SimpleNamespace

    from shrike_amd.models.poresun import (BoundedDense, BucketAttention, GatedLatentAttention, PoresunConfig,
                                           PoresunLayer, UngatedMixture)

    h, d, H, KV = qcfg.hidden_size, qcfg.head_dim, qcfg.num_attention_heads, qcfg.num_key_value_heads
    inter = qcfg.intermediate_size
    up64 = lambda x: max(64, -(-int(x) // 64) * 64)  # noqa: E731
    # an expert has two matrices where Qwen2's feed-forward has three
    ff = max(64, 3 * inter // (4 * top) // 64 * 64)
    shared = up64(3 * inter / 4)
    # (a key/value latent of at most 512: with the rotated part a cached row of at most 640 elements, which the
    # latent attention's kernel on the matrix units takes)
    latent = GatedLatentAttention(heads=H, dim=d, rot_dim=d // 2, vdim=d, q_rank=up64(3 * h / 8),
                                  kv_rank=min(up64(h / 8), 512), scale=(1.5 * d) ** -0.5, rot_base=10000.0,
                                  rot_dims=d // 2)
    layers, last_b = [], None
    for i in range(qcfg.num_hidden_layers):
        letter = pattern[i % len(pattern)]
        if letter == "s" and last_b is None:
            letter = "b"
        if letter == "a":
            kind, mixer = "attention", BucketAttention(heads=H, kv_heads=KV, dim=d, vdim=d, scale=d**-0.5, bias_max=4096,
                                                       weighted_norm=False, window=window, softcap=30.0, bias_rows=32)
        elif letter in "bs":
            kind, mixer = "attention_2", BucketAttention(heads=H, kv_heads=KV, dim=d, vdim=d, scale=d**-0.5, bias_max=4096,
                                                         weighted_norm=True, q_temp=(0.25, 256), bias_rows=32,
                                                         kv_from=last_b if letter == "s" else None)
            last_b = i if letter == "b" else last_b
        elif letter == "l":
            kind, mixer = "latent_attention", latent
        else:
            raise SystemExit(f"--pattern: unknown letter {letter!r} for --poresun (a, b, s, l)")
        mlp = BoundedDense(ff=inter, limit=7.0) if i % len(pattern) == 0 else \
            UngatedMixture(experts=experts, top=top, ff=ff, shared_ff=shared)
        layers.append((letter, PoresunLayer(kind, mixer, mlp)))
    pcfg = PoresunConfig(vocab=qcfg.vocab_size, width=h, norm_eps=qcfg.rms_norm_eps, alpha=2.0,
                         layers=tuple(layer for _, layer in layers), embedding_scale=float(h) ** 0.5)
    n = len(layers)
    mixer_elements = {
        "a": 2 * (H + KV) * d * h, "b": 2 * (H + KV) * d * h, "s": 2 * H * d * h,
        "l": (latent.q_rank + latent.kv_rank + latent.rot_dim) * h + H * (d + latent.rot_dim) * latent.q_rank
        + 2 * H * d * latent.kv_rank + 2 * H * d * h,
    }
    cached = {"a": 2 * KV * d, "b": 2 * KV * d, "s": 0, "l": latent.kv_rank + latent.rot_dim}
    dense_layers = sum(isinstance(layer.mlp, BoundedDense) for _, layer in layers)
    mixers = sum(mixer_elements[letter] for letter, _ in layers)
    sizes = SimpleNamespace(
        hidden_size=h, head_dim=d, num_attention_heads=H, num_key_value_heads=KV, intermediate_size=inter,
        num_hidden_layers=n, vocab_size=qcfg.vocab_size, attention_layers=sum(letter != "l" for letter, _ in layers),
        kv_elements_per_token=sum(cached[letter] for letter, _ in layers))

    def elements(per_expert_layer: float) -> int:
        moe = (experts + 1) * h + 2 * h * shared + per_expert_layer
        return int((mixers + dense_layers * 3 * h * inter + (n - dense_layers) * moe) // n)

    def at_batch(b: int) -> None:
        touched = experts * (1.0 - (1.0 - top / experts) ** b)
        sizes.layer_elements = elements(touched * 2 * h * ff)

    sizes.at_batch = at_batch
    sizes.layer_elements = elements(top * 2 * h * ff)  # a prompt: every token's own experts are work
    return pcfg, sizes


def run_designs(args, qcfg) -> dict:
    """Another design beside Qwen2 at equal layer sizes, random weights: a prompt of 2,048
    tokens in one step, decode steps at batch 1, 8 and 64 from that context, and what each
    kernel takes in a decode step at batch 8 and in the prompt's step."""
    import gc

    import torch

    from shrike_amd import SamplingParams
    from shrike_amd.models import ligipel, minilorn, mofarax, poresun, qwen2

    if args.poresun:
        pcfg, psizes = poresun_like(qcfg, args.window, args.pattern if set(args.pattern) <= set("absl") else "absl",
                                    args.experts, args.top)
        other = ("poresun", poresun.build_spec(pcfg), psizes)
    elif args.ligipel:
        lcfg, lsizes = ligipel_like(qcfg, args.window, args.pattern if set(args.pattern) <= set("pr") else "pppr",
                                    args.experts, args.top)
        other = ("ligipel", ligipel.build_spec(lcfg), lsizes)
    elif args.minilorn:
        mcfg, msizes = minilorn_like(qcfg, args.window, args.pattern)
        other = ("minilorn", minilorn.build_spec(mcfg), msizes)
    else:
        mcfg, msizes = mofarax_like(qcfg, args.mask_size, args.side_dim)
        other = ("mofarax", mofarax.build_spec(mcfg), msizes)
    out = {}
    for name, spec, sizes in (("qwen2", qwen2.build_spec(qcfg), qcfg), other):
        if args.design_only and name != args.design_only:
            continue
        engine = make_engine(sizes, spec, 64, args.seed)
        rng = random.Random(args.seed + 5)

        def add_prompt(engine=engine, rng=rng, sizes=sizes):
            engine.add_request([rng.randrange(sizes.vocab_size) for _ in range(PROMPT_LEN)],
                               SamplingParams(max_new_tokens=1, ignore_eos=True))

        res = {"prefill": run_prefill(engine, sizes, args.seed)}
        res["prefill_kernels_us"] = kernel_breakdown(engine, steps=2, before_step=add_prompt)
        for batch in (1, 8, 64):
            if hasattr(sizes, "at_batch"):
                sizes.at_batch(batch)
            d = run_decode(engine, sizes, batch, args.design_steps, args.warmup, args.seed)
            res[f"decode_b{batch}"] = {"tok_s": round(d["tok_s"], 1), "ms_per_step": round(d["ms_per_step"], 3),
                                       "roofline_frac": round(d["gb_s"] / HBM_PEAK_GBS, 3)}
        # the kernels of a decode step at batch 8
        sampling = SamplingParams(max_new_tokens=64, ignore_eos=True)
        for _ in range(8):
            engine.add_request([rng.randrange(sizes.vocab_size) for _ in range(PROMPT_LEN)], sampling)
        while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
            engine.step()
        res["decode_b8_kernels_us"] = kernel_breakdown(engine, steps=3)
        for req in list(engine.scheduler.running):
            engine.abort(req.req_id)
        out[name] = res
        del engine
        gc.collect()
        torch.cuda.empty_cache()
    return out


def run_mixed(engine, cfg, decodes: int, budget: int, seed: int) -> dict:
    """`decodes` requests decoding at a context of about PROMPT_LEN while one more
    PROMPT_LEN-token prompt is admitted under a token budget of `budget` a step:
    the time of the steps that hold `decodes` single tokens and a prompt portion."""
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed)
    sampling = SamplingParams(max_new_tokens=400, ignore_eos=True)
    for _ in range(decodes):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(PROMPT_LEN)], sampling)
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        engine.step()
    for _ in range(20):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(50):
        engine.step()
    torch.cuda.synchronize()
    decode_ms = (time.perf_counter() - t0) / 50 * 1e3
    late = engine.requests[engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(PROMPT_LEN)],
                                              SamplingParams(max_new_tokens=8, ignore_eos=True))]
    full = []  # steps that use the whole budget
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        done = late.num_computed_tokens
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        # (a decode step that was already running when the prompt arrived is not one of them)
        if late.num_computed_tokens - done >= budget - decodes:
            full.append((time.perf_counter() - t0) * 1e3)
    for req in list(engine.scheduler.running):
        engine.abort(req.req_id)
    mean = sum(full) / len(full)
    return {"decode_only_ms": round(decode_ms, 3), "mixed_step_ms": round(mean, 3), "mixed_steps": len(full),
            "tokens_per_s": round(budget / mean * 1e3, 1)}


def run_products(cfg, tokens: list[int]) -> dict:
    """Microseconds of each of a layer's four products (and of the output head) with
    the engine's kernels and, beside them, with the vendor library's matrix product
    (torch.matmul) on the same sizes: a yardstick only, the engine never calls it.
    The engine's gate/up product includes the gate's activation and writes half the
    columns; its products of few tokens include no reader of their shares of k."""
    import statistics

    import torch

    from shrike_amd.kernels import ops

    dev = "cuda:0"

    def graph_us(fn, repeats=5):
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(repeats):
                fn()
        times = []
        for _ in range(5):
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e3 / repeats)
        return statistics.median(times)

    h, inter = cfg.hidden_size, cfg.intermediate_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    shapes = [("qkv", qkv, h, False), ("o", h, cfg.num_attention_heads * cfg.head_dim, False),
              ("gate_up", inter, h, True), ("down", h, inter, False), ("lm_head", cfg.vocab_size, h, False)]
    out = {}
    for n in tokens:
        for name, m, k, gated in shapes:
            if name == "lm_head" and n > 64:
                continue  # the head only ever sees the rows whose logits are wanted
            rows = 2 * m if gated else m
            w = (torch.randn(rows, k, device=dev) * k**-0.5).to(torch.bfloat16)
            x = torch.randn(n, k, device=dev).to(torch.bfloat16)
            y = torch.empty(n, rows, device=dev, dtype=torch.bfloat16)
            library = graph_us(lambda: torch.matmul(x, w.t(), out=y))
            if gated:
                tiled = ops.interleave_gate_up(w[:m].contiguous(), w[m:].contiguous())
            else:
                tiled = ops.retile_weight(w)
            del w
            splits = 1 if gated else ops.gemm_splits(n, m, k)
            z = (torch.empty(splits, n, m, device=dev) if splits > 1
                 else torch.empty(n, m, device=dev, dtype=torch.bfloat16))
            if gated:
                own = graph_us(lambda: ops.gemm_tiled_weight(x, tiled, m, k, z, gated="silu"))
            else:
                own = graph_us(lambda: ops.gemm_tiled_weight(x, tiled, m, k, z, splits=splits))
            out[f"{name}_n{n}"] = {"own_us": round(own, 1), "library_us": round(library, 1), "k_shares": splits}
            print(f"[bench] {n:5d} tokens {name:8s} {rows:6d} x {k:5d}: own {own:7.1f} us ({splits} shares of k), "
                  f"library {library:7.1f} us", file=sys.stderr)
            del tiled, x, y, z
    return out


def main() -> int:
    global CONTEXT_END
    started = time.perf_counter()
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=int(os.environ.get("WORLD_SIZE", "1")))
    ap.add_argument("--steps", type=int, default=1900,
                    help="timed decode steps; 1900 after 2048-token prompts reach context 4,000")
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None,
                    help="run fewer layers than the configuration has (both numbers are reported)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--context", type=int, default=PROMPT_LEN, metavar="N",
                    help="start decoding at a context of N tokens (N-token prompts) instead of 2,048")
    ap.add_argument("--context-end", type=int, default=CONTEXT_END, metavar="N",
                    help="the context length the cache is made for (the configuration's 4,096; more for runs "
                         "at longer contexts)")
    ap.add_argument("--far-context", type=int, default=4000 - 64, metavar="N",
                    help="context of the extra points decode_b*_ctx4000 (0: leave them out)")
    ap.add_argument("--no-peaks", action="store_true",
                    help="skip the measurement of this GPU's copy bandwidth and product rate")
    ap.add_argument("--shape", choices=SHAPE_NAMES, default="7b",
                    help="layer sizes: Qwen2.5-7B (the default and the reported figure), 0.5B, 14B or 32B")
    ap.add_argument("--mixed", type=int, default=0, metavar="DECODES",
                    help="instead: time steps of DECODES single tokens plus a portion of a 2,048-token "
                         "prompt under a 512-token budget (prints its own JSON line)")
    ap.add_argument("--offline", type=int, default=0, metavar="REQUESTS",
                    help="instead: the reference's offline throughput run, REQUESTS short prompts with 32 to "
                         "256 new tokens each through generate() (prints its own JSON line)")
    ap.add_argument("--products", action="store_true",
                    help="instead: time a layer's matrix products at 1 to 2,048 tokens with the engine's kernels "
                         "and, as a yardstick, with the vendor library (prints its own JSON line)")
    ap.add_argument("--mofarax", action="store_true",
                    help="instead of the default run: the Mofarax design beside Qwen2 at the layer sizes of "
                         "--shape, random weights: prompt, decode at batch 1 / 8 / 64, per-kernel times")
    ap.add_argument("--minilorn", action="store_true",
                    help="Minilorn beside Qwen2 at equal layer sizes: prompt, decode at batch 1/8/64, time per kernel")
    ap.add_argument("--ligipel", action="store_true",
                    help="Ligipel beside Qwen2 at equal layer sizes: prompt, decode at batch 1/8/64, time per kernel")
    ap.add_argument("--poresun", action="store_true",
                    help="the Poresun design beside Qwen2 at the layer sizes of --shape, random weights")
    ap.add_argument("--experts", type=int, default=8, metavar="N", help="--ligipel, --poresun: routed experts a layer")
    ap.add_argument("--top", type=int, default=2, metavar="N", help="--ligipel, --poresun: experts a token uses")
    ap.add_argument("--pattern", default="alml", metavar="LETTERS",
                    help="--minilorn: the layers' mixers in order, repeated: a(ttention), l(atent attention), m(atrix memory); "
                         "--ligipel: p(arallel attention and scan), r(etention), default pppr; --poresun: a(ttention "
                         "with a window), b (causal attention), s (reads the last b layer's keys and values), "
                         "l(atent attention), default absl")
    ap.add_argument("--window", type=int, default=4096, metavar="N",
                    help="--minilorn: sliding window of its latent attention (4096: no fewer keys than Qwen2 reads)")
    ap.add_argument("--design-only", choices=["qwen2", "mofarax", "minilorn", "ligipel", "poresun"], default=None,
                    help="--mofarax / --minilorn / --ligipel / --poresun: run only this one of the two (for a profile of "
                         "one model's kernels)")
    ap.add_argument("--mask-size", type=int, default=8192, metavar="N",
                    help="--mofarax: positions per block of its attention (8192: no fewer keys than Qwen2 reads)")
    ap.add_argument("--side-dim", type=int, default=256, metavar="N", help="--mofarax: width of its per-layer token input")
    ap.add_argument("--design-steps", type=int, default=300, metavar="K", help="--mofarax: timed decode steps per batch size")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.steps < 1 or args.warmup < 0 or args.batch < 1:
        print("bench.py: --steps and --batch must be positive, --warmup non-negative")
        return 2
    CONTEXT_END = args.context_end
    if not 1 <= args.context < CONTEXT_END:
        print(f"bench.py: --context must lie in [1, {CONTEXT_END})")
        return 2
    room = CONTEXT_END - args.context - args.warmup - max(args.batch, 1 if args.no_points else 64) - 2
    if args.steps > room:
        print(f"bench.py: at most {room} steps fit between context {args.context} and {CONTEXT_END}")
        return 2

    import torch

    import shrike_amd.models  # noqa: F401
    from shrike_amd.models.qwen2 import Qwen2Config, build_spec

    raw = _shape(args.shape)
    layers_of_config = raw["num_hidden_layers"]
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    cfg = Qwen2Config.from_dict(raw)
    spec = build_spec(cfg)
    if args.mofarax or args.minilorn or args.ligipel or args.poresun:
        designs = run_designs(args, cfg)
        design = "Poresun" if args.poresun else "Ligipel" if args.ligipel else "Minilorn" if args.minilorn else "Mofarax"
        config = {"shape": args.shape, "layers": cfg.num_hidden_layers, "prompt": PROMPT_LEN,
                  "decode_steps": args.design_steps}
        config.update({"pattern": args.pattern if set(args.pattern) <= set("absl") else "absl", "window": args.window,
                       "experts": args.experts, "top": args.top} if args.poresun
                      else {"pattern": args.pattern if set(args.pattern) <= set("pr") else "pppr", "window": args.window,
                            "experts": args.experts, "top": args.top} if args.ligipel
                      else {"pattern": args.pattern, "window": args.window} if args.minilorn
                      else {"mask_size": args.mask_size, "side_dim": args.side_dim})
        print(json.dumps({
            "metric": f"{design} beside Qwen2 at the Qwen2.5-{args.shape.upper()} layer sizes: prompt tok/s, decode "
                      "tok/s, us per kernel",
            "value": designs[args.design_only or design.lower()]["decode_b8"]["tok_s"], "unit": "tok/s", "n_gpus": 1, "higher_is_better": True,
            "dtype": "bf16", "data": "synthetic: random weights, prompt ids uniform in [0, vocab)",
            "config": config, "designs": designs}))
        return 0
    if args.products:
        products = run_products(cfg, [1, 8, 64, 512, PROMPT_LEN])
        print(json.dumps({
            "metric": f"us of a layer's matrix products, own kernels and vendor library (Qwen2.5-{args.shape.upper()} shape)",
            "unit": "us", "n_gpus": 1, "higher_is_better": False, "dtype": "bf16",
            "data": "synthetic: random operands", "products": products}))
        return 0
    if args.offline:
        offline = run_offline(cfg, spec, args.offline, args.seed)
        print(json.dumps({
            "metric": f"generated tok/s of {args.offline} requests with 32 to 256 new tokens each through "
                      f"generate() (Qwen2.5-{args.shape.upper()} shape)",
            "value": offline["tok_s"], "unit": "tok/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16",
            "data": "synthetic: random weights N(0, 0.02), prompts of 24 to 72 random ids",
            "config": {"model": f"Qwen2.5-{args.shape.upper()} shape (Qwen2ForCausalLM)",
                       "layers": cfg.num_hidden_layers, "layers_of_config": layers_of_config,
                       "requests": args.offline, "sampling": "greedy"},
            **offline}))
        return 0
    if args.mixed:
        engine = make_engine(cfg, spec, args.mixed + 1, args.seed, budget=512)
        mixed = run_mixed(engine, cfg, args.mixed, 512, args.seed)
        print(json.dumps({
            "metric": f"ms of a step of {args.mixed} decodes plus a prompt portion, 512-token budget "
                      f"(Qwen2.5-{args.shape.upper()} shape)",
            "value": mixed["mixed_step_ms"], "unit": "ms", "n_gpus": 1, "higher_is_better": False,
            "dtype": "bf16", "data": "synthetic: random weights N(0, 0.02), prompt ids uniform in [0, vocab)",
            "config": {"model": f"Qwen2.5-{args.shape.upper()} shape (Qwen2ForCausalLM)",
                       "layers": cfg.num_hidden_layers, "layers_of_config": layers_of_config,
                       "decodes": args.mixed, "token_budget": 512, "prompt_len": PROMPT_LEN,
                       "page_size": PAGE_SIZE},
            **mixed}))
        return 0
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    engine = make_engine(cfg, spec, max(batches), args.seed)

    results = {}
    for b in batches:
        results[b] = run_decode(engine, cfg, b, args.steps, args.warmup, args.seed + b, args.context)
        print(f"[bench] batch {b}: {results[b]['tok_s']:.1f} tok/s, "
              f"{results[b]['ms_per_step']:.3f} ms/step, {results[b]['gb_s']:.0f} GB/s",
              file=sys.stderr)
    # the same batches near the end of the 4,096-token context, a short run each
    far = {}
    far_steps = min(args.steps, 40)
    if args.far_context and not args.no_points and args.far_context + far_steps + args.warmup + 66 <= CONTEXT_END:
        for b in batches:
            far[b] = run_decode(engine, cfg, b, far_steps, args.warmup, args.seed + 100 + b, args.far_context)
            print(f"[bench] batch {b} at context {far[b]['context_start']:.0f}: {far[b]['tok_s']:.1f} tok/s, "
                  f"{far[b]['ms_per_step']:.3f} ms/step, {far[b]['gb_s']:.0f} GB/s", file=sys.stderr)
    # the main batch once more with temperature and a nucleus instead of the argmax, a short run
    sampled = None
    if not args.no_points:
        sampled = run_decode(engine, cfg, args.batch, min(args.steps, 200), args.warmup, args.seed + 200 + args.batch,
                             args.context, temperature=0.8, top_p=0.95)
        print(f"[bench] batch {args.batch}, temperature 0.8, top_p 0.95: {sampled['tok_s']:.1f} tok/s, "
              f"{sampled['ms_per_step']:.3f} ms/step", file=sys.stderr)
    prefill = run_prefill(engine, cfg, args.seed)
    print(f"[bench] prefill: {prefill}", file=sys.stderr)
    more_points = {}
    if not args.no_points and args.shape == "7b":
        more_points["prefill_2048_budget512_ms"] = round(run_chunked_prefill(engine, cfg, args.seed), 3)
        print(f"[bench] 2,048-token prompt in portions of 512: {more_points['prefill_2048_budget512_ms']} ms",
              file=sys.stderr)
        if 8 * (16000 // PAGE_SIZE + 16) <= engine.cache.num_pages:
            long_ms = run_chunked_prefill(engine, cfg, args.seed, budget=PROMPT_LEN, prompt_len=16000)
            more_points["prefill_16000_budget2048_ms"] = round(long_ms, 2)
            more_points["prefill_16000_bf16_frac"] = round(
                prefill_flops(cfg, 16000) / (long_ms * 1e-3) / BF16_PEAK_FLOPS, 4)
            print(f"[bench] 16,000-token prompt in portions of {PROMPT_LEN}: {long_ms:.1f} ms", file=sys.stderr)
            long_run = run_decode(engine, cfg, 8, min(args.steps, 40), args.warmup, args.seed + 300, 16000)
            more_points["decode_b8_ctx16000"] = round(long_run["tok_s"], 1)
            more_points["decode_b8_ctx16000_hbm_frac"] = round(long_run["gb_s"] / HBM_PEAK_GBS, 4)
            print(f"[bench] batch 8 at context {long_run['context_start']:.0f}: {long_run['tok_s']:.1f} tok/s, "
                  f"{long_run['ms_per_step']:.3f} ms/step, {long_run['gb_s']:.0f} GB/s", file=sys.stderr)
    # one batch left running for the per-kernel times
    from shrike_amd import SamplingParams

    rng = random.Random(args.seed + 7)
    for _ in range(args.batch):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(args.context)],
                           SamplingParams(max_new_tokens=64, ignore_eos=True))
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        engine.step()
    breakdown = kernel_breakdown(engine)
    for req in list(engine.scheduler.running):
        engine.abort(req.req_id)
    print(f"[bench] decode step by kernel (us): {breakdown}", file=sys.stderr)
    peaks = None if args.no_peaks else measure_peaks()
    if peaks:
        print(f"[bench] this GPU: {peaks}", file=sys.stderr)
        prefill["gemm_tflops"] = peaks["gemm_tflops"]
        prefill["mfma_tflops"] = peaks["mfma_tflops"]  # the matrix units alone, random operands
        prefill["achievable_frac"] = round(
            prefill_flops(cfg, PROMPT_LEN) / (prefill["ms"] * 1e-3) / (peaks["gemm_tflops"] * 1e12), 4)

    graphs_on = bool(engine.config.graphs and engine.runner.use_graphs)
    points_shapes = ""
    if not args.no_points and args.shape == "7b":
        del engine
        torch.cuda.empty_cache()
        extra, points_shapes = other_shapes(args, started)
        more_points.update(extra)

    main_run = results[args.batch]
    line = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen2.5-{args.shape.upper()} shape, "
                  f"{args.context}-token prompts, decoding from context "
                  f"{main_run['context_start']:.0f} to {main_run['context_end']:.0f})",
        "value": round(main_run["tok_s"], 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_run["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic: random weights N(0, 0.02), prompt ids uniform in [0, vocab)",
        "config": {
            "model": f"Qwen2.5-{args.shape.upper()} shape (Qwen2ForCausalLM)",
            "layers": cfg.num_hidden_layers,
            "layers_of_config": layers_of_config,
            "hidden": cfg.hidden_size,
            "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size,
            "global_batch": args.batch,
            "seq_len": CONTEXT_END,
            "prompt_len": args.context,
            "context_start": round(main_run["context_start"], 1),
            "context_end": round(main_run["context_end"], 1),
            "page_size": PAGE_SIZE,
            "parallelism": "single GPU",
            "sampling": "greedy",
            "hip_graphs": graphs_on,
            "points_shapes": points_shapes,
        },
        "prefill": prefill,
        "roofline": {
            "bound": "hbm",
            "achieved": round(main_run["gb_s"], 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(main_run["gb_s"] / HBM_PEAK_GBS, 4),
        },
        "points": {f"decode_b{b}": round(r["tok_s"], 1) for b, r in results.items() if b != args.batch},
        "breakdown_us": breakdown,
    }
    line["points"][f"decode_b{args.batch}"] = round(main_run["tok_s"], 1)
    for b, r in far.items():
        line["points"][f"decode_b{b}_ctx4000"] = round(r["tok_s"], 1)
    if sampled:
        line["points"][f"decode_b{args.batch}_top_p"] = round(sampled["tok_s"], 1)
    line["points"].update(more_points)
    if peaks:
        line["roofline"]["achievable"] = peaks["copy_gbs"]
        line["roofline"]["achievable_read"] = peaks["read_gbs"]
        line["roofline"]["achievable_frac"] = round(main_run["gb_s"] / max(peaks["copy_gbs"], peaks["read_gbs"]), 4)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
