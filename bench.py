#!/usr/bin/env python3
"""Benchmark of the batch-split SwiGLU MLP hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the configuration the headline metric is quoted on): one
Llama-3-8B-shaped MLP layer in bf16, x[4096,4096] ~ N(0,1) pre-normed by RMSNorm
(eps 1e-5, weight 1), W_gate/W_up [4096,14336] and W_down [14336,4096] ~
N(0,0.02), split into 2 nano-batches of 2048 tokens; nano-batch 1's gate/up
GEMMs run beside nano-batch 0's SiLU*mul + down projection on a second HIP
stream.  Inputs are generated on the host from fixed seeds and are resident in
HBM before the timed region starts.

A step is one forward of that layer through the complete path
(torch.compile backend -> DynaFlowManager -> engine -> scheduler -> HIP
operators).  Three ways of issuing the same kernels are timed, K steps each:

  serialized         every launch on one stream
  overlapped (eager) two streams, scheduler coroutine per forward
  overlapped (graph) the same two-stream schedule replayed as one hipGraph

`value` is tokens/s of the overlapped hipGraph replay.  One JSON line is printed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

TOKENS, HIDDEN, INTER, SPLITS = 4096, 4096, 14336, 2
BF16_MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0            # MI355X HBM3E
# HBM-side bytes per launch, measured with hardware counters; the summaries are under profiles/
GATE_GEMM_TRAFFIC_BYTES = 432.9e6      # fetch 369.4 MB + write 63.5 MB
GATE_UP_SILU_TRAFFIC_BYTES = 845.8e6   # fetch 738.9 MB + write 106.9 MB (non-temporal stores leave in 64-byte pieces:
                                       # runs that straddle two are counted twice; 58.7 MB of results)
GATE_UP_SILU_SQUARE_TRAFFIC_BYTES = 797.3e6   # the 256 x (128 + 128) tile: fetch 738.6 MB + write 58.7 MB
GATE_UP_SILU_PAIR_KERNEL = "gemm_bf16_ring_kernel<true>, 256 x (128 + 128) tile"
METRIC = "MLP-layer tokens/s + overlap speedup vs serial, 8B-shape bf16, 1 MI355X"


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=15)
    p.add_argument("--skip-cpu", action="store_true", help="leave out the host baseline (profiling runs)")
    p.add_argument("--sustain-seconds", type=float, default=3.0,
                   help="seconds of continuous load ahead of the `sustained` figures (0: leave them out)")
    p.add_argument("--settle-seconds", type=float, default=0.5,
                   help="seconds of the same step, untimed, ahead of the warm-up steps of every timed loop (the "
                        "package's clocks in their loaded state; 0: none)")
    p.add_argument("--headline-config-only", action="store_true",
                   help="leave out the `other_configs` object (decoder layer, fp8 layer, decode step)")
    p.add_argument("--kernels-only", action="store_true",
                   help="run only the single-kernel timing loops plus a 256 MiB device copy (used to calibrate "
                        "FETCH_SIZE / WRITE_SIZE under rocprofv3 --pmc); prints the kernel figures as JSON")
    p.add_argument("--operands", choices=("random", "zeros"), default="random",
                   help="with --kernels-only: `zeros` runs the same launches on all-zero operands (no bit toggles in "
                        "the data paths: what the kernels do when the package power limit is out of the way)")
    p.add_argument("--headline-only", action="store_true",
                   help="only the headline mode (fused epilogue, two streams, one hipGraph): for kernel traces of the step")
    p.add_argument("--fp8", action="store_true",
                   help="measure the fp8 70B-shaped MLP layer (x[8192,8192], I=28672, 4 nano-batches of 2048) "
                        "instead of the headline bf16 configuration")
    p.add_argument("--decode-kernels", action="store_true",
                   help="time the decode-step kernels at the shape of one nano-batch of the decode configuration "
                        "(128 sequences, 32 query / 8 kv heads, 2048 cached positions): RoPE + cache append + "
                        "attention, against the HBM roofline")
    p.add_argument("--decode-projection-launches", action="store_true",
                   help="eager launches of the four projections of a decode layer at 128 rows over rotating weight "
                        "copies (for rocprofv3 counters and kernel traces)")
    p.add_argument("--prefill-attention-kernels", action="store_true",
                   help="time causal prefill attention at the shape of one nano-batch of the decoder-layer "
                        "configuration (4 sequences x 2048 tokens, 32 query / 8 kv heads), PyTorch's fused "
                        "attention beside it")
    p.add_argument("--decode", action="store_true",
                   help="measure one decode step over 32 stacked 8B-shaped layers (256 single-token queries, "
                        "2048 cached positions each, 2 nano-batches of 128) instead of the headline configuration")
    p.add_argument("--decoder", action="store_true",
                   help="measure the full Llama-3-8B-shaped decoder layer (prefill 8 x 2048, attention of one "
                        "nano-batch beside the MLP of the other) instead of the headline configuration")
    p.add_argument("--knob", action="append", default=[], metavar="NAME=VALUE",
                   help="extra entry of DynaFlowConfig.additional_config for every mode of the run (value read as "
                        "JSON when it parses, else as a string), e.g. --knob streams=by_nano_batch")
    return p.parse_args()


EXTRA_KNOBS: dict = {}


def read_knobs(pairs):
    for pair in pairs:
        name, _, value = pair.partition("=")
        try:
            EXTRA_KNOBS[name] = json.loads(value)
        except ValueError:
            EXTRA_KNOBS[name] = value


def build_path(torch, x, weights, **knobs):
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.manager import DynaFlowManager
    from dynaflow_amd.mlp import SwiGLUMLP

    wg, wu, wd = weights
    model = SwiGLUMLP(HIDDEN, INTER, dtype=torch.bfloat16, device="cuda")
    with torch.no_grad():
        model.gate_proj.weight.copy_(wg)
        model.up_proj.weight.copy_(wu)
        model.down_proj.weight.copy_(wd)
    extra = {"min_nano_split_tokens": 64, "num_nano_batches": SPLITS, "dump_graph": False}
    extra.update(knobs)
    extra.update(EXTRA_KNOBS)          # --knob on the command line wins over the mode's own knobs
    cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", SPLITS, InductorConfig(enabled=True),
                         CUDAGraphConfig(enabled=False, capture_sizes=[TOKENS]), extra)
    manager = DynaFlowManager()
    torch._dynamo.reset()
    torch._dynamo.mark_dynamic(x, 0)
    compiled = torch.compile(model, backend=make_backend(manager, cfg), fullgraph=True)
    with torch.no_grad():
        manager.prepare(TOKENS, [TOKENS])
        compiled(x)
    return manager, compiled


def time_steps(torch, manager, compiled, x, steps, warmup, use_graph, settle_s=0.0):
    """ms per step over exactly ``steps`` steps after ``warmup`` untimed ones, a device synchronisation on both
    sides; ``settle_s`` seconds of the same step run before the warm-up steps (untimed)."""
    def step():
        manager.prepare(TOKENS, [TOKENS], use_cudagraph=use_graph)
        return compiled(x)

    with torch.no_grad():
        if settle_s > 0:
            step()                                   # set-up of the first call (graph capture) is not load
            torch.cuda.synchronize()
            until = time.perf_counter() + settle_s
            while time.perf_counter() < until:
                for _ in range(10):
                    step()
                torch.cuda.synchronize()
        for _ in range(warmup):
            y = step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            y = step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, y


def vendor_library_layer(torch, x, weights, steps, warmup, settle_s):
    """ms per step of ``down(silu(gate(x)) * up(x))`` on the whole batch through ``torch.nn.functional`` (the vendor's
    GEMM library, aten's SiLU and multiplication), captured once and replayed as one graph; timed like every other
    loop of this file.  A yardstick, not part of the path."""
    import torch.nn.functional as F

    wg, wu, wd = weights
    side = torch.cuda.Stream()
    with torch.no_grad():
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
        torch.cuda.synchronize()
        if settle_s > 0:
            until = time.perf_counter() + settle_s
            while time.perf_counter() < until:
                for _ in range(10):
                    graph.replay()
                torch.cuda.synchronize()
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    del graph, y
    return (t1 - t0) * 1e3 / steps


def gpu_time_of_steps(torch, manager, compiled, x, steps):
    """GPU-side duration of one eagerly issued step (median over ``steps``, ms): the GPU is kept busy with a
    spin kernel while the host issues the whole step behind it, so the interval between the two events holds the
    step's kernels back to back and none of the host's issue time."""
    spin_cycles = 8_000_000   # about 4 ms: longer than the host needs to issue a step
    times = []
    with torch.no_grad():
        for _ in range(steps):
            manager.prepare(TOKENS, [TOKENS], use_cudagraph=False)
            start = torch.cuda.Event(enable_timing=True)
            stop = torch.cuda.Event(enable_timing=True)
            torch.cuda._sleep(spin_cycles)
            start.record()
            compiled(x)
            stop.record()
            stop.synchronize()
            times.append(start.elapsed_time(stop))
    times.sort()
    return times[len(times) // 2]


def sustained_steps(torch, manager, compiled, x, steps, load_seconds):
    """ms per step of the graph replay after ``load_seconds`` of the same replay without a pause: the package
    sits at its power limit by then and the clocks have settled, which a short timed loop does not show."""
    def step():
        manager.prepare(TOKENS, [TOKENS], use_cudagraph=True)
        return compiled(x)

    with torch.no_grad():
        until = time.perf_counter() + load_seconds
        while time.perf_counter() < until:
            for _ in range(25):
                step()
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps


def sustained_kernel(torch, fn, iters, load_seconds):
    """Average launch duration (ms) right after ``load_seconds`` of back-to-back launches of the same kernel."""
    until = time.perf_counter() + load_seconds
    while time.perf_counter() < until:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
    return time_kernel(torch, fn, iters, warmup=0)


def time_kernel(torch, fn, iters, warmup=20):
    """Average duration of one launch, from HIP events on the stream it is launched on."""
    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


_PAIR_STREAMS: list = []


def time_pair(torch, fn, iters, warmup=20):
    """Average duration (ms) of two launches that run side by side: a loop of ``fn(0)`` on one stream beside a loop of
    ``fn(1)`` on another (the host issues them alternately, each stream runs its launches back to back); the two
    streams fork from the timing stream once before the loops and join it once after them, HIP events on that
    stream around the whole."""
    if not _PAIR_STREAMS:       # made once: streams are dealt to a few hardware queues, and two streams that land
        _PAIR_STREAMS.extend([torch.cuda.Stream(), torch.cuda.Stream()])   # on one queue would run one after the other
    side = _PAIR_STREAMS
    origin = torch.cuda.current_stream()

    def loops(count):
        fork = torch.cuda.Event()
        fork.record(origin)
        for stream in side:
            stream.wait_event(fork)
        for _ in range(count):
            for i, stream in enumerate(side):
                with torch.cuda.stream(stream):
                    fn(i)
        for stream in side:
            join = torch.cuda.Event()
            join.record(stream)
            origin.wait_event(join)

    loops(warmup)
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    loops(iters)
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def single_kernels(torch, ops, x, weights, iters, calibration_copy=False):
    """Average launch durations (ms) of the kernels of one nano-batch, each timed alone."""
    mb = TOKENS // SPLITS
    xb = x[:mb]
    gate = ops.linear(xb, weights[0])
    up = ops.linear(xb, weights[1])
    act = ops.silu_mul(gate, up, True)
    for _ in range(60):                         # clocks and caches settle before the first timed loop
        ops.linear(xb, weights[0])
    out = {
        "gate_ms": time_kernel(torch, lambda: ops.linear(xb, weights[0]), iters),
        "down_ms": time_kernel(torch, lambda: ops.linear(act, weights[2]), iters),
        "silu_ms": time_kernel(torch, lambda: ops.silu_mul(gate, up, True), iters),
        "gate_up_silu_ms": time_kernel(torch, lambda: ops.gate_up_silu(xb, weights[0], weights[1]), iters),
        "blas_ms": time_kernel(torch, lambda: torch.nn.functional.linear(xb, weights[0]), iters),
    }
    # the two nano-batches' launches side by side, planned for the pair (knob side_by_side=2): gate/up/SiLU with the
    # 256 x (128 + 128) tile, down projections with one workgroup per tile
    halves = (x[:mb], x[mb:2 * mb])
    acts = (act, act.clone())

    def fused_of(i):
        with ops.launch_options(side_by_side=2):
            return ops.gate_up_silu(halves[i], weights[0], weights[1])

    def down_of(i):
        with ops.launch_options(side_by_side=2):
            return ops.linear(acts[i], weights[2])

    out["gate_up_silu_pair_ms"] = time_pair(torch, fused_of, iters)
    out["down_pair_ms"] = time_pair(torch, down_of, iters)
    if calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        out["copy_256MiB_ms"] = time_kernel(torch, lambda: dst.copy_(src), iters)
    return out


def decode_kernels(torch, ops, iters):
    """Decode attention of one nano-batch (128 new tokens, each over 2048 cached positions of its own
    sequence): every cached K and V element is read once, so the algorithmic bytes are the cache size."""
    from dynaflow_amd.decoder import rope_tables

    seqs, heads, kv_heads, capacity, d = 128, 32, 8, 2048, 128
    gen = torch.Generator(device="cuda").manual_seed(5)
    k_cache = torch.randn(seqs, kv_heads, capacity, d, generator=gen, device="cuda").bfloat16()
    v_cache = torch.randn(seqs, kv_heads, capacity // 8, d, 8, generator=gen, device="cuda").bfloat16()
    qkv = torch.randn(seqs, (heads + 2 * kv_heads) * d, generator=gen, device="cuda").bfloat16()
    slots = torch.arange(seqs, dtype=torch.int32, device="cuda")
    lengths = torch.full((seqs,), capacity, dtype=torch.int32, device="cuda")
    cos, sin = (t.cuda() for t in rope_tables(capacity, d, 500000.0))
    ms = time_kernel(torch, lambda: ops.decode_attention(qkv, k_cache, v_cache, slots, lengths, cos, sin, heads,
                                                         kv_heads), iters)
    cache_bytes = 2.0 * seqs * kv_heads * capacity * d * 2
    return {
        "workload": f"decode attention, {seqs} sequences x {capacity} cached positions, {heads} query / "
                    f"{kv_heads} kv heads, head_dim {d}, bf16 (rope + append kernel and attention kernel)",
        "ms": ms,
        "roofline": {"kernel": "decode_attention_kernel", "bound": "hbm", "achieved": cache_bytes / (ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": cache_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "algorithmic_bytes": cache_bytes},
    }


def decode_projections(torch, ops, iters):
    """The four projections of a decode layer at 128 rows (one nano-batch), weights rotated over several copies so
    that they come from HBM as in a 32-layer model; every case is a captured graph of four launches (or pairs):
    one launch alone, the two nano-batches' launches side by side on two streams over the same weights (planned
    alone and planned for two), and one launch over all 256 rows.  us per launch or pair."""
    H, I, rows = HIDDEN, INTER, 128
    gen = torch.Generator(device="cuda").manual_seed(6)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]

    def replayed(body):
        body()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            body()
        best = min(time_kernel(torch, graph.replay, iters) for _ in range(3))
        return round(best * 1e3 / 4, 1)

    out = {}
    for name, n, k, fused in (("qkv", 6144, H, False), ("o", H, H, False), ("gate_up_silu", I, H, True),
                              ("down", H, I, False)):
        xs = [torch.randn(rows, k, generator=gen, device="cuda").bfloat16() for _ in range(2)]
        both = torch.cat(xs)
        copies = 4 if fused else 8
        ws = [(torch.randn(n, k, generator=gen, device="cuda") * 0.02).bfloat16() for _ in range(copies)]
        call = (lambda x, i: ops.gate_up_silu(x, ws[i], ws[(i + 1) % copies])) if fused else \
               (lambda x, i: ops.linear(x, ws[i]))

        def alone():
            for it in range(4):
                call(xs[0], it)

        def whole():
            for it in range(4):
                call(both, it)

        def pairs(share):
            def body():
                for it in range(4):
                    here = torch.cuda.current_stream()
                    for stream in streams:
                        stream.wait_stream(here)
                    with ops.launch_options(side_by_side=share):
                        for x, stream in zip(xs, streams):
                            with torch.cuda.stream(stream):
                                call(x, it)
                    for stream in streams:
                        here.wait_stream(stream)
            return body

        out[name] = {"one_launch_128_rows_us": replayed(alone), "pair_planned_alone_us": replayed(pairs(1)),
                     "pair_planned_for_two_us": replayed(pairs(2)), "one_launch_256_rows_us": replayed(whole),
                     "weight_bytes": (2 if fused else 1) * n * k * 2}
        del ws
    return out


def decode_projection_launches(torch, ops, iters):
    """Eager launches of the four projections of a decode layer at 128 rows, for hardware counters and kernel traces
    (one kernel per launch, nothing else on the GPU): every projection ``iters`` times over eight rotating weight
    copies (they come from HBM, as in a 32-layer model), once planned as a lone launch and once with the plan for two
    launches side by side (the form the two-stream decode schedule runs; traced alone here).  Returns us per launch
    from HIP events around each loop."""
    H, I, rows = HIDDEN, INTER, 128
    gen = torch.Generator(device="cuda").manual_seed(6)
    out = {}
    for name, n, k, fused in (("qkv", 6144, H, False), ("o", H, H, False), ("gate_up_silu", I, H, True),
                              ("down", H, I, False)):
        x = torch.randn(rows, k, generator=gen, device="cuda").bfloat16()
        copies = 4 if fused else 8
        ws = [(torch.randn(n, k, generator=gen, device="cuda") * 0.02).bfloat16() for _ in range(copies)]
        for share in (1, 2):
            state = {"i": 0}

            def call():
                i = state["i"] = (state["i"] + 1) % copies
                with ops.launch_options(side_by_side=share):
                    if fused:
                        ops.gate_up_silu(x, ws[i], ws[(i + 1) % copies])
                    else:
                        ops.linear(x, ws[i])

            out[f"{name}_planned_for_{share}_us"] = round(time_kernel(torch, call, iters, warmup=8) * 1e3, 1)
        del ws
    return out


def prefill_attention_kernels(torch, ops, iters):
    """Causal grouped-query attention of one prefill nano-batch.  Algorithmic work: the causal half of the
    two products, 2 * B * heads * S * S * d FLOP."""
    B, S, heads, kv_heads, d = 4, 2048, 32, 8, 128
    gen = torch.Generator(device="cuda").manual_seed(9)
    q = torch.randn(B, S, heads, d, generator=gen, device="cuda").bfloat16()
    k = torch.randn(B, S, kv_heads, d, generator=gen, device="cuda").bfloat16()
    v = torch.randn(B, S, kv_heads, d, generator=gen, device="cuda").bfloat16()
    # the first loop starts from an idle GPU whose clocks are still coming up (this kernel does not reach the
    # power limit, so unlike the GEMMs it gets faster as the run goes on); the figure of record is taken after
    # 300 more launches, as inside a model's step
    ms_first = time_kernel(torch, lambda: ops.causal_attention(q, k, v), iters)
    ms = time_kernel(torch, lambda: ops.causal_attention(q, k, v), iters, warmup=300)
    qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    sdpa = torch.nn.functional.scaled_dot_product_attention
    aten_ms = time_kernel(torch, lambda: sdpa(qt, kt, vt, is_causal=True, enable_gqa=True), iters, warmup=150)
    flop = 2.0 * B * heads * S * S * d
    return {
        "workload": f"causal prefill attention, {B} sequences x {S} tokens, {heads} query / {kv_heads} kv heads, "
                    f"head_dim {d}, bf16 (V re-layout kernel + attention kernel)",
        "ms": ms,
        "ms_first_loop_from_idle": ms_first,
        "torch_sdpa_ms": aten_ms,
        "roofline": {"kernel": "causal_attention_kernel", "bound": "mfma", "achieved": flop / (ms * 1e-3) / 1e12,
                     "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": flop / (ms * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, "algorithmic_flop": flop},
    }


def rel_err_of(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def fp8_config(torch, steps, warmup, brief=False):
    """fp8 70B-shaped layer: x[8192,8192] bf16 quantised per tensor inside the graph, weights e4m3 with
    per-output-channel scales, 4 nano-batches of 2048 through the manager on two streams.  ``brief``: only the
    reported mode and its one-stream baseline."""
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.fp8_mlp import Fp8SwiGLU
    from dynaflow_amd.manager import DynaFlowManager

    tokens, hidden, inter, splits = 8192, 8192, 28672, 4
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(tokens, hidden, generator=gen, device="cuda", dtype=torch.float32).bfloat16()
    parts = []
    for shape in ((inter, hidden), (inter, hidden), (hidden, inter)):
        w = (torch.randn(shape, generator=gen, device="cuda", dtype=torch.float32) * 0.02).bfloat16()
        parts.append(w)
    layer = Fp8SwiGLU.from_weights(*parts)
    del parts
    results = {}
    fused = {"whole_graph": True, "fuse_silu_epilogue": True}
    modes = [("serialized", {"serialize": True}), ("overlapped", {"whole_graph": True}),
             ("serialized_fused_gate_up", {"serialize": True, **fused}),
             ("overlapped_fused_gate_up", dict(fused)),
             ("stream_per_nano_batch_fused_gate_up", {**fused, "streams": "by_nano_batch"})]
    if brief:
        modes = [m for m in modes if m[0] in ("serialized_fused_gate_up", "overlapped_fused_gate_up")]
    y_best = None
    for name, knobs in modes:
        # the fused mode: gate, up and SiLU*mul + absmax in ONE GEMM launch, cut in front of the down projection
        layer.fuse_gate_up = bool(knobs.get("fuse_silu_epilogue", False))
        extra = {"min_nano_split_tokens": 64, "num_nano_batches": splits, "dump_graph": False, **EXTRA_KNOBS}
        extra.update(knobs)
        cfg = DynaFlowConfig("dynaflow_amd.schedulers:MLPOverlapScheduler", splits, InductorConfig(enabled=True),
                             CUDAGraphConfig(enabled=False, capture_sizes=[tokens]), extra)
        manager = DynaFlowManager()
        torch._dynamo.reset()
        torch._dynamo.mark_dynamic(x, 0)
        compiled = torch.compile(layer, backend=make_backend(manager, cfg), fullgraph=True)
        with torch.no_grad():
            manager.prepare(tokens, [tokens])
            compiled(x)

            def step(use_graph):
                manager.prepare(tokens, [tokens], use_cudagraph=use_graph)
                return compiled(x)

            timed = (("eager", False),) if name == "serialized" else \
                    (("graph", True),) if brief else (("eager", False), ("graph", True))
            for mode, use_graph in timed:
                for _ in range(warmup):
                    step(use_graph)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    y = step(use_graph)
                torch.cuda.synchronize()
                results[f"{name}_{mode}_ms"] = (time.perf_counter() - t0) * 1e3 / steps
            if name == "overlapped_fused_gate_up":
                y_best = y.clone()
    flops = 6.0 * tokens * hidden * inter
    candidates = [m for m in ("overlapped_graph_ms", "overlapped_fused_gate_up_graph_ms",
                              "stream_per_nano_batch_fused_gate_up_graph_ms") if m in results]
    best_mode = min(candidates, key=lambda m: results[m])
    best = results[best_mode]
    # the dominant kernel, alone: gate + up + SiLU*mul + absmax of one nano-batch in one launch
    from dynaflow_amd import _cabi, ops
    lib = _cabi.load()
    mb = tokens // splits
    with torch.no_grad():
        xq, xs = ops.quant_fp8(x[:mb])
    act = torch.empty((mb, inter), dtype=torch.bfloat16, device="cuda")
    amax = torch.zeros(1, dtype=torch.float32, device="cuda")

    def fused_launch():
        _cabi.check("dfhip_gemm_fp8_gate_up_silu_absmax", lib.dfhip_gemm_fp8_gate_up_silu_absmax(
            xq.data_ptr(), hidden, layer.w_gate_q.data_ptr(), layer.w_up_q.data_ptr(), hidden, act.data_ptr(), inter,
            xs.data_ptr(), layer.w_gate_s.data_ptr(), layer.w_up_s.data_ptr(), amax.data_ptr(), mb, inter, hidden,
            torch.cuda.current_stream().cuda_stream))

    ms_fused = time_kernel(torch, fused_launch, 30)
    fused_flops = 4.0 * mb * hidden * inter
    del act, xq

    # sampled rows of the fused mode's result against an evaluation that takes nothing from the kernels: torch's own
    # e4m3 conversion of the activations, gate / up of the whole nano-batch as fp32 products of the dequantised
    # operands (torch on the GPU), and - in the CPU leg - the oracle's SiLU*mul, its absmax over the whole
    # nano-batch, the oracle's e4m3 encoder for the sampled rows, an fp32 down projection
    prepared = []
    if y_best is not None:
        fp8_max = 448.0
        with torch.no_grad():
            wg = layer.w_gate_q.float() * layer.w_gate_s[:, None]
            wu = layer.w_up_q.float() * layer.w_up_s[:, None]
            for nano_batch, picked in ((0, [0, 777, 2047]), (3, [1, 2046])):
                xb = x[nano_batch * mb:(nano_batch + 1) * mb].float()
                x_scale = xb.abs().max().clamp_min(1e-12) / fp8_max
                xd = (xb / x_scale).clamp(-fp8_max, fp8_max).to(torch.float8_e4m3fn).float() * x_scale
                rows = torch.tensor(picked, device="cuda")
                prepared.append(((xd @ wg.t()).bfloat16(), (xd @ wu.t()).bfloat16(), rows,
                                 y_best[nano_batch * mb + rows].float()))
            del wg, wu, xb, xd

    def oracle_check(mods):
        oracle_mlp = mods["mlp"]
        errs = []
        wd = layer.w_down_q.float() * layer.w_down_s[:, None]
        for g, u, rows, got in prepared:
            a = oracle_mlp.silu_mul_exact(g, u)
            a_scale = a.float().abs().max().clamp_min(1e-12) / 448.0
            scaled = (a[rows].float() / a_scale).clamp(-448.0, 448.0).cpu()
            codes = torch.from_numpy(oracle_mlp.e4m3_encode(scaled.numpy()))
            a_rows = oracle_mlp.dequant(codes, a_scale.reshape(1).cpu())
            errs.append(rel_err_of(got, a_rows.cuda() @ wd.t()))
        return {"worst": max(errs), "bound": 5e-2, "rows": "3 of nano-batch 0, 2 of nano-batch 3",
                "against": "fp32 evaluation of the dequantised operands, re-quantisation by the oracle's encoder"}

    line = {
        "metric": "fp8 MLP-layer tokens/s, 70B-shape e4m3, 1 MI355X",
        "value": tokens / (best * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": best, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": {"workload": "fp8 70B-shaped SwiGLU MLP layer, x[8192,8192], I=28672, 4 nano-batches of 2048, "
                               "per-tensor activation / per-channel weight scales, bf16 output; gate / up / "
                               "SiLU*mul + absmax as one launch per nano-batch, then re-quantisation and the down "
                               "projection; whole two-stream schedule as one hipGraph",
                   "issue_mode": best_mode[:-3]},
        "timings": results,
        "layer": {"tflops": flops / (best * 1e-3) / 1e12, "frac_of_fp8_mfma_peak": flops / (best * 1e-3) / 1e12 / 5000.0},
        "roofline": {
            "kernel": "gemm_fp8_ring_kernel<true> (gate and up projection of one nano-batch with the SiLU*mul + absmax "
                      "epilogue: [2048,8192] x 2 x [28672,8192]^T -> act[2048,28672]), timed alone with HIP events",
            "bound": "mfma", "achieved": fused_flops / (ms_fused * 1e-3) / 1e12, "peak": 5000.0, "unit": "TFLOP/s",
            "frac": fused_flops / (ms_fused * 1e-3) / 1e12 / 5000.0, "ms": ms_fused,
            # HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (1410.2 MB fetched + 117.7 MB
            # written; the summary is under profiles/); algorithmic: 16.8 + 2 x 234.9 MB read, 117.4 MB written
            "traffic": 1527.9e6, "traffic_unit": "bytes per launch",
        },
        "oracle_check": oracle_check if prepared else None,
    }
    if "serialized_fused_gate_up_graph_ms" in results and "overlapped_fused_gate_up_graph_ms" in results:
        # the same kernels and split on one stream against the two-stream schedule, graph against graph
        line["overlap_speedup"] = results["serialized_fused_gate_up_graph_ms"] / results["overlapped_fused_gate_up_graph_ms"]
    if "serialized_eager_ms" in results:
        line["speedup_vs_separate_kernels_serialized_eager"] = results["serialized_eager_ms"] / best
    return line


def decoder_config(torch, steps, warmup, brief=False):
    """Full decoder layer, random-init bf16: hidden 4096, 32 q / 8 kv heads, head_dim 128, RoPE theta 5e5,
    causal attention, SwiGLU 14336; prefill batch 8 x seq 2048, tokens ~ U[0, 128256)."""
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.decoder import DecoderLayer
    from dynaflow_amd.manager import DynaFlowManager

    batch, S, H, I, vocab = 8, 2048, 4096, 14336, 128256
    layer = DecoderLayer(vocab=vocab, hidden=H, heads=32, kv_heads=8, head_dim=128, inter=I, seq_len=S,
                         dtype=torch.bfloat16, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(0)
    with torch.no_grad():
        for name, p in layer.named_parameters():
            if "norm" in name:
                continue
            p.copy_((torch.randn(p.shape, generator=gen, device="cuda", dtype=torch.float32)
                     * (1.0 if name == "embed" else 0.02)).to(p.dtype))
    ids = torch.randint(0, vocab, (batch * S,), generator=torch.Generator().manual_seed(4)).cuda()
    T = batch * S
    results = {}
    modes = [("serialized", {"serialize": True}), ("overlapped", {"whole_graph": True}),
             ("overlapped_fused_silu", {"whole_graph": True, "fuse_silu_epilogue": True}),
             # every nano-batch on a stream of its own instead of one stream per kind of sub-graph (kernels planned
             # for the two launches of a kind that then run side by side)
             ("stream_per_nano_batch_fused_silu", {"whole_graph": True, "fuse_silu_epilogue": True,
                                                   "streams": "by_nano_batch"}),
             # the same kernels and split as the mode above on ONE stream: the baseline of the overlap figure
             ("one_stream_same_kernels", {"whole_graph": True, "fuse_silu_epilogue": True, "serialize": True,
                                          "side_by_side": 2})]
    if brief:
        modes = modes[3:]
    y_best = None
    for name, knobs in modes:
        extra = {"min_nano_split_tokens": 64, "dump_graph": False, **EXTRA_KNOBS}
        extra.update(knobs)
        cfg = DynaFlowConfig("dynaflow_amd.schedulers:DecoderOverlapScheduler", 2, InductorConfig(enabled=True),
                             CUDAGraphConfig(enabled=False, capture_sizes=[T]), extra)
        manager = DynaFlowManager()
        torch._dynamo.reset()
        torch._dynamo.mark_dynamic(ids, 0)
        compiled = torch.compile(layer, backend=make_backend(manager, cfg), fullgraph=True)
        with torch.no_grad():
            manager.prepare(batch, [S] * batch)
            compiled(ids)
            timed = (("eager", False),) if name == "serialized" else \
                    (("graph", True),) if brief or name == "one_stream_same_kernels" else (("eager", False), ("graph", True))
            for mode, use_graph in timed:
                for _ in range(warmup):
                    manager.prepare(batch, [S] * batch, use_cudagraph=use_graph)
                    compiled(ids)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    manager.prepare(batch, [S] * batch, use_cudagraph=use_graph)
                    y = compiled(ids)
                torch.cuda.synchronize()
                results[f"{name}_{mode}_ms"] = (time.perf_counter() - t0) * 1e3 / steps
            if name == "stream_per_nano_batch_fused_silu":
                y_best = y.clone()
    flops = 2.0 * T * H * 6144 + 2.0 * T * H * H + 2.0 * batch * 32 * S * S * 128 + 6.0 * T * H * I
    candidates = [m for m in ("overlapped_graph_ms", "overlapped_eager_ms", "overlapped_fused_silu_graph_ms",
                              "stream_per_nano_batch_fused_silu_graph_ms") if m in results]
    best_mode = min(candidates, key=lambda m: results[m])
    best = results[best_mode]
    # the dominant kernel, alone: gate + up + SiLU*mul of one nano-batch (8192 tokens) in one launch
    from dynaflow_amd import ops
    mb = T // 2
    xb = torch.randn(mb, H, generator=gen, device="cuda", dtype=torch.float32).bfloat16()
    w_gate = next(p for n, p in layer.named_parameters() if n.endswith("w_gate"))
    w_up = next(p for n, p in layer.named_parameters() if n.endswith("w_up"))
    with torch.no_grad():
        ms_fused = time_kernel(torch, lambda: ops.gate_up_silu(xb, w_gate, w_up), 20)
    fused_flops = 4.0 * mb * H * I
    ids_host = ids.cpu()
    rows = [255, 2047, 5 * S + 1000]             # two sequences, one of each nano-batch
    got_rows = y_best[rows].float().cpu() if y_best is not None else None

    def oracle_check(mods):
        ref = mods["decoder"]
        want = ref.decoder_layer_rows(ids_host, ref.params_of(layer), rows, S, 32, 8, 128)
        return {"worst": rel_err_of(got_rows, want), "bound": 2e-2, "rows": rows,
                "against": "float64 oracle of the layer restricted to the sampled rows' sequences"}

    line = {
        "metric": "decoder-layer prefill tokens/s, 8B-shape bf16, 1 MI355X",
        "value": T / (best * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": best, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "Llama-3-8B-shaped decoder layer, prefill 8 x 2048 tokens, 2 nano-batches of 4 "
                               "sequences, attention sub-graph of one beside the MLP sub-graph of the other; "
                               "projections, RoPE, causal attention, norms and MLP on the hand-written HIP "
                               "operators (embedding gather, residual adds and the final concatenation on aten)",
                   "issue_mode": best_mode[:-3]},
        "timings": results,
        "layer": {"algorithmic_tflop": flops / 1e12, "tflops": flops / (best * 1e-3) / 1e12,
                  "frac_of_bf16_mfma_peak": flops / (best * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS},
        "roofline": {
            "kernel": "gemm_bf16_ring_kernel<true> (gate and up projection of one nano-batch with the SiLU*mul "
                      "epilogue: [8192,4096] x 2 x [14336,4096]^T -> act[8192,14336]), timed alone with HIP events",
            "bound": "mfma", "achieved": fused_flops / (ms_fused * 1e-3) / 1e12, "peak": BF16_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": fused_flops / (ms_fused * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, "ms": ms_fused,
            # HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (2821.9 MB fetched + 234.9 MB
            # written; the summary is under profiles/); algorithmic: 67.1 + 2 x 117.4 MB read, 234.9 MB written
            "traffic": 3056.8e6, "traffic_unit": "bytes per launch",
        },
        "oracle_check": oracle_check if got_rows is not None else None,
    }
    if "one_stream_same_kernels_graph_ms" in results and "stream_per_nano_batch_fused_silu_graph_ms" in results:
        # the same kernels and split on one stream against the two-stream schedule, graph against graph
        line["overlap_speedup"] = (results["one_stream_same_kernels_graph_ms"]
                                   / results["stream_per_nano_batch_fused_silu_graph_ms"])
    if "serialized_eager_ms" in results:
        line["speedup_vs_separate_kernels_serialized_eager"] = results["serialized_eager_ms"] / best
    return line


def decode_config(torch, steps, warmup, layers=32, brief=False):
    """Decode step: 256 sequences, one new token each, KV caches of 2048 positions ~N(0,1), 2 nano-batches of
    128; attention sub-graph of one nano-batch beside the MLP sub-graph of the other in every layer."""
    from dynaflow_amd.backend import make_backend
    from dynaflow_amd.config import CUDAGraphConfig, DynaFlowConfig, InductorConfig
    from dynaflow_amd.decode import DecodeModel
    from dynaflow_amd.manager import DynaFlowManager

    seqs, capacity, H, I, heads, kv_heads, vocab = 256, 2048, 4096, 14336, 32, 8, 128256
    model = DecodeModel(layers=layers, vocab=vocab, hidden=H, heads=heads, kv_heads=kv_heads, inter=I, slots=seqs,
                        capacity=capacity, dtype=torch.bfloat16, device="cuda")
    model.init_weights(0)
    model.fill_caches(5)
    gen = torch.Generator().manual_seed(4)
    ids = torch.randint(0, vocab, (seqs,), generator=gen).cuda()
    slots = torch.arange(seqs, dtype=torch.int32).cuda()
    lengths = torch.full((seqs,), capacity, dtype=torch.int32).cuda()
    inputs = (ids, slots, lengths)
    half = seqs // 2
    results = {}
    # the last mode is the comparison without nano-batches: all 256 queries as one batch on one stream (the
    # weights are read once per step instead of once per nano-batch, nothing overlaps), sub-graphs replayed
    # "whole" modes: the complete two-stream schedule of all layers captured once and replayed as ONE hipGraph
    modes = [("serialized_eager", {"serialize": True}, False), ("overlapped_eager", {}, False),
             ("overlapped_sub_graph_replay", {}, True),
             # one stream per nano-batch with the kernels planned as lone launches (override of what the
             # manager derives from the stream policy), for comparison
             ("stream_per_nano_batch_planned_alone_sub_graph_replay",
              {"streams": "by_nano_batch", "side_by_side": 1}, True),
             ("serialized_whole_graph", {"serialize": True, "whole_graph": True}, "whole"),
             ("overlapped_whole_graph", {"whole_graph": True}, "whole"),
             ("stream_per_nano_batch_planned_alone_whole_graph",
              {"streams": "by_nano_batch", "side_by_side": 1, "whole_graph": True}, "whole"),
             # one stream per nano-batch: the same sub-graph of both nano-batches runs at the same time and
             # the kernels are planned for the pair (the weight-streaming GEMMs split K over half as many
             # workgroups and move half as many fp32 blocks; another order of additions)
             ("stream_per_nano_batch_planned_for_two_sub_graph_replay", {"streams": "by_nano_batch"}, True),
             ("stream_per_nano_batch_planned_for_two_whole_graph",
              {"streams": "by_nano_batch", "whole_graph": True}, "whole"),
             # the same kernels and split as the mode above on ONE stream: the baseline of the overlap figure
             ("one_stream_same_kernels_whole_graph",
              {"serialize": True, "side_by_side": 2, "whole_graph": True}, "whole"),
             ("unsplit_sub_graph_replay", {"min_nano_split_tokens": 1 << 30}, True)]
    if brief:
        modes = [m for m in modes if m[0] in ("stream_per_nano_batch_planned_for_two_whole_graph",
                                              "one_stream_same_kernels_whole_graph")]
    y_best = None
    for name, knobs, graphs in modes:
        extra = {"min_nano_split_tokens": 1, "dump_graph": False, "max_tokens": seqs, "fuse_silu_epilogue": True,
                 **EXTRA_KNOBS}
        extra.update(knobs)
        cfg = DynaFlowConfig("dynaflow_amd.schedulers:DecoderOverlapScheduler", 2, InductorConfig(enabled=True),
                             CUDAGraphConfig(enabled=graphs is True, capture_sizes=[half, seqs]), extra)
        print(f"decode: mode {name}", file=sys.stderr, flush=True)
        manager = DynaFlowManager()
        torch._dynamo.reset()
        for t in inputs:
            torch._dynamo.mark_dynamic(t, 0)
        compiled = torch.compile(model, backend=make_backend(manager, cfg), fullgraph=True)
        with torch.no_grad():
            manager.prepare(seqs, [1] * seqs)
            compiled(*inputs)
            if graphs is True:   # capture every (nano-batch size, nano-batch index) sub-graph in a dry-run
                size = seqs if name.startswith("unsplit") else half
                manager.prepare(size, [1] * size, is_dryrun=True, use_cudagraph=True)
                compiled(*(t[:size].contiguous() for t in inputs))
                torch.cuda.synchronize()
            for _ in range(warmup):
                manager.prepare(seqs, [1] * seqs, use_cudagraph=bool(graphs))
                compiled(*inputs)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                manager.prepare(seqs, [1] * seqs, use_cudagraph=bool(graphs))
                y = compiled(*inputs)
            torch.cuda.synchronize()
            results[f"{name}_ms"] = (time.perf_counter() - t0) * 1e3 / steps
            if graphs == "whole":
                assert len(manager._schedule_graphs) == 1, "the step was not replayed as one graph"
            if name == "stream_per_nano_batch_planned_for_two_whole_graph":
                y_best = y.clone()
        del manager, compiled
    weight_bytes = layers * 2.0 * ((heads + 2 * kv_heads) * 128 * H + H * heads * 128 + 3 * H * I)
    kv_bytes = layers * 2.0 * seqs * kv_heads * capacity * 128 * 2
    # reported beside the two-stream nano-batch modes, never as `value`: the unsplit batch, and the serialized
    # issue of the same nano-batches (the baseline of the overlap figure)
    aside = {k: results.pop(k) for k in ("unsplit_sub_graph_replay_ms", "serialized_eager_ms",
                                          "serialized_whole_graph_ms", "one_stream_same_kernels_whole_graph_ms")
             if k in results}
    best_mode = min(results, key=results.get)
    best = results[best_mode]
    results.update(aside)

    sampled = [0, 127, 255]
    got_rows = y_best[sampled].float().cpu() if y_best is not None else None

    def oracle_check(mods):
        """The float64 oracle on the sampled tokens (a token's result depends on its own sequence only).  A decode
        step with fixed lengths rewrites only the position it appends to, which the oracle writes too, so the
        caches can be read after the timed steps."""
        from dynaflow_amd.decode import unpack_v_cache

        ref = mods["decode"]
        rows = slots[sampled].long()

        class Params(dict):
            def __getitem__(self, name):
                if name == "embed":
                    return model.embed.detach()[ids[sampled]].double().cpu()
                kind, i = name.rsplit(".", 1)
                a, m = model.attn[int(i)], model.mlp[int(i)]
                t = {"attn_norm": a.norm_weight, "wqkv": a.wqkv, "wo": a.wo, "mlp_norm": m.norm_weight,
                     "w_gate": m.w_gate, "w_up": m.w_up, "w_down": m.w_down}[kind]
                return t.detach().double().cpu()

        class Caches:
            def __init__(self, values):
                self.values = values

            def __len__(self):
                return layers

            def __getitem__(self, i):
                a = model.attn[i]
                c = unpack_v_cache(a.v_cache[rows]) if self.values else a.k_cache[rows]
                return c.double().cpu().permute(0, 2, 1, 3).contiguous()

        local = torch.arange(len(sampled))
        want = ref.decode_step(local, local, lengths[sampled].cpu(), Params(), Caches(False), Caches(True), heads,
                               kv_heads)
        return {"worst": rel_err_of(got_rows, want), "bound": 0.1, "rows": sampled,
                "against": "float64 oracle over all 32 layers on the sampled tokens; the bf16 roundings of the "
                           "residual stream add up over the layers (eager PyTorch in bf16 is 0.04 from the same "
                           "oracle), one layer's arithmetic is held to 2e-2 by the test suite"}

    line = {
        "metric": "decode-step tokens/s, 32 x 8B-shaped layers, bf16, 1 MI355X",
        "value": seqs / (best * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": best, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"decode step over {layers} Llama-3-8B-shaped layers, {seqs} single-token queries, "
                               f"{capacity} cached positions per sequence, 2 nano-batches of {half}, attention "
                               "sub-graph and MLP sub-graph per layer; the fastest of the issue modes timed in "
                               "this run is reported and named in issue_mode (by default: one stream per "
                               "nano-batch, kernels planned for the two launches of a kind that run side by side, "
                               "the whole split schedule replayed as one hipGraph)",
                   "issue_mode": best_mode[:-3]},
        "timings": results,
        "roofline": {"bound": "hbm", "achieved": (weight_bytes + kv_bytes) / (best * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": (weight_bytes + kv_bytes) / (best * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "algorithmic_bytes": weight_bytes + kv_bytes,
                     "note": "weights counted once per step (each nano-batch reads them again: 2x in practice)"},
        "oracle_check": oracle_check if got_rows is not None else None,
    }
    if "one_stream_same_kernels_whole_graph_ms" in results and \
            "stream_per_nano_batch_planned_for_two_whole_graph_ms" in results:
        # the same kernels and split on one stream against the two-stream schedule, graph against graph
        line["overlap_speedup"] = (results["one_stream_same_kernels_whole_graph_ms"]
                                   / results["stream_per_nano_batch_planned_for_two_whole_graph_ms"])
    if "serialized_eager_ms" in results:
        line["speedup_vs_serialized_lone_plans"] = min(results["serialized_eager_ms"],
                                                       results["serialized_whole_graph_ms"]) / best
    return line


def synthetic_inputs(torch, tokens, hidden, inter, dtype):
    """The layer's synthetic operands: x ~ N(0,1) pre-normed by RMSNorm (eps 1e-5, weight 1), W_gate / W_up /
    W_down ~ N(0, 0.02) in ``linear`` layout, one CPU generator per tensor (seeds 0 .. 3), made in fp32 and cast -
    the same bits on every box."""
    def normal(seed, shape, std):
        g = torch.Generator(device="cpu").manual_seed(seed)
        return torch.randn(shape, generator=g, dtype=torch.float32) * std

    x = normal(0, (tokens, hidden), 1.0)
    x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5)
    return (x.to(dtype), normal(1, (inter, hidden), 0.02).to(dtype), normal(2, (inter, hidden), 0.02).to(dtype),
            normal(3, (hidden, inter), 0.02).to(dtype))


def cpu_baseline(torch, sampled=None, other_checks=None, time_it=True):
    """The schedule restated with eager PyTorch on the host cores (the CPU oracle), on a bounded sample.  This leg is
    the only place where the bench touches the oracle: it times it and, with ``sampled = (x rows, W_gate, W_up,
    W_down, {name: the GPU result's same rows})``, checks the timed GPU results against its fp32 evaluation;
    ``other_checks``: {configuration: callable(oracle modules) -> error figures} for the other configurations'
    sampled rows.  ``time_it`` False: only those checks (returned as they are)."""
    from oracle import decode as oracle_decode
    from oracle import decoder as oracle_decoder
    from oracle import mlp as oracle_mlp

    modules = {"mlp": oracle_mlp, "decoder": oracle_decoder, "decode": oracle_decode}
    others = {name: check(modules) for name, check in (other_checks or {}).items() if check is not None}
    if not time_it:
        return others
    checks = {}
    if sampled is not None:
        x_rows, wg_s, wu_s, wd_s, got = sampled
        want = oracle_mlp.mlp_fp32_from(x_rows, wg_s, wu_s, wd_s)
        for name, rows in got.items():
            checks[name] = ((rows - want).abs().max() / want.abs().max()).item()
    sample_tokens = 512
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    x, wg, wu, wd = oracle_mlp.make_inputs(sample_tokens, HIDDEN, INTER, torch.float32, prenorm=True)
    split = [0, sample_tokens // 2, sample_tokens]
    oracle_mlp.mlp_schedule(x, wg, wu, wd, split)
    times = []
    budget_start = time.perf_counter()
    while len(times) < 10 and time.perf_counter() - budget_start < 20.0:
        t0 = time.perf_counter()
        oracle_mlp.mlp_schedule(x, wg, wu, wd, split)
        times.append(time.perf_counter() - t0)
    times.sort()
    median = times[len(times) // 2]
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    # the reference's own CPU-runnable case at its exact size: x[256,1024] fp32, I=2816, 2 nano-batches of 128
    c1 = oracle_mlp.make_inputs(256, 1024, 2816, torch.float32)
    c1_split = [0, 128, 256]
    for _ in range(3):
        oracle_mlp.mlp_schedule(*c1, c1_split)
    c1_times = []
    for _ in range(15):
        t0 = time.perf_counter()
        oracle_mlp.mlp_schedule(*c1, c1_split)
        c1_times.append(time.perf_counter() - t0)
    c1_times.sort()
    c1_median = c1_times[len(c1_times) // 2]
    return {
        "gpu_results_rel_err_vs_fp32_oracle_sampled_rows": checks,
        "other_configs_rel_err_vs_oracle_sampled_rows": others,
        "value": sample_tokens / median,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "config1_cpu_case": {
            "workload": "x[256,1024] fp32, W_gate/W_up [1024,2816], W_down [2816,1024], 2 nano-batches of 128, "
                        "eager PyTorch on all host cores, median of 15 runs after 3 warm-ups",
            "ms": c1_median * 1e3, "tokens_per_s": 256 / c1_median,
            "gflops": 6.0 * 256 * 1024 * 2816 / c1_median / 1e9,
        },
        "sample": f"{sample_tokens} of {TOKENS} tokens of the same layer (H={HIDDEN}, I={INTER}) in fp32, "
                  f"2 nano-batches of {sample_tokens // 2}, eager PyTorch, median of {len(times)} runs",
        "gflops": 6.0 * sample_tokens * HIDDEN * INTER / median / 1e9,
        "cpu_model": model,
        "os_cpu_count": os.cpu_count(),
    }


#: the issue mode that `value` is measured in (fixed, not the best of several): one stream per nano-batch, the
#: gate/up GEMM with the SiLU*mul as its epilogue, kernels planned for the two launches of a kind that run side by
#: side (the manager derives that from the stream policy), the whole two-stream schedule as one hipGraph
HEADLINE_KNOBS = {"whole_graph": True, "fuse_silu_epilogue": True, "streams": "by_nano_batch"}
HEADLINE_MODE = "overlapped_hipgraph+silu_mul_epilogue+staggered+stream_per_nano_batch+kernels_planned_for_the_pair"


def headline_workload(mb):
    return (f"Llama-3-8B-shaped SwiGLU MLP layer, x[{TOKENS},{HIDDEN}] bf16 pre-normed, I={INTER}, {SPLITS} "
            f"nano-batches of {mb} tokens, each on a HIP stream of its own: per nano-batch ONE launch for the gate "
            "and up projections with the SiLU*mul as its epilogue, then the down projection; the two nano-batches' "
            "launches of the same kind run side by side (the gate/up/SiLU launch of nano-batch 1 beside that of "
            "nano-batch 0, then the two down projections) with kernels planned for the pair; the whole two-stream "
            "schedule replayed as one hipGraph")


def other_configs(torch, args):
    """The other three GPU configurations with few steps each, for the one default line: (name, figures, check)
    with ``check(oracle modules) -> error of sampled rows`` run later by the CPU leg."""
    out, checks = {}, {}
    steps, warmup = max(5, args.steps // 4), max(3, args.warmup // 2)
    for name, fn in (("decoder_layer_prefill_8x2048", decoder_config), ("fp8_mlp_70b_shape", fp8_config),
                     ("decode_step_32_layers", decode_config)):
        print(f"bench.py: other configuration {name}", file=sys.stderr, flush=True)
        line = fn(torch, steps, warmup, brief=True)
        checks[name] = line.pop("oracle_check", None)
        out[name] = {k: line[k] for k in ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "dtype", "config",
                                          "roofline", "timings") if k in line}
        for extra in ("layer", "overlap_speedup"):
            if extra in line:
                out[name][extra] = line[extra]
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    return out, checks


def main() -> int:
    args = parse_args()
    read_knobs(args.knob)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported in this build "
              "(the path has no multi-GPU part)", file=sys.stderr)
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (no GPU visible)", file=sys.stderr)
        return 2
    from dynaflow_amd import _cabi, ops

    _cabi.load()
    info = _cabi.device_info(0)
    single = [(args.decoder, decoder_config), (args.decode, decode_config), (args.fp8, fp8_config)]
    for wanted, fn in single:
        if wanted:
            line = fn(torch, max(5, args.steps // 5), max(3, args.warmup // 5))
            check = line.pop("oracle_check", None)
            if check is not None and not args.skip_cpu:
                line["rel_err_vs_oracle_sampled_rows"] = cpu_baseline(torch, None, {"this": check}, time_it=False)["this"]
            print(json.dumps(line))
            return 0
    if args.decode_kernels:
        line = decode_kernels(torch, ops, max(20, args.steps))
        line["projections"] = decode_projections(torch, ops, max(20, args.steps))
        print(json.dumps(line))
        return 0
    if args.decode_projection_launches:
        print(json.dumps(decode_projection_launches(torch, ops, max(16, args.steps))))
        return 0
    if args.prefill_attention_kernels:
        print(json.dumps(prefill_attention_kernels(torch, ops, max(20, args.steps))))
        return 0
    x_cpu, wg, wu, wd = synthetic_inputs(torch, TOKENS, HIDDEN, INTER, torch.bfloat16)
    x = x_cpu.cuda()
    weights = (wg.cuda(), wu.cuda(), wd.cuda())

    if args.kernels_only:
        if args.operands == "zeros":
            x.zero_()
            for w in weights:
                w.zero_()
        print(json.dumps(single_kernels(torch, ops, x, weights, max(20, args.steps), calibration_copy=True)))
        return 0

    settle = args.settle_seconds
    if args.headline_only:
        m_h, c_h = build_path(torch, x, weights, **HEADLINE_KNOBS)
        ms_h, _ = time_steps(torch, m_h, c_h, x, args.steps, args.warmup, use_graph=True, settle_s=settle)
        print(json.dumps({"mode": HEADLINE_MODE, "ms_per_step": ms_h, "steps": args.steps}))
        return 0

    mb = TOKENS // SPLITS
    # ---- the headline mode first: straight after its set-up (the GPU has idled through the trace), then with the
    # package settled - every timed loop of this run is preceded by `settle` seconds of the same step, untimed, so
    # that the modes are compared in one state of the clocks; W warm-up steps and exactly K timed steps follow
    m_head, c_head = build_path(torch, x, weights, **HEADLINE_KNOBS)
    assert m_head.launches_side_by_side(m_head.prepare(TOKENS, [TOKENS])) == SPLITS
    ms_head_from_idle, _ = time_steps(torch, m_head, c_head, x, args.steps, args.warmup, use_graph=True)
    ms_head, y_head = time_steps(torch, m_head, c_head, x, args.steps, args.warmup, use_graph=True, settle_s=settle)
    y_head = y_head.clone()
    load_s = args.sustain_seconds
    ms_sustained = sustained_steps(torch, m_head, c_head, x, args.steps, load_s) if load_s > 0 else None
    # the same kernels and the same split on ONE stream, as one graph: the baseline of `overlap_speedup`
    m_h1, c_h1 = build_path(torch, x, weights, serialize=True, whole_graph=True, fuse_silu_epilogue=True,
                            side_by_side=SPLITS)
    ms_head_one_stream, y_head_one_stream = time_steps(torch, m_h1, c_h1, x, args.steps, args.warmup, use_graph=True,
                                                       settle_s=settle)
    head_identical = bool(torch.equal(y_head, y_head_one_stream))

    # ---- separate kernels (gate GEMM, up GEMM, SiLU*mul, down GEMM): every launch on one stream, eagerly and as one
    # graph; then the north star's own pattern - streams by sub-graph kind, staggered: the gate/up GEMMs of nano-batch
    # 1 beside SiLU*mul + down projection of nano-batch 0
    m_ser, c_ser = build_path(torch, x, weights, serialize=True, whole_graph=True)
    ms_serial, y_serial = time_steps(torch, m_ser, c_ser, x, args.steps, args.warmup, use_graph=False, settle_s=settle)
    y_serial = y_serial.clone()
    ms_serial_gpu = gpu_time_of_steps(torch, m_ser, c_ser, x, min(args.steps, 20))
    ms_serial_graph, y_serial_graph = time_steps(torch, m_ser, c_ser, x, args.steps, args.warmup, use_graph=True,
                                                 settle_s=settle)
    serial_graph_identical = bool(torch.equal(y_serial, y_serial_graph))
    m_ovl, c_ovl = build_path(torch, x, weights, whole_graph=True)
    ms_eager, y_eager = time_steps(torch, m_ovl, c_ovl, x, args.steps, args.warmup, use_graph=False, settle_s=settle)
    y_eager = y_eager.clone()
    ms_graph, y_graph = time_steps(torch, m_ovl, c_ovl, x, args.steps, args.warmup, use_graph=True, settle_s=settle)
    identical = bool(torch.equal(y_serial, y_eager) and torch.equal(y_eager, y_graph))
    y_graph = y_graph.clone()
    # the same separate kernels with one stream per nano-batch, planned for the pair
    m_op, c_op = build_path(torch, x, weights, whole_graph=True, streams="by_nano_batch")
    ms_graph_pair, y_graph_pair = time_steps(torch, m_op, c_op, x, args.steps, args.warmup, use_graph=True,
                                             settle_s=settle)
    y_graph_pair = y_graph_pair.clone()
    m_ops, c_ops = build_path(torch, x, weights, serialize=True, side_by_side=SPLITS)
    _, y_serial_pair = time_steps(torch, m_ops, c_ops, x, 2, 1, use_graph=False)
    pair_identical = bool(torch.equal(y_serial_pair, y_graph_pair))

    # ---- the SiLU*mul as the epilogue of one gate/up GEMM, in the other issue modes
    m_fs, c_fs = build_path(torch, x, weights, serialize=True, whole_graph=True, fuse_silu_epilogue=True)
    ms_fused_serial, yf_serial = time_steps(torch, m_fs, c_fs, x, args.steps, args.warmup, use_graph=False,
                                            settle_s=settle)
    yf_serial = yf_serial.clone()
    ms_fused_serial_gpu = gpu_time_of_steps(torch, m_fs, c_fs, x, min(args.steps, 20))
    ms_fused_serial_graph, _ = time_steps(torch, m_fs, c_fs, x, args.steps, args.warmup, use_graph=True,
                                          settle_s=settle)
    # the north star's pattern again (streams by kind, staggered): the fused GEMM of nano-batch 1 beside the down
    # projection of nano-batch 0
    m_fo, c_fo = build_path(torch, x, weights, whole_graph=True, fuse_silu_epilogue=True)
    ms_fused_graph, yf_graph = time_steps(torch, m_fo, c_fo, x, args.steps, args.warmup, use_graph=True,
                                          settle_s=settle)
    yf_graph = yf_graph.clone()
    # weights-major orders (both nano-batches' launches against the same weights back to back; the second finds most
    # of them in the memory-side cache), kernels planned as lone launches: one stream per nano-batch, or the
    # round-robin schedule (the NanoFlow order of the reference)
    m_fn, c_fn = build_path(torch, x, weights, whole_graph=True, fuse_silu_epilogue=True, streams="by_nano_batch",
                            side_by_side=1)
    ms_fused_graph_nb, yf_graph_nb = time_steps(torch, m_fn, c_fn, x, args.steps, args.warmup, use_graph=True,
                                                settle_s=settle)
    yf_graph_nb = yf_graph_nb.clone()
    m_fr, c_fr = build_path(torch, x, weights, whole_graph=True, fuse_silu_epilogue=True, schedule="round_robin")
    ms_fused_graph_rr, yf_graph_rr = time_steps(torch, m_fr, c_fr, x, args.steps, args.warmup, use_graph=True,
                                                settle_s=settle)
    yf_graph_rr = yf_graph_rr.clone()
    fused_identical = all(bool(torch.equal(yf_serial, other)) for other in (yf_graph, yf_graph_nb, yf_graph_rr))
    fused_modes = {"+staggered+streams_by_sub_graph_kind": (ms_fused_graph, yf_graph),
                   "+staggered+stream_per_nano_batch": (ms_fused_graph_nb, yf_graph_nb),
                   "+round_robin+streams_by_sub_graph_kind": (ms_fused_graph_rr, yf_graph_rr),
                   "+staggered+stream_per_nano_batch+kernels_planned_for_the_pair": (ms_head, y_head)}
    fastest_fused_mode = min(fused_modes, key=lambda m: fused_modes[m][0])

    # ---- for comparison only: the 4096 tokens as ONE batch (no nano-batches, one stream, two launches)
    m_un, c_un = build_path(torch, x, weights, min_nano_split_tokens=1 << 30, fuse_silu_epilogue=True)
    ms_unsplit_gpu = gpu_time_of_steps(torch, m_un, c_un, x, min(args.steps, 20))
    # for scale: the same layer on the whole batch through PyTorch's own operators (the vendor GEMM library and aten's
    # SiLU and multiplication), replayed as one graph on one stream so that no host time is in the figure
    ms_vendor = vendor_library_layer(torch, x, weights, args.steps, args.warmup, settle)

    if not (head_identical and fused_identical and identical and serial_graph_identical and pair_identical):
        print("bench.py: issue modes that run the same kernels disagree bit for bit: "
              f"headline vs its one-stream issue {head_identical}, fused modes {fused_identical}, separate kernels "
              f"{identical and serial_graph_identical}, pair plan {pair_identical}", file=sys.stderr)
        return 1

    # ---- sampled rows of the timed results, checked against the fp32 oracle (same bf16 operands) in the CPU leg
    rows = torch.tensor([0, 2047, 2048, 4095])
    sampled = (x_cpu[rows], wg, wu, wd, {"separate_kernels_graph": y_graph[rows].float().cpu(),
                                         "headline_mode": y_head[rows].float().cpu(),
                                         "fused_lone_plans": yf_graph[rows].float().cpu()})

    # ---- single kernels, HIP events on the launching stream
    k = single_kernels(torch, ops, x, weights, max(20, args.steps))
    ms_gate, ms_down, ms_silu, ms_blas = k["gate_ms"], k["down_ms"], k["silu_ms"], k["blas_ms"]
    ms_gus = k["gate_up_silu_ms"]
    ms_gus_pair, ms_down_pair = k["gate_up_silu_pair_ms"], k["down_pair_ms"]
    gemm_flops = 2.0 * mb * HIDDEN * INTER          # one projection of one nano-batch
    silu_bytes = 3.0 * mb * INTER * 2               # read gate + up, write out
    layer_flops = 6.0 * TOKENS * HIDDEN * INTER
    # the same launches on all-zero operands: the same instructions, memory traffic and stalls, but no bit toggles in
    # the data paths, so the package stays below its power limit and the clocks stay up
    x_zero, w_zero = torch.zeros_like(x), tuple(torch.zeros_like(w) for w in weights)
    kz = single_kernels(torch, ops, x_zero, w_zero, max(20, args.steps))
    m_z, c_z = build_path(torch, x_zero, w_zero, **HEADLINE_KNOBS)
    ms_head_zero, _ = time_steps(torch, m_z, c_z, x_zero, args.steps, args.warmup, use_graph=True, settle_s=settle)
    del m_z, c_z

    result = {
        "metric": METRIC,
        "value": TOKENS / (ms_head * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_head,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": headline_workload(mb),
            "issue_mode": HEADLINE_MODE,
            "device": info["arch_name"],
            "compute_units": info["compute_units"],
            # every timed loop: `settle` seconds of the same step untimed (clocks of the package in their loaded
            # state), then W warm-up steps, then exactly K timed steps between two device synchronisations
            "settle_seconds_before_each_timed_loop": settle,
            "ms_per_step_straight_after_set_up": ms_head_from_idle,
        },
        # the overlap figure of the measurement plan: the same kernels and the same split issued on one stream against
        # the two-stream schedule, both replayed as one hipGraph
        "overlap_speedup": ms_head_one_stream / ms_head,
        "overlap_speedup_parts": {
            "one_stream_same_kernels_graph_ms": ms_head_one_stream,
            "two_streams_graph_ms": ms_head,
            "what_runs_side_by_side": "launches of the same kind: gate/up/SiLU of both nano-batches, then both down "
                                      "projections (a lone launch of these plans fills half the compute units)",
            # the one-stream schedule in ITS best form (kernels planned as lone launches)
            "one_stream_lone_plans_graph_ms": ms_fused_serial_graph,
            "speedup_vs_one_stream_lone_plans_graph": ms_fused_serial_graph / ms_head,
            "outputs_bit_identical_to_the_one_stream_issue": head_identical,
        },
        # the pattern the north star names - streams by sub-graph kind, staggered: the GEMM sub-graph of nano-batch 1
        # beside SiLU*mul + down projection of nano-batch 0 - against the same kernels on one stream, graph vs graph
        "north_star_pattern_gemm_beside_tail_of_previous_nano_batch": {
            "separate_silu_mul_kernel": {"one_stream_graph_ms": ms_serial_graph, "two_streams_graph_ms": ms_graph,
                                         "speedup": ms_serial_graph / ms_graph},
            "silu_mul_as_gemm_epilogue": {"one_stream_graph_ms": ms_fused_serial_graph,
                                          "two_streams_graph_ms": ms_fused_graph,
                                          "speedup": ms_fused_serial_graph / ms_fused_graph},
        },
        # reported beside the nano-batch schedule, never as `value`: every operator of this layer is MFMA-bound, so
        # on one GPU two nano-batches have nothing of a different kind to hide behind each other
        "unsplit_one_batch": {"silu_mul_as_gemm_epilogue_gpu_side_ms": ms_unsplit_gpu,
                              "pytorch_operators_one_graph_ms": ms_vendor,
                              "headline_over_pytorch_operators": ms_vendor / ms_head},
        "overlap": {
            "serialized_ms": ms_serial,
            "serialized_gpu_side_ms": ms_serial_gpu,
            "serialized_graph_ms": ms_serial_graph,
            "overlapped_eager_ms": ms_eager,
            "overlapped_graph_ms": ms_graph,
            "overlapped_graph_stream_per_nano_batch_planned_for_the_pair_ms": ms_graph_pair,
            "speedup_best_vs_serialized_graph": ms_serial_graph / min(ms_graph, ms_graph_pair),
            "planned_for_the_pair_bit_identical_to_its_serialized_issue": pair_identical,
            "speedup_eager_vs_serialized": ms_serial / ms_eager,
            "speedup_graph_vs_serialized": ms_serial / ms_graph,
            "speedup_graph_vs_serialized_gpu_side": ms_serial_gpu / ms_graph,
            "speedup_graph_vs_serialized_graph": ms_serial_graph / ms_graph,
            "outputs_bit_identical": identical and serial_graph_identical,
        },
        "silu_mul_as_gemm_epilogue": {
            "serialized_ms": ms_fused_serial,
            "serialized_gpu_side_ms": ms_fused_serial_gpu,
            "serialized_graph_ms": ms_fused_serial_graph,
            "overlapped_graph_ms": ms_fused_graph,
            "overlapped_graph_stream_per_nano_batch_ms": ms_fused_graph_nb,
            "overlapped_graph_round_robin_ms": ms_fused_graph_rr,
            "overlapped_graph_stream_per_nano_batch_planned_for_the_pair_ms": ms_head,
            "speedup_graph_vs_serialized": ms_fused_serial / ms_fused_graph,
            "speedup_graph_vs_serialized_gpu_side": ms_fused_serial_gpu / ms_fused_graph,
            "speedup_graph_vs_serialized_graph": ms_fused_serial_graph / ms_fused_graph,
            "fastest_mode_of_this_run": fastest_fused_mode[1:],
            "headline_mode_ms": ms_head,
            "speedup_headline_vs_serialized": ms_fused_serial / ms_head,
            "speedup_headline_vs_serialized_graph": ms_fused_serial_graph / ms_head,
            "outputs_bit_identical": fused_identical,
            "planned_for_the_pair_bit_identical_to_its_serialized_issue": head_identical,
        },
        "layer": {
            "tflops": layer_flops / (ms_head * 1e-3) / 1e12,
            "frac_of_bf16_mfma_peak": layer_flops / (ms_head * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
        },
        "kernels": {
            "gate_or_up_gemm": {"ms": ms_gate, "tflops": gemm_flops / (ms_gate * 1e-3) / 1e12},
            "down_gemm": {"ms": ms_down, "tflops": gemm_flops / (ms_down * 1e-3) / 1e12},
            "silu_mul": {"ms": ms_silu, "gbs": silu_bytes / (ms_silu * 1e-3) / 1e9,
                         "frac_of_hbm_peak": silu_bytes / (ms_silu * 1e-3) / 1e9 / HBM_PEAK_GBS},
            "gate_up_silu_gemm": {"ms": ms_gus, "tflops": 2 * gemm_flops / (ms_gus * 1e-3) / 1e12},
            "rocblas_same_gemm_for_scale": {"ms": ms_blas, "tflops": gemm_flops / (ms_blas * 1e-3) / 1e12},
            # two loops of launches side by side on two streams, kernels planned for the pair; ms per pair
            "gate_up_silu_gemm_pair": {"ms": ms_gus_pair, "tflops": 4 * gemm_flops / (ms_gus_pair * 1e-3) / 1e12},
            "down_gemm_pair": {"ms": ms_down_pair, "tflops": 2 * gemm_flops / (ms_down_pair * 1e-3) / 1e12},
        },
        # the reference's stand-alone experiment (examples/ae/up-silu-overlap.cu:320-341: GEMM only, SiLU only,
        # serial = their sum, the fused kernel, speedup = serial / fused, FUSED / GEMM) on one nano-batch of this
        # layer, from the single-kernel loops above: the GEMM is the gate and the up projection as two launches
        "gate_up_silu_experiment": {
            "gemm_only_us": 2e3 * ms_gate,
            "silu_only_us": 1e3 * ms_silu,
            "serial_us": 2e3 * ms_gate + 1e3 * ms_silu,
            "fused_us": 1e3 * ms_gus,
            "speedup_fused_vs_serial": (2 * ms_gate + ms_silu) / ms_gus,
            "fused_over_gemm_only": ms_gus / (2 * ms_gate),
            "fused_us_beside_the_other_nano_batch": 0.5e3 * ms_gus_pair,
            "speedup_fused_beside_the_other_nano_batch_vs_serial": (2 * ms_gate + ms_silu) / (0.5 * ms_gus_pair),
        },
        # the layer the same way: separate GEMM and SiLU*mul launches of both nano-batches one after the other on
        # one stream (the reference's serial baseline) against the issue mode that `value` comes from
        "speedup_best_vs_serialized_separate_kernels": ms_serial / ms_head,
        "speedup_best_vs_serialized_separate_kernels_graph": ms_serial_graph / ms_head,
    }
    # the dominant kernel of the issue mode that `value` comes from
    result["roofline"] = {
        "kernel": GATE_UP_SILU_PAIR_KERNEL + " (gate and up projection of one nano-batch with the SiLU*mul epilogue: "
                  "[2048,4096] x 2 x [14336,4096]^T -> act[2048,14336]); the two nano-batches' launches run side by "
                  "side on two streams and are timed as pairs (two loops of launches, one per stream)",
        "bound": "mfma",
        "achieved": 4 * gemm_flops / (ms_gus_pair * 1e-3) / 1e12,
        "peak": BF16_MFMA_PEAK_TFLOPS,
        "unit": "TFLOP/s",
        "frac": 4 * gemm_flops / (ms_gus_pair * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
        "launches_timed_together": 2,
        # per launch, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy of known size; algorithmic:
        # 16.8 + 2 x 117.4 MB read, 58.7 MB written
        "traffic": GATE_UP_SILU_SQUARE_TRAFFIC_BYTES,
        "traffic_unit": "bytes per launch",
    }
    # how much of the distance to the peak is the package power limit: the same pairs on all-zero operands
    result["power_limit_check"] = {
        "what": "the same launches timed the same way on all-zero operands (same instructions, memory traffic and "
                "stalls; no bit toggles, so the package stays below its 1400 W limit and the clocks stay up)",
        "gate_up_silu_pair_ms": {"synthetic_operands": ms_gus_pair, "zero_operands": kz["gate_up_silu_pair_ms"]},
        "down_pair_ms": {"synthetic_operands": ms_down_pair, "zero_operands": kz["down_pair_ms"]},
        "gate_up_silu_pair_frac_of_peak_on_zero_operands":
            4 * gemm_flops / (kz["gate_up_silu_pair_ms"] * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
        "down_pair_frac_of_peak_on_zero_operands":
            2 * gemm_flops / (kz["down_pair_ms"] * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
        "rocblas_same_gemm_ms": {"synthetic_operands": ms_blas, "zero_operands": kz["blas_ms"]},
        # the whole headline step (same issue mode, same graph shape) on a zero input and zero weights
        "layer_ms_per_step": {"synthetic_operands": ms_head, "zero_operands": ms_head_zero},
        "layer_frac_of_peak_on_zero_operands": layer_flops / (ms_head_zero * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
    }
    # ---- the same figures under sustained load
    if load_s > 0:
        mb_x = x[:mb]
        halves = (x[:mb], x[mb:2 * mb])
        with torch.no_grad():
            def pair_of(i):
                with ops.launch_options(side_by_side=SPLITS):
                    return ops.gate_up_silu(halves[i], weights[0], weights[1])

            until = time.perf_counter() + load_s
            while time.perf_counter() < until:
                for _ in range(50):
                    ops.gate_up_silu(mb_x, weights[0], weights[1])
                torch.cuda.synchronize()
            ms_k_pair = time_pair(torch, pair_of, max(20, args.steps), warmup=5)
        result["sustained"] = {
            "method": f"the same graph replay / the same pair of launches timed right after {load_s:g} s of running "
                      "the step / the kernel back to back (package at its power limit, clocks settled)",
            "load_seconds": load_s,
            "ms_per_step": ms_sustained,
            "value": TOKENS / (ms_sustained * 1e-3),
            "layer_frac_of_bf16_mfma_peak": layer_flops / (ms_sustained * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
            "dominant_kernel_pair_ms": ms_k_pair,
            "dominant_kernel_frac": 4 * gemm_flops / (ms_k_pair * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS,
        }
    checks = {}
    if not args.headline_config_only:
        del m_head, c_head, m_h1, c_h1, m_ser, c_ser, m_ovl, c_ovl, m_op, c_op, m_ops, c_ops, m_fs, c_fs, m_fo, c_fo
        del m_fn, c_fn, m_fr, c_fr, m_un, c_un, weights, x
        torch.cuda.empty_cache()
        result["other_configs"], checks = other_configs(torch, args)
    if not args.skip_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, sampled, checks)
        worst = max(result["cpu_baseline"]["gpu_results_rel_err_vs_fp32_oracle_sampled_rows"].values())
        if not worst < 2e-2:
            print(f"bench.py: the timed result is off the fp32 oracle by {worst:.3g} (bf16 bound 2e-2)", file=sys.stderr)
            return 1
        for name, err in result["cpu_baseline"].pop("other_configs_rel_err_vs_oracle_sampled_rows", {}).items():
            result["other_configs"][name]["rel_err_vs_oracle_sampled_rows"] = err
            bound = 5e-2 if "fp8" in name else 0.1 if "decode_step" in name else 2e-2
            if not err["worst"] < bound:
                print(f"bench.py: {name}: sampled rows are off the oracle by {err['worst']:.3g} (bound {bound})",
                      file=sys.stderr)
                return 1
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
