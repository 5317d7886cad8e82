"""Benchmark of the paged decode-attention hot path on one MI355X.

A step is one call of the decode op (split-KV GQA attention, then the merge launch that also appends the new token)
for one layer over one batch of synthetic sequences.  The headline workload is the Qwen2.5-7B-like shape (B=64, 28 q heads /
4 kv heads, D=128, page 16, contexts uniform in [512, 4096]) with an int8 KV cache (quantizing append included), the
configuration the bandwidth target is stated on; the same shape with a bf16 cache, the fp8 rollout shape and the fp8
prefill shape are measured too and reported under "workloads" (next to a few decode shapes beside the benchmark's and
the backward of the varlen op).  Inputs are resident in HBM before timing starts.  Steps rotate over several copies
of the KV pools so that the working set exceeds the 256 MB Infinity Cache and the reads really come from HBM.

Prints ONE JSON line.  `value` is microseconds per step: the median of 15 timings of exactly `--steps` steps replayed
from HIP graphs (how the engine runs decode), `value_p10_p90` their spread.  The steps run as an engine runs the
layers of a model: block table and lengths are the same for every layer of a decode step, so one plan launch
(`areno_hip_paged_decode_plan`) serves 28 steps; it is part of the timed sequence.  `value_without_plan` is the same
sequence with every step deriving its work list by itself.  Every timing is bracketed by `torch.cuda.synchronize()`,
so it carries the host's launch of the first graph and its wake-up once (`host_bracket_us`, timed by itself on a
graph of one tiny kernel: 30-45 us, i.e. ~0.2 us per step at the default 200 steps and ~1.5 us at 20);
`value_on_device` is the same samples by events on the stream, without that.  `roofline` is for the split-KV kernel alone: algorithmic
bytes of one launch divided by its mean duration measured with events on the launch stream, next to what a plain reader
of the same pools reaches (`stream_ceiling_*`); `cpu_baseline` is the CPU oracle timed on the host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
POOL_TARGET_BYTES = 1.3e9  # rotate over at least this much distinct KV
# HBM bytes per launch of the dominant kernel as two rocprofv3 counter runs of this script recorded them (FETCH_SIZE,
# scaled by the factor 2.0 that a copy of known size gives for it, plus WRITE_SIZE).  Recorded constants, not
# measurements of the present run: the summaries they come from are under profiles/.
PROFILED_TRAFFIC_BYTES = {"cfg1-qwen7b-bf16": 311.03e6, "cfg2-qwen7b-int8": 153.97e6, "cfg3-rollout-fp8": 1065.92e6,
                          "cfg4-prefill-fp8": 1624.87e6}
PROFILED_TRAFFIC_SOURCE = {
    "decode": "recorded from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script: profiles/decode_mfma_kernel_hbm_traffic_cfg1_cfg2_cfg3.md",
    "prefill": "recorded from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script: profiles/prefill_mfma_kernel_hbm_traffic_cfg4.md",
}


def _clone_pools(w, copies):
    pools = [(w.k_cache, w.v_cache, w.k_scale, w.v_scale)]
    for _ in range(copies - 1):
        pools.append(tuple(None if t is None else t.clone() for t in pools[0]))
    return pools


def _gpu_quantize(x, cache_dtype):
    import torch

    from areno_amd.accel import attention as ops

    n, hkv, d = x.shape
    sdt = torch.float16 if cache_dtype == torch.int8 else torch.float32
    kc = torch.empty((n, 1, hkv, d), dtype=cache_dtype, device=x.device)
    vc = torch.empty_like(kc)
    ks = torch.empty((n, 1, hkv), dtype=sdt, device=x.device)
    vs = torch.empty_like(ks)
    ids = torch.arange(n, device=x.device, dtype=torch.int64)
    ops.areno_paged_cache_write(x, x, kc, vc, ids, torch.zeros_like(ids), k_scale=ks, v_scale=vs)
    return kc.view(n, hkv, d), ks.view(n, hkv)


LAYERS_PER_PLAN = 28  # layers of the Qwen2.5-7B-like model the shapes come from: one plan serves the layers of a step


def _groups(w):
    if "shared_prefix_lens" in w.meta:  # what the rollout scheduler knows: rows per prompt, shared tokens per prompt
        return dict(prefix_group_rows=w.meta["prefix_group_rows"], shared_prefix_lens=w.meta["shared_prefix_lens"])
    return {}


def _plan(w, pool, buffer=None):
    from areno_amd.accel import attention as ops

    kc, vc, ks, vs = pool
    return ops.areno_paged_decode_plan(w.block_table, w.cache_seqlens, kc, vc, q_heads=w.q.shape[1], q_dtype=w.q.dtype,
                                       k_scale=ks, v_scale=vs, buffer=buffer, **_groups(w))  # fmt: skip


def _step(w, pool, plan=None):
    from areno_amd.accel import attention as ops

    kc, vc, ks, vs = pool
    return ops.areno_paged_causal_attention_decode(
        w.q, w.k_update, w.v_update, kc, vc, w.block_table, w.cache_seqlens,
        softmax_scale=w.softmax_scale, k_scale=ks, v_scale=vs, plan=plan, **_groups(w),
    )  # fmt: skip


def _parity_sample(w, out, rows=4):
    """Max-abs error of the first rows against the CPU oracle (dequantized cache for int8/fp8)."""
    from oracle import attention_ref as ar
    from oracle import quant_ref as qr

    if w.k_scale is None:
        kc, vc = w.k_cache.cpu().float(), w.v_cache.cpu().float()
    else:
        kc, vc = qr.dequantize(w.k_cache.cpu(), w.k_scale.cpu()), qr.dequantize(w.v_cache.cpu(), w.v_scale.cpu())
    want = ar.ref_paged_decode(
        w.q[:rows].cpu().float(), kc, vc, w.block_table[:rows].cpu(), w.cache_seqlens[:rows].cpu(), -1, w.softmax_scale
    )
    return float((out[:rows].cpu().float() - want).abs().max())


def measure_decode(w, steps, warmup, *, kernel_iters=20, kernel_samples=15, repeats=15, plan_mode="both"):
    """Time the whole op (graph replay and eager) and each kernel of it; returns a dict of numbers.

    A step is one layer's decode op.  The layers of a model's decode step share block table and lengths, so the timed
    sequence is what an engine runs: one plan launch, then LAYERS_PER_PLAN ops that use it, each on another layer's
    pools, replayed from HIP graphs; the plan launch is inside the timed region and its cost is spread over the steps
    it serves.  The same sequence without plans is timed next to it (`plan_mode` "only" / "off" leave one of the two
    out, so that a profiler's per-kernel averages belong to one of them)."""
    import torch

    from areno_amd.accel import cabi

    pool_bytes = sum(t.numel() * t.element_size() for t in (w.k_cache, w.v_cache, w.k_scale, w.v_scale) if t is not None)
    copies = max(2, int(-(-POOL_TARGET_BYTES // pool_bytes)))
    pools = _clone_pools(w, copies)
    alg_bytes = w.algorithmic_bytes()

    out = _step(w, pools[0])
    torch.cuda.synchronize()
    parity = _parity_sample(w, out)
    planned_equal = bool(torch.equal(_step(w, pools[0], _plan(w, pools[0])), out))
    plan_mode = plan_mode if plan_mode in ("both", "only", "off") else "both"

    # ---- whole op, replayed from HIP graphs ---------------------------------------------------------------------------
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for pool in pools:
            _step(w, pool, _plan(w, pool))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    plan_buffer = torch.empty(cabi.decode_plan_bytes(w.q.shape[0]), dtype=torch.uint8, device=w.q.device)

    def capture(n, planned, first_pool=0):
        """A graph of n steps: with plans, a plan launch in front of every LAYERS_PER_PLAN steps."""
        g = torch.cuda.CUDAGraph()
        keep = []
        with torch.cuda.graph(g):
            plan = None
            for i in range(n):
                pool = pools[(first_pool + i) % copies]
                if planned and i % LAYERS_PER_PLAN == 0:
                    plan = _plan(w, pool, plan_buffer)
                keep.append(_step(w, pool, plan))
        return g, keep

    def timed_replays(planned):
        """us/step over exactly `steps` steps, `repeats` times."""
        full_n = min(steps, LAYERS_PER_PLAN * max(1, copies // LAYERS_PER_PLAN + 1))
        full_n -= full_n % LAYERS_PER_PLAN if full_n >= LAYERS_PER_PLAN else 0
        full, keep_full = capture(full_n, planned)
        rem_n = steps % full_n
        rem, _ = capture(rem_n, planned) if rem_n else (None, None)
        for _ in range(max(1, -(-warmup // full_n))):
            full.replay()
        torch.cuda.synchronize()
        samples, on_device = [], []
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(repeats):
            t0 = time.perf_counter()
            first.record()
            for _ in range(steps // full_n):
                full.replay()
            if rem is not None:
                rem.replay()
            last.record()
            torch.cuda.synchronize()
            samples.append((time.perf_counter() - t0) / steps * 1e6)
            on_device.append(first.elapsed_time(last) * 1e3 / steps)
        samples.sort()
        # graph replays must reproduce the eager result (checked on the first pool)
        return (statistics.median(samples), [samples[len(samples) // 10], samples[(len(samples) * 9) // 10]],
                bool(torch.equal(keep_full[0], out)), statistics.median(on_device))  # fmt: skip

    def host_bracket():
        """What the bracket around a timed sample costs by itself: the host's launch of one graph and its wake-up from
        torch.cuda.synchronize(), on a graph of one tiny kernel.  A sample of `steps` steps carries it once."""
        flag = torch.zeros(1, device=w.q.device)
        side2 = torch.cuda.Stream()
        side2.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side2):
            flag.zero_()
        torch.cuda.current_stream().wait_stream(side2)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            flag.zero_()
        times = []
        for _ in range(31):
            t0 = time.perf_counter()
            g.replay()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e6)
        return statistics.median(times[1:])

    with_plan, without_plan = plan_mode != "off", plan_mode != "only"
    nan = float("nan")
    us_graph, us_graph_spread, graph_ok, us_graph_device = timed_replays(True) if with_plan else (nan, [nan, nan], True, nan)
    us_graph_plain, us_graph_plain_spread, graph_plain_ok, us_graph_plain_device = (
        timed_replays(False) if without_plan else (nan, [nan, nan], True, nan))  # fmt: skip
    us_bracket = host_bracket()

    # ---- whole op, eager launches (host launch overhead included), a plan per LAYERS_PER_PLAN steps ------------------
    def eager(n):
        plan = None
        for i in range(n):
            if with_plan and i % LAYERS_PER_PLAN == 0:
                plan = _plan(w, pools[i % copies], plan_buffer)
            _step(w, pools[i % copies], plan)

    eager(warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eager(steps)
    torch.cuda.synchronize()
    us_eager = (time.perf_counter() - t0) / steps * 1e6

    # ---- per-kernel durations: events on the launch stream around back-to-back launches through the C ABI ---
    b, hq, hkv, d, bs = w.shape
    group_rows = w.meta.get("prefix_group_rows")
    shared_lens = w.meta.get("shared_prefix_lens")
    if shared_lens is None:
        ws_bytes = cabi.decode_workspace_bytes(b, hq, d, bs, w.block_table.shape[1])
    else:
        ws_bytes = cabi.decode_grouped_workspace_bytes(b, hq, hkv, d, bs, w.block_table.shape[1], group_rows)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=w.q.device)
    caches = [cabi.describe_cache(*pool) for pool in pools]
    out2 = torch.empty_like(w.q)
    spread = {}

    def build_plan():
        return cabi.paged_decode_plan(caches[0], w.q.dtype, hq, w.block_table, w.cache_seqlens, plan_buffer,
                                      group_rows=group_rows, shared_lens=shared_lens)  # fmt: skip

    def time_launches(launch, name):
        """Mean duration of `kernel_iters` back-to-back launches, by events on the stream around one replay of a graph
        that holds them (launched one by one from Python the host cannot keep up with kernels shorter than ~8 us, and
        the figure would be its launch rate)."""
        side3 = torch.cuda.Stream()
        side3.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side3):
            for i in range(max(copies, 20)):
                launch(i)
        torch.cuda.current_stream().wait_stream(side3)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(kernel_iters):
                launch(i)
        graph.replay()
        torch.cuda.synchronize()
        samples = []
        for _ in range(kernel_samples):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            e1.synchronize()
            samples.append(e0.elapsed_time(e1) * 1e3 / kernel_iters)
        samples.sort()
        spread[name] = [samples[len(samples) // 10], samples[(len(samples) * 9) // 10]]
        return statistics.median(samples)

    def time_stage(stage, plan, name):
        def launch(i):
            cabi.paged_decode(caches[i % copies], w.q, w.k_update, w.v_update, out2, w.block_table, w.cache_seqlens,
                              workspace, softmax_scale=w.softmax_scale, stages=stage, group_rows=group_rows,
                              shared_lens=shared_lens, plan=plan)  # fmt: skip

        return time_launches(launch, name)

    plan = build_plan() if with_plan else None
    # the op folds the append into the merge launch; the stand-alone append launch is timed for reference only
    us_split_plain = time_stage(cabi.STAGE_SPLIT, None, "split_plain") if without_plan else nan
    us_split = time_stage(cabi.STAGE_SPLIT, plan, "split") if with_plan else nan
    us_reduce = time_stage(cabi.STAGE_APPEND | cabi.STAGE_REDUCE, plan, "merge")
    us_append = time_stage(cabi.STAGE_APPEND, None, "append")
    us_plan = time_launches(lambda i: build_plan(), "plan") if with_plan else nan
    if not with_plan:  # a run without plans reports the plain figures in the headline fields
        us_graph, us_graph_spread, us_split, spread["split"] = us_graph_plain, us_graph_plain_spread, us_split_plain, spread["split_plain"]
    torch.cuda.synchronize()
    assert torch.equal(out2, out), "C-ABI staged run disagrees with the op"

    if not with_plan:  # a run without plans reports the plain launches as the step and as the kernel
        us_graph, us_graph_spread, us_split = us_graph_plain, us_graph_plain_spread, us_split_plain
        us_graph_device = us_graph_plain_device
    gbps = alg_bytes / (us_split * 1e-6) / 1e9
    ceiling = measure_stream_ceiling(w, pools)
    return {
        "workload": w.name,
        "us_per_step": us_graph,
        "us_per_step_p10_p90": us_graph_spread,
        # the same samples by events on the stream (first replay's start to last replay's end): without the host's
        # launch of the first graph and its wake-up from the synchronize, which `host_bracket_us` times on a graph of
        # one tiny kernel and which a sample of `steps` steps carries once
        "us_per_step_on_device": us_graph_device,
        "host_bracket_us": us_bracket,
        "us_per_step_without_plan": us_graph_plain,
        "us_per_step_without_plan_p10_p90": us_graph_plain_spread,
        "us_per_step_eager": us_eager,
        "plan": {"layers_per_plan": LAYERS_PER_PLAN, "plan_kernel_us": us_plan,
                 "plan_us_per_step": us_plan / LAYERS_PER_PLAN, "planned_equals_plain_bitwise": planned_equal},
        "kernel_us": {"split": us_split, "split_without_plan": us_split_plain, "merge_with_append": us_reduce,
                      "append_alone_not_in_op": us_append, "plan": us_plan},
        # 10th / 90th percentile of the kernels' samples (each the mean of back-to-back launches)
        "split_us_p10_p90": spread["split"],
        "split_without_plan_us_p10_p90": spread.get("split_plain"),
        "tokens_per_s": w.q.shape[0] / (us_graph * 1e-6),
        "algorithmic_bytes": alg_bytes,
        "op_gbps": alg_bytes / (us_graph * 1e-6) / 1e9,
        "roofline": {
            "bound": "hbm", "kernel": "decode_mfma_kernel", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": gbps / HBM_PEAK_GBPS, "traffic": PROFILED_TRAFFIC_BYTES.get(w.name),
            "traffic_source": PROFILED_TRAFFIC_SOURCE["decode"] if w.name in PROFILED_TRAFFIC_BYTES else None,
            "frac_without_plan": alg_bytes / (us_split_plain * 1e-6) / 1e9 / HBM_PEAK_GBPS,
            # what a reader that computes nothing reaches over the same pools (all pages in address order / the distinct
            # pages of the block table in random order), and the split kernel against the latter
            "stream_ceiling_gbps": ceiling["linear_gbps"], "stream_ceiling_paged_gbps": ceiling["paged_gbps"],
            "stream_ceiling_paged_prefetch_gbps": ceiling["paged_prefetch_gbps"],
            "stream_ceiling_paged_kv_adjacent_gbps": ceiling["paged_kv_adjacent_gbps"],
            "frac_of_stream_ceiling": gbps / max(ceiling["paged_gbps"], ceiling["paged_prefetch_gbps"]),
        },  # fmt: skip
        "pool_copies": copies,
        "parity_max_abs_4rows": parity,
        "graph_replay_matches_eager": graph_ok and graph_plain_ok,
        "kv_tokens": {"logical": w.logical_tokens, "unique": w.unique_tokens},
        "block_tables": measure_block_tables(w),
    }


def measure_other_shapes(device, steps=56, repeats=7):
    """us/step (graph replay, a plan per LAYERS_PER_PLAN steps where the shape takes one) of decode shapes next to the
    benchmark's: cfg 2's rows with more than 16 query heads per KV head (several column tiles per KV head on the
    matrix-core kernel) and on pages whose size is no power of two (a multiply-shift division in the kernel's page
    arithmetic), and a single sequence of 4 096 cached tokens (a launch with as many cost positions as units: the
    latency of a decode step that has next to nothing to read).  Two pool copies only, so part of the working set may
    sit in the Infinity Cache: these are orders of magnitude, not roofline figures."""
    import torch

    from areno_amd import workloads
    from areno_amd.accel import cabi

    shapes = {
        "mqa_32q_1kv_int8": dict(hq=32, hkv=1, bs=16, kv="int8"),
        "gqa_64q_2kv_bf16": dict(hq=64, hkv=2, bs=16, kv="bf16"),
        "cfg2_rows_page48_int8": dict(hq=28, hkv=4, bs=48, kv="int8"),
        "one_sequence_4096_tokens_int8": dict(hq=28, hkv=4, bs=16, kv="int8", lengths=[4096]),
    }
    g = torch.Generator().manual_seed(2002)
    cfg2_like_lengths = torch.randint(512, 4097, (64,), generator=g)
    result = {}
    for name, sh in shapes.items():
        lengths = torch.tensor(sh["lengths"]) if "lengths" in sh else cfg2_like_lengths
        batch = int(lengths.numel())
        w = workloads.make_decode_workload(name, seed=7, batch=batch, hq=sh["hq"], hkv=sh["hkv"], d=128, bs=sh["bs"],
                                           kv=sh["kv"], lengths=lengths, device=device, quantize_fn=_gpu_quantize)  # fmt: skip
        pools = _clone_pools(w, 2)
        plan_buffer = torch.empty(max(16, cabi.decode_plan_bytes(batch)), dtype=torch.uint8, device=device)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for pool in pools:
                _step(w, pool, _plan(w, pool))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        keep = []
        with torch.cuda.graph(graph):
            plan = None
            for i in range(steps):
                if i % LAYERS_PER_PLAN == 0:
                    plan = _plan(w, pools[0], plan_buffer)
                keep.append(_step(w, pools[i % 2], plan))
        graph.replay()
        torch.cuda.synchronize()
        samples = []
        for _ in range(repeats):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            samples.append((time.perf_counter() - t0) / steps * 1e6)
        us = statistics.median(samples)
        result[name] = {"us_per_step": us, "algorithmic_gbps": w.algorithmic_bytes() / (us * 1e-6) / 1e9,
                        "kernel": "matrix cores" if plan is not None and plan.units > 0 else "vector ALU",
                        "parity_max_abs_4rows": _parity_sample(w, keep[0])}  # fmt: skip
        del w, pools, keep, graph
        torch.cuda.empty_cache()
    return result


def measure_backward(device, seqs=2, new=2048, hq=28, hkv=4, d=128, iters=10):
    """us per call of the varlen op's backward (dQ, dK, dV through autograd, bf16, the matrix-core kernels) and its
    rate counted as 2.5 x the forward's FLOPs, next to the forward on the same inputs; the training-side companion of
    the path, reported for completeness."""
    import torch

    from areno_amd.accel import attention as ops

    g = torch.Generator().manual_seed(7)
    t = seqs * new
    cu = torch.arange(0, t + 1, new, dtype=torch.int32, device=device)
    q, k, v, go = (torch.randn(t, h, d, generator=g).bfloat16().to(device) for h in (hq, hkv, hkv, hq))
    q, k, v = (x.requires_grad_(True) for x in (q, k, v))
    out = ops.areno_varlen_causal_attention(q, k, v, cu)

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        first.record()
        for _ in range(iters):
            fn()
        last.record()
        torch.cuda.synchronize()
        return first.elapsed_time(last) / iters * 1e3

    us_backward = timed(lambda: torch.autograd.grad(out, (q, k, v), go, retain_graph=True))
    with torch.no_grad():
        us_forward = timed(lambda: ops.areno_varlen_causal_attention(q, k, v, cu))
    flops = seqs * 4 * hq * d * new * (new + 1) / 2
    return {"shape": f"{seqs} x {new} tokens, {hq}/{hkv} heads, D = {d}, bf16", "backward_us": us_backward,
            "backward_tflops_as_2.5x_forward": 2.5 * flops / us_backward / 1e6, "forward_us": us_forward,
            "forward_tflops": flops / us_forward / 1e6}  # fmt: skip


def measure_stream_ceiling(w, pools, iters=10, samples=9):
    """GB/s of `areno_hip_probe_stream_read` (16-byte loads, a page per wave at a time, nothing computed; one launch
    reads a page set from the K and the V pool, as a decode launch does) over the K and V pools of all pool copies:
    every page in address order (`linear`); the distinct pages the block table names in a random order, each wave
    fetching a page's id when it gets there (`paged`) or one page ahead, as the decode kernel does
    (`paged_prefetch`); and the same number of bytes as runs of two pages from one pool in random order
    (`paged_kv_adjacent`: what a layout that keeps a block's K and V pages side by side would offer)."""
    import torch

    from areno_amd.accel import cabi

    page_bytes = w.k_cache[0].numel() * w.k_cache.element_size()
    sink = torch.zeros(16, dtype=torch.int32, device=w.q.device)
    bs = w.k_cache.shape[1]
    lens = w.cache_seqlens.cpu()
    table = w.block_table.cpu()
    used = torch.unique(torch.cat([table[b, : (int(lens[b]) + bs) // bs] for b in range(table.shape[0])]))
    # every page once (rows of a rollout share pages), in a fixed random order as the shuffled pools give it to the kernel
    used = used[torch.randperm(used.numel(), generator=torch.Generator().manual_seed(7))].to(torch.int32).to(w.q.device)
    # runs of two pages inside one pool: half as many ids, drawn over the pool's page pairs
    pairs = (used[: used.numel() // 2] // 2).contiguous()

    def timed(ids, **kw):
        def once():
            if kw.get("adjacent"):
                return sum(cabi.probe_stream_read(pool[0], pool[1], 2 * page_bytes, sink, ids, prefetch_ids=True) for pool in pools)
            return sum(cabi.probe_stream_read(pool[0], pool[1], page_bytes, sink, ids, prefetch_ids=kw.get("prefetch", False))
                       for pool in pools)  # fmt: skip

        nbytes = once()
        torch.cuda.synchronize()
        out = []
        for _ in range(samples):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                once()
            e1.record()
            e1.synchronize()
            out.append(e0.elapsed_time(e1) * 1e-3 / iters)
        return nbytes / statistics.median(out) / 1e9

    return {"linear_gbps": timed(None), "paged_gbps": timed(used), "paged_prefetch_gbps": timed(used, prefetch=True),
            "paged_kv_adjacent_gbps": timed(pairs, adjacent=True), "page_bytes": page_bytes}  # fmt: skip


def measure_block_tables(w, inner=20, repeats=5):
    """The page bookkeeping of one decode step for the workload's rows: on the device (pages for the next position, then the
    padded table; replayed from a HIP graph) and the way the reference does it (positions to the host, a walk over Python lists,
    a new table uploaded; areno/engine/inference.py:561-580), here with the oracle's list code as the port."""
    import torch

    from areno_amd.engine import DeviceBlockTables
    from oracle.block_table_ref import RefBlockTables

    dev = w.q.device
    b, _, _, _, bs = w.shape
    max_blocks = w.block_table.shape[1]
    lens = w.cache_seqlens.cpu().tolist()
    pages_needed = sum(-(-(n + 1) // bs) for n in lens)
    rows = list(range(b))
    tables = DeviceBlockTables(pages_needed + b, b, max_blocks, bs, dev)
    lists = RefBlockTables(pages_needed + b, b, max_blocks, bs)
    tables.reserve(rows, lens)
    lists.reserve(rows, lens)
    rows_dev = torch.arange(b, device=dev)
    out = torch.empty(b, max_blocks, dtype=torch.int32, device=dev)

    def device_step():
        tables.decode_step(rows_dev, w.cache_seqlens, out=out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        device_step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(inner):
            device_step()
    samples = []
    for _ in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        samples.append((time.perf_counter() - t0) / inner * 1e6)
    us_device = statistics.median(samples)

    def host_step():
        active = rows_dev.cpu().tolist()
        positions = w.cache_seqlens.cpu().tolist()
        lists.ensure_decode(active, positions)
        table = torch.tensor(lists.gather(active, False), dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        return table

    same = bool(torch.equal(host_step(), out))
    samples = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        host_step()
        samples.append((time.perf_counter() - t0) * 1e6)
    return {"rows": b, "max_blocks": max_blocks, "device_us_per_step": us_device,
            "host_lists_us_per_step": statistics.median(samples), "tables_equal": same}  # fmt: skip


MFMA_BF16_PEAK_TFLOPS = 2500.0


def measure_prefill(w, iters=20):
    """Time the paged-prefill op (and the quantizing cache write that precedes it) on cfg 4; MFMA-bound."""
    import torch

    from areno_amd.accel import attention as ops

    def write():
        ops.areno_paged_cache_write(w.k_new, w.v_new, w.k_cache, w.v_cache, w.cache_block_ids, w.cache_block_offsets,
                                    k_scale=w.k_scale, v_scale=w.v_scale)  # fmt: skip

    def attend():
        return ops.areno_paged_varlen_causal_attention(
            w.q, w.k_cache, w.v_cache, w.block_table, w.cu_seqlens_q, w.context_lens,
            softmax_scale=w.softmax_scale, k_scale=w.k_scale, v_scale=w.v_scale,
        )  # fmt: skip

    spread = {}

    def timed(fn, inner=1, warm=3, name=None):
        """Median over `iters` samples of `inner` back-to-back calls (short ops: the queue stays ahead of the GPU);
        with a name, the 10th and 90th percentile of the samples are kept in `spread`."""
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        samples = []
        for _ in range(iters):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(inner):
                fn()
            e1.record()
            e1.synchronize()
            samples.append(e0.elapsed_time(e1) * 1e3 / inner)
        if name is not None:
            ordered = sorted(samples)
            spread[name] = [ordered[len(ordered) // 10], ordered[(len(ordered) * 9) // 10]]
        return statistics.median(samples)

    def timed_graph(fn, inner=20):
        """Short ops: `inner` calls captured in one HIP graph, so the host's per-call cost is not in the figure."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        keep = []
        with torch.cuda.graph(g):
            for _ in range(inner):
                keep.append(fn())
        return timed(g.replay) / inner

    us_write = timed_graph(write)
    us_attend = timed(attend, warm=40, name="prefill")  # ~1 ms launches: an idle part's clocks settle over tens of ms

    # the fused step in front of the path at the same shape: QK RMSNorm + rotary + quantizing write of the new rows
    t, hq, d = w.q.shape
    hkv = w.k_new.shape[1]
    gen = torch.Generator(device=w.q.device).manual_seed(5)
    inv_freq = 1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    emb = torch.outer(torch.arange(32768, dtype=torch.float32), inv_freq)
    cos, sin = (torch.cat((f, f), dim=-1).to(w.q.device) for f in (emb.cos(), emb.sin()))
    positions = torch.randint(0, 32768, (t,), generator=gen, device=w.q.device)
    ones = torch.ones(d, device=w.q.device)

    def front():
        return ops.areno_qk_norm_rope_cache_write(
            w.q, w.k_new, w.v_new, positions, cos, sin, q_norm_weight=ones, k_norm_weight=ones, eps=1e-6,
            k_cache=w.k_cache, v_cache=w.v_cache, cache_block_ids=w.cache_block_ids,
            cache_block_offsets=w.cache_block_offsets, k_scale=w.k_scale, v_scale=w.v_scale,
        )  # fmt: skip

    us_front = timed_graph(front)
    # the same step with the rotary rows of the step's tokens prepared once for all layers (positions are the same in
    # every layer): the rows kernel's time is spread over the layers it serves
    rows = ops.areno_rope_rows(positions, cos, sin, w.q.dtype)

    def front_rows():
        return ops.areno_qk_norm_rope_cache_write(
            w.q, w.k_new, w.v_new, positions, cos, sin, q_norm_weight=ones, k_norm_weight=ones, eps=1e-6,
            k_cache=w.k_cache, v_cache=w.v_cache, cache_block_ids=w.cache_block_ids,
            cache_block_offsets=w.cache_block_offsets, k_scale=w.k_scale, v_scale=w.v_scale, rope_rows=rows,
        )  # fmt: skip

    rows_equal = all(bool(torch.equal(a, b)) for a, b in zip(front(), front_rows()))
    us_front_rows = timed_graph(front_rows)
    us_rows = timed_graph(lambda: ops.areno_rope_rows(positions, cos, sin, w.q.dtype))
    act = w.q.element_size()
    scale_bytes = 0 if w.k_scale is None else 2 * w.k_scale.element_size()
    front_bytes = t * ((hq + 2 * hkv) * d * act + (hq + hkv) * d * act + hkv * (2 * d * w.k_cache.element_size() + scale_bytes))
    us_front_step = us_front_rows + us_rows / LAYERS_PER_PLAN
    write()  # leave the pages as the attention measurement expects them
    flops = w.flops()
    tflops = flops / (us_attend * 1e-6) / 1e12
    return {
        "workload": w.name,
        "us_per_step": us_attend + us_write,
        "kernel_us": {"cache_write": us_write, "prefill": us_attend, "qk_norm_rope_cache_write": us_front,
                      "qk_norm_rope_cache_write_from_rows": us_front_rows, "rope_rows": us_rows},
        "prefill_us_p10_p90": spread["prefill"],
        "qk_norm_rope_cache_write": {
            "us": us_front, "algorithmic_bytes": front_bytes, "gbps": front_bytes / (us_front * 1e-6) / 1e9,
            "frac_of_hbm_peak": front_bytes / (us_front * 1e-6) / 1e9 / HBM_PEAK_GBPS,
            # with the step's rotary rows prepared once per LAYERS_PER_PLAN layers (their share of that launch included)
            "us_from_rows": us_front_step, "rows_kernel_us": us_rows, "layers_per_rows": LAYERS_PER_PLAN,
            "frac_of_hbm_peak_from_rows": front_bytes / (us_front_step * 1e-6) / 1e9 / HBM_PEAK_GBPS,
            "rows_equal_tables_bitwise": rows_equal,
        },  # fmt: skip
        "new_tokens": int(w.q.shape[0]),
        "tokens_per_s": w.q.shape[0] / ((us_attend + us_write) * 1e-6),
        "flops": flops,
        "roofline": {
            "bound": "mfma", "kernel": "prefill_mfma_kernel", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": PROFILED_TRAFFIC_BYTES.get(w.name),
            "traffic_source": PROFILED_TRAFFIC_SOURCE["prefill"],
            # what the matrix cores sustain on this part when they are asked for nothing but products of one shape
            # (areno_hip_probe_mfma_rate, timed here): the kernel's products are 16 x 16 x 32
            **measure_mfma_ceilings(w.q.device, tflops),
        },  # fmt: skip
    }


def measure_mfma_ceilings(device, kernel_tflops, iters=40000, samples=5):
    """TFLOP/s of launches of independent matrix products on register operands, per shape of product (f16, the type
    the prefill kernel computes fp8 pages in; bf16 next to it), median of a few launches."""
    import torch

    from areno_amd.accel import cabi

    sink = torch.zeros(4, dtype=torch.float32, device=device)
    rates = {}
    for name, shape in (("16x16x32_f16", 2), ("32x32x16_f16", 3), ("16x16x32_bf16", 0), ("32x32x16_bf16", 1)):
        cabi.probe_mfma_rate(shape, 1000, sink)
        torch.cuda.synchronize()
        got = []
        for _ in range(samples):
            first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            first.record()
            flops = cabi.probe_mfma_rate(shape, iters, sink)
            last.record()
            torch.cuda.synchronize()
            got.append(flops / (first.elapsed_time(last) * 1e-3) / 1e12)
        rates[name] = statistics.median(got)
    return {"mfma_ceiling_tflops": rates, "frac_of_16x16x32_f16_ceiling": kernel_tflops / rates["16x16x32_f16"]}


def wave_trace(w, launches=18):
    """Per-wave timeline of the split kernel (tuning builds only: ``ARENO_TRACE=1 python setup.py build_ext --inplace``
    makes the kernel stamp its waves with the 100 MHz wall clock): when waves start, have the work list, start their
    first four tiles and finish, relative to the first wave's start, over the last launches of a warm sequence; with a
    per-step plan and without one.  The finish times are also set against what the work list gives each unit: tile
    steps, segments (items it holds quanta of) and 16-token quanta."""
    import ctypes

    import numpy as np
    import torch

    from areno_amd.accel import cabi

    lib = cabi.lib()
    if not hasattr(lib, "areno_hip_debug_set_trace"):
        raise SystemExit("--wave-trace needs a library built with ARENO_TRACE=1")
    lib.areno_hip_debug_set_trace.argtypes = [ctypes.c_void_p]
    b, hq, hkv, d, bs = w.shape
    pools = _clone_pools(w, 6)
    workspace = torch.empty(cabi.decode_workspace_bytes(b, hq, d, bs, w.block_table.shape[1]), dtype=torch.uint8, device=w.q.device)
    out = torch.empty_like(w.q)
    buf = torch.zeros(8192 * 8, dtype=torch.int64, device=w.q.device)
    plan_buffer = torch.empty(cabi.decode_plan_bytes(b), dtype=torch.uint8, device=w.q.device)
    plan = cabi.paged_decode_plan(cabi.describe_cache(*pools[0]), w.q.dtype, hq, w.block_table, w.cache_seqlens, plan_buffer)
    keys = ("start", "work_list_ready", "tile0", "tile1", "tile2", "tile3", "finish")

    def pct(a, q):
        return float(np.percentile(a, q))

    def timeline(use_plan):
        lib.areno_hip_debug_set_trace(buf.data_ptr())
        runs = []
        for it in range(launches):
            buf.zero_()
            cabi.paged_decode(cabi.describe_cache(*pools[it % len(pools)]), w.q, w.k_update, w.v_update, out, w.block_table,
                              w.cache_seqlens, workspace, softmax_scale=w.softmax_scale, stages=cabi.STAGE_SPLIT,
                              plan=plan if use_plan else None)  # fmt: skip
            torch.cuda.synchronize()
            runs.append(buf.cpu().view(-1, 8).numpy().copy())
        lib.areno_hip_debug_set_trace(None)
        runs = runs[launches // 3:]
        waves = int((runs[0][:, 6] != 0).sum())
        us = {k: np.stack([(r[:waves, col] - r[:waves, 0].min()) / 100.0 for r in runs]) for col, k in enumerate(keys)}
        table = {k: {"mean": float(v.mean()), "p10": pct(v, 10), "p50": pct(v, 50), "p90": pct(v, 90),
                     "max": float(v.max(1).mean())} for k, v in us.items()}  # fmt: skip
        fin = us["finish"]
        return waves, table, fin

    waves, planned, fin = timeline(True)
    _, plain, _ = timeline(False)
    result = {"workload": w.name, "launches_averaged": launches - launches // 3, "waves": waves,
              "us_since_first_wave_start": {"with_plan": planned, "without_plan": plain}}  # fmt: skip
    # the finish times of the planned launches against the units' work (plain launches of one workgroup row: wave i
    # belongs to unit i // 4); the same arithmetic as areno_amd/csrc/decode_items.hpp
    if hkv <= 4 and waves % 4 == 0 and w.k_scale is not None:
        lens = w.cache_seqlens.cpu().numpy().astype(np.int64)
        switch, tile = 3, 32
        quanta = (lens + 15) // 16
        extent = np.where(quanta > 0, quanta + switch, 0)
        cum = np.concatenate([[0], np.cumsum(extent)])
        units = waves // 4
        borders = np.arange(units + 1) * cum[-1] // units
        steps, segments = np.zeros(units), np.zeros(units)
        for u in range(units):
            for v in range(len(lens)):
                lo, hi = max(borders[u], cum[v] + switch), min(borders[u + 1], cum[v + 1])
                if hi > lo:
                    tokens = min(lens[v], (hi - cum[v] - switch) * 16) - (lo - cum[v] - switch) * 16
                    steps[u] += -(-tokens // tile)
                    segments[u] += 1
        unit_finish = fin.mean(0).reshape(units, 4).mean(1)
        result["finish_by_segments_in_unit"] = {
            int(k): {"units": int((segments == k).sum()), "mean_finish_us": float(unit_finish[segments == k].mean())}
            for k in sorted(set(segments.tolist()))
        }
        result["finish_by_steps_in_unit"] = {
            int(k): {"units": int((steps == k).sum()), "mean_finish_us": float(unit_finish[steps == k].mean())}
            for k in sorted(set(steps.tolist()))
        }
        result["finish_spread"] = {"std_of_unit_means_us": float(fin.mean(0).std()), "std_within_unit_over_launches_us": float(fin.std(0).mean())}
    return result


def cpu_baseline(w, warmups=3, repeats=7):
    """The CPU oracle (PyTorch restatement of the reference's native path: cache append, per-sequence block-table gather,
    fp32 softmax attention with GQA) on all sequences of the workload, on the host cores: three warm-ups, median of
    seven runs."""
    import torch

    from oracle import attention_ref as ar
    from oracle import quant_ref as qr

    threads = torch.get_num_threads()
    if w.k_scale is None:
        kc, vc = w.k_cache.cpu().float(), w.v_cache.cpu().float()
    else:
        kc, vc = qr.dequantize(w.k_cache.cpu(), w.k_scale.cpu()), qr.dequantize(w.v_cache.cpu(), w.v_scale.cpu())
    q, ku, vu = w.q.cpu().float(), w.k_update.cpu().float(), w.v_update.cpu().float()
    table, lens = w.block_table.cpu(), w.cache_seqlens.cpu()

    def once():
        ar.ref_decode_update(ku, vu, kc, vc, table, lens)
        return ar.ref_paged_decode(q, kc, vc, table, lens, -1, w.softmax_scale)

    for _ in range(warmups):
        once()
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        once()
        times.append(time.perf_counter() - t0)
    return {
        "value": statistics.median(times) * 1e6, "unit": "us/step", "cores": threads, "kind": "port",
        "sample": f"all {w.q.shape[0]} sequences of {w.name} (dequantized fp32 caches; append + gather + attention), "
                  f"{warmups} warm-ups, median of {repeats} runs, fastest-slowest {min(times) * 1e6:.0f}-{max(times) * 1e6:.0f} us",
    }  # fmt: skip


def _without_nan(x):
    """Figures a run did not measure (`--plan only` / `off`) as null instead of NaN, which JSON has no literal for."""
    if isinstance(x, dict):
        return {k: _without_nan(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_without_nan(v) for v in x]
    return None if isinstance(x, float) and x != x else x


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg2_b256"], default=None,
                    help="measure a single workload")  # fmt: skip
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-other-shapes", action="store_true",
                    help="leave out the probe of decode shapes next to the benchmark's (for profiler runs, whose per-kernel "
                         "averages should belong to the benchmark's workloads)")
    ap.add_argument("--plan", choices=["both", "only", "off"], default="both",
                    help="decode workloads: time the steps with a per-step plan and without one (both), or only one of the "
                         "two (for profiler runs whose per-kernel averages should belong to one of them)")  # fmt: skip
    ap.add_argument("--wave-trace", choices=["cfg1", "cfg2", "cfg3"], default=None,
                    help="print the split kernel's per-wave timeline for a workload (needs an ARENO_TRACE=1 build) and exit")  # fmt: skip
    args = ap.parse_args()
    if args.gpus != 1:
        print(
            "bench.py measures one GPU: the decode path has no cross-GPU step (sequences and heads shard with no "
            "exchange), so --gpus above 1 is not a configuration of this benchmark.",
            file=sys.stderr,
        )
        return 2

    import torch

    from areno_amd import workloads

    if not torch.cuda.is_available():
        print("bench.py needs an AMD GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        return 2
    dev = "cuda:0"
    torch.cuda.set_device(0)

    builders = {
        "cfg1": lambda: workloads.cfg1_qwen7b("bf16", device=dev),
        "cfg2": lambda: workloads.cfg2_qwen7b_int8(device=dev, quantize_fn=_gpu_quantize),
        "cfg3": lambda: workloads.cfg3_rollout("fp8", device=dev, quantize_fn=_gpu_quantize),
        "cfg4": lambda: workloads.cfg4_prefill("fp8", device=dev, quantize_fn=_gpu_quantize),
        # not a configuration of the benchmark: cfg 2 at four times the batch, to show how the per-launch fixed
        # cost (launch, dependent first loads, uneven wave finish: ~13 us) weighs on the B = 64 figures
        "cfg2_b256": lambda: workloads.cfg2_qwen7b_int8(device=dev, quantize_fn=_gpu_quantize, batch=256),
    }
    if args.wave_trace:
        w = builders[args.wave_trace]()
        w.meta.pop("shared_prefix_lens", None)  # the plain kernel's timeline
        print(json.dumps(wave_trace(w)))
        return 0
    names = [args.only] if args.only else ["cfg2", "cfg1", "cfg3", "cfg4", "cfg2_b256"]
    results = {}
    baseline = None
    for name in names:
        w = builders[name]()
        results[name] = measure_prefill(w) if name == "cfg4" else measure_decode(w, args.steps, args.warmup, plan_mode=args.plan)
        if name == names[0] and not args.no_cpu and name != "cfg4":
            baseline = cpu_baseline(w)
        del w
        torch.cuda.empty_cache()

    if not args.only and not args.skip_other_shapes:
        results["other_shapes"] = measure_other_shapes(dev)
        results["varlen_backward"] = measure_backward(dev)
        # (a launch that fills the compute units many times over: the kernels' shapes for large launches)
        results["varlen_backward_4x4096"] = measure_backward(dev, seqs=4, new=4096, hq=32, hkv=8, iters=5)

    head = results[names[0]]
    dtype = {"cfg1": "bf16", "cfg2": "int8", "cfg3": "fp8", "cfg4": "fp8", "cfg2_b256": "int8"}[names[0]]
    line = {
        "metric": "paged_decode_attn_us_per_step",
        "value": head["us_per_step"],
        "unit": "us/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["us_per_step"] / 1e3,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {
            "workload": head["workload"],
            "shape": "B=64 Hq=28 Hkv=4 D=128 page=16 ctx~U[512,4096]" if names[0] != "cfg3" else "B=256 Hq=32 Hkv=8 D=128",
            "launch": "HIP graph replay, KV pools rotated over >1.3 GB",
            "step": "one layer's decode op (split + merge launch); per-step plan: one plan launch per "
                    f"{LAYERS_PER_PLAN} steps, inside the timed region" if "plan" in head else "one paged prefill",
        },
        "value_p10_p90": head.get("us_per_step_p10_p90"),
        "value_on_device": head.get("us_per_step_on_device"),
        "host_bracket_us": head.get("host_bracket_us"),
        "value_without_plan": head.get("us_per_step_without_plan"),
        "tokens_per_s": head["tokens_per_s"],
        "hbm_gbps_op": head.get("op_gbps"),
        "roofline": head["roofline"],
        "cpu_baseline": baseline,
        "workloads": results,
        "device": torch.cuda.get_device_name(0),
    }
    print(json.dumps(_without_nan(line)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
