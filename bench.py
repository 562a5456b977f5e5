#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

Prints ONE JSON line.  The headline (`metric`/`value`) is paged-KV batched
decode attention (64 sequences, context U[256, 8192], 32 query heads, 8 KV
heads, D=128, block 16) in GB/s of algorithmic traffic; the prefill-side
figures (TFLOP/s of the causal prefill and of the chunked prefill over a
paged cache) and the two latency-bound workloads ride along under
`workloads`.  A "step" is one pass of the hot path over one batch of
synthetic input that is already resident in HBM.

Every workload carries
  roofline      for its dominant kernel: algorithmic bytes (or flops) per
                launch / the kernel's mean duration, measured with HIP events
                on the launch stream (the library's per-kernel timer);
  cpu_baseline  the CPU restatement of Granite's CPU attention (the oracle)
                timed on this host on a bounded sample, with the thread count.
The oracle is only the checker and the baseline here; the measured path is
the HIP library.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
for p in (ROOT, ROOT / "tests"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA

CPU_SAMPLE_SECONDS = 10.0   # time box of each workload's CPU-baseline sample
FLOAT_QUERY_LEG = True  # prefill workloads: also time the launch with float queries
CLOCK_RAMP_MS = 100.0       # untimed work in front of every measurement, see Timer.run

# HBM bytes per launch of each workload's dominant kernel, as counted by rocprofv3
# (FETCH_SIZE + WRITE_SIZE per dispatch, scaled by what the same counters read for a plain
# copy of known size).  They are not measured by this run: profiles/traffic.json holds what
# the last profiling pass counted, keyed by workload name, and an entry is reported only for
# the exact workload it was counted on.
TRAFFIC_FILE = ROOT / "profiles" / "traffic.json"


def profiled_traffic(name: str, workload: str):
    try:
        entry = json.loads(TRAFFIC_FILE.read_text()).get(name)
    except (OSError, ValueError):
        return None
    if not entry or entry.get("workload") != workload:
        return None
    return entry.get("traffic_bytes")


def log(msg: str) -> None:
    print(msg, file=sys.stderr, flush=True)


class Timer:
    """Times K back-to-back steps with events on the launch stream."""

    def __init__(self, gpu):
        self.gpu = gpu

    def run(self, step, warmup: int, steps: int):
        gpu = self.gpu
        # The part leaves its idle clocks only after some tens of milliseconds of work, and the
        # shorter workloads here run 50 steps in 3 ms: untimed steps for CLOCK_RAMP_MS first (a
        # causal prefill step measured 57 us cold, 51 us from 50 ms of work on), then the
        # warm-up steps asked for, then the timed region.
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < CLOCK_RAMP_MS:
            for _ in range(10):
                step()
            gpu.sync()
        for _ in range(warmup):
            step()
        gpu.sync()
        # whole-job time: K steps back to back
        e0, e1 = gpu.event(), gpu.event()
        t0 = time.perf_counter()
        gpu.record(e0)
        for _ in range(steps):
            step()
        gpu.record(e1)
        gpu.sync()
        wall_ms = (time.perf_counter() - t0) * 1e3
        ev_ms = gpu.elapsed_ms(e0, e1)
        gpu.destroy_event(e0)
        gpu.destroy_event(e1)
        # per-kernel durations: same K steps with the library's kernel timer on
        gpu.reset_kernel_timing()
        gpu.enable_kernel_timing(True)
        for _ in range(steps):
            step()
        gpu.sync()
        stats = gpu.get_kernel_timing_stats()
        gpu.enable_kernel_timing(False)
        return ev_ms / steps, wall_ms / steps, {k: (ms / max(n, 1), n) for k, (ms, n) in stats.items()}


def roofline(bound: str, work: float, kernel_ms: float, traffic):
    if bound == "hbm":
        achieved = work / (kernel_ms * 1e-3) / 1e9
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic}
    achieved = work / (kernel_ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 4), "traffic": traffic}


def max_err(got, want):
    d = np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64))
    return float(d.max(initial=0.0))


# ---------------------------------------------------------------------------
# workloads
# ---------------------------------------------------------------------------

def bench_paged_decode(gpu, steps, warmup, cpu):
    from granite_amd import F16, DeviceBuffer, workloads as W
    dev = DeviceBuffer.from_numpy
    t0 = time.perf_counter()
    c = W.make_paged_decode()
    log(f"[paged_decode] inputs: {int(c.seq_lens.sum())} tokens, pool {c.k_pool.nbytes * 2 / 2**30:.2f} GiB "
        f"({time.perf_counter() - t0:.1f}s)")
    B, hq = c.batch, c.num_heads
    bufs = dict(q=dev(c.q), k=dev(c.k_pool), v=dev(c.v_pool), t=dev(c.block_tables), l=dev(c.seq_lens))
    out, lse = dev(np.zeros((B, hq, 128), np.float32)), dev(np.zeros((B, hq), np.float32))

    def step():
        gpu.decode_attention(q=bufs["q"], q_dtype=F16, k_cache=bufs["k"], v_cache=bufs["v"],
                             block_tables=bufs["t"], seq_lens=bufs["l"], out=out, lse=lse, batch_size=B,
                             num_heads=hq, num_kv_heads=c.num_kv_heads, head_dim=128, scale=c.scale,
                             block_size=c.block_size, max_blocks_per_seq=c.max_blocks)

    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    nbytes = c.algorithmic_bytes()

    # the same batch through the reference-shaped entry point, whose queries are float
    # (MetalCompute::batched_paged_attention_decode): 0.5 MB more to read, no log-sum-exp
    q32 = dev(c.q.astype(np.float32))
    out32 = dev(np.zeros((B, hq, 128), np.float32))

    def step_f32():
        gpu.batched_paged_attention_decode(q32, bufs["k"], bufs["v"], bufs["t"], bufs["l"], out32, B, hq,
                                           c.num_kv_heads, 128, c.block_size, c.max_blocks, c.scale)

    ms32, _, _ = Timer(gpu).run(step_f32, warmup, steps)
    res = {
        "workload": "paged_decode_b64_ctx256-8192_hq32_hkv8_d128_bs16",
        "metric": "paged_decode_attn_GBps", "unit": "GB/s", "value": round(nbytes / (ms * 1e-3) / 1e9, 1),
        "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall_ms, 4),
        "algorithmic_bytes": nbytes, "flops": c.flops(), "dtype": "f16 K/V, f32 accumulate",
        "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
        "q_dtype": "f16",
        "reference_entry_point_f32_q": {"ms_per_step": round(ms32, 4),
                                        "GBps": round((nbytes + c.q.nbytes) / (ms32 * 1e-3) / 1e9, 1)},
    }
    main_kernel = "decode_stream" if "decode_stream" in kern else "decode_splitk"
    res["roofline"] = roofline("hbm", nbytes, kern[main_kernel][0], profiled_traffic("paged_decode", res["workload"]))
    res["roofline"]["kernel"] = main_kernel + "_kernel"
    if cpu:
        import oracle_bind
        oracle = oracle_bind.load()
        q32 = c.q.astype(np.float32)
        passes, t0 = 0, time.perf_counter()
        while passes == 0 or time.perf_counter() - t0 < CPU_SAMPLE_SECONDS:
            want, want_lse = oracle.batched_paged_decode(q32, c.k_pool, c.v_pool, c.block_tables, c.seq_lens,
                                                         c.block_size, c.scale)
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        res["cpu_baseline"] = {"value": round(nbytes / cpu_s / 1e9, 3), "unit": "GB/s",
                               "cores": oracle.lib.go_get_num_threads(), "kind": "port",
                               "seconds": round(cpu_s * passes, 2),
                               "sample": f"the whole workload (all 64 sequences), mean of {passes} passes"}
        res["parity"] = {"max_abs_err": max_err(out.read(np.float32, (B, hq, 128)), want),
                         "max_lse_err": max_err(lse.read(np.float32, (B, hq)), want_lse)}
    return res


def bench_prefill(gpu, steps, warmup, cpu):
    from granite_amd import F16, MASK_CAUSAL, DeviceBuffer, workloads as W
    dev = DeviceBuffer.from_numpy
    c = W.make_prefill()
    S, hq, hkv = c.seq, c.num_heads, c.num_kv_heads
    dq, dk, dv = dev(c.q), dev(c.k_cache), dev(c.v_cache)
    out, lse = dev(np.zeros((S, hq, 128), np.float16)), dev(np.zeros((hq, S), np.float32))

    def step():
        gpu.attention(q=dq, q_dtype=F16, q_tok_stride=hq * 128, q_head_stride=128, out=out, out_dtype=F16,
                      out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=S, num_heads=hq,
                      num_kv_heads=hkv, head_dim=128, scale=c.scale, k_cache=dk, v_cache=dv, cache_len=S,
                      max_seq=c.max_seq, mask_mode=MASK_CAUSAL, start_pos=0)

    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    flops = c.flops()
    res = {
        "workload": "causal_prefill_s2048_hq32_hkv8_d128", "metric": "prefill_attn_TFLOPs", "unit": "TFLOP/s",
        "value": round(flops / (ms * 1e-3) / 1e12, 2), "ms_per_step": round(ms, 4),
        "wall_ms_per_step": round(wall_ms, 4), "flops": flops, "algorithmic_bytes": c.algorithmic_bytes(),
        "dtype": "f16 MFMA, f32 accumulate", "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
    }
    res["roofline"] = roofline("mfma", flops, kern["attention_tiles"][0], profiled_traffic("prefill", res["workload"]))
    res["roofline"]["kernel"] = "attention_tiles_dma_kernel"
    # the same launch with float queries and float output, which is what the reference's callers
    # (and ChunkedPrefill of the host layer) pass: an fp16 head and an fp16 remainder of Q, i.e.
    # half as many MFMAs again in the scores
    from granite_amd import F32
    dq32, out32 = dev(c.q.astype(np.float32)), dev(np.zeros((S, hq, 128), np.float32))

    def step_f32():
        gpu.attention(q=dq32, q_dtype=F32, q_tok_stride=hq * 128, q_head_stride=128, out=out32, out_dtype=F32,
                      out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=S, num_heads=hq,
                      num_kv_heads=hkv, head_dim=128, scale=c.scale, k_cache=dk, v_cache=dv, cache_len=S,
                      max_seq=c.max_seq, mask_mode=MASK_CAUSAL, start_pos=0)

    if FLOAT_QUERY_LEG:
        ms32, _, kern32 = Timer(gpu).run(step_f32, warmup, steps)
        res["float_queries"] = {"ms_per_step": round(ms32, 4), "TFLOPs": round(flops / (ms32 * 1e-3) / 1e12, 2),
                                "kernels_ms": {k: round(v[0], 4) for k, v in kern32.items()}}
        step()  # (the parity leg below reads the half-query result)
        gpu.sync()
    if cpu:
        import oracle_bind
        oracle = oracle_bind.load()
        # the whole workload as the reference's CPU path runs it: the cache is gathered and
        # widened to float on every call (transformer.mm:1750-1763), then the attention core
        q32 = c.q[None].astype(np.float32)
        passes, t0 = 0, time.perf_counter()
        while passes == 0 or time.perf_counter() - t0 < CPU_SAMPLE_SECONDS:
            want, wl = oracle.attention_cached(q32, c.k_cache, c.v_cache, S, 0, c.scale)
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        got = out.read(np.float16, (S, hq, 128)).astype(np.float32)
        res["cpu_baseline"] = {"value": round(flops / cpu_s / 1e12, 5), "unit": "TFLOP/s",
                               "cores": oracle.lib.go_get_num_threads(), "kind": "port",
                               "seconds": round(cpu_s * passes, 2),
                               "sample": f"the whole workload (all {S} rows x {hq} heads, incl. the cache "
                                         f"gather), mean of {passes} passes"}
        res["parity"] = {"max_abs_err": max_err(got, want[0]),
                         "max_lse_err": max_err(lse.read(np.float32, (hq, S)), wl[0])}
    return res


def bench_chunked_prefill(gpu, steps, warmup, cpu):
    from granite_amd import F16, MASK_CAUSAL, DeviceBuffer, workloads as W
    dev = DeviceBuffer.from_numpy
    c = W.make_chunked_prefill()
    hq, hkv, bs, prefix, chunk = c.num_heads, c.num_kv_heads, c.block_size, c.prefix_len, c.chunk
    total = prefix + chunk
    dq, dk, dv, dt = dev(c.q), dev(c.k_pool), dev(c.v_pool), dev(c.block_table)
    dkn, dvn = dev(c.k_new), dev(c.v_new)
    out, lse = dev(np.zeros((chunk, hq, 128), np.float16)), dev(np.zeros((hq, chunk), np.float32))

    def step():  # append the chunk's K/V into its fresh blocks, then attend
        gpu.paged_kv_cache_append_ex(dkn, dvn, F16, hkv * 128, 128, dk, dv, dt, hkv, 128, prefix, chunk, bs)
        gpu.attention(q=dq, q_dtype=F16, q_tok_stride=hq * 128, q_head_stride=128, out=out, out_dtype=F16,
                      out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=chunk, num_heads=hq,
                      num_kv_heads=hkv, head_dim=128, scale=c.scale, k_cache=dk, v_cache=dv, cache_len=total,
                      block_table=dt, block_size=bs, mask_mode=MASK_CAUSAL, start_pos=prefix)

    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    flops = c.flops()
    res = {
        "workload": "chunked_prefill_prefix32768_chunk512_hq64_hkv8_d128_bs32",
        "metric": "prefill_attn_TFLOPs", "unit": "TFLOP/s", "value": round(flops / (ms * 1e-3) / 1e12, 2),
        "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall_ms, 4), "flops": flops,
        "algorithmic_bytes": c.algorithmic_bytes(), "dtype": "f16 MFMA, f32 accumulate",
        "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
    }
    res["roofline"] = roofline("mfma", flops, kern["attention_tiles"][0],
                               profiled_traffic("chunked_prefill", res["workload"]))
    res["roofline"]["kernel"] = "attention_tiles_dma_kernel"
    # with float queries and float output (see bench_prefill)
    from granite_amd import F32
    dq32, out32 = dev(c.q.astype(np.float32)), dev(np.zeros((chunk, hq, 128), np.float32))

    def step_f32():
        gpu.paged_kv_cache_append_ex(dkn, dvn, F16, hkv * 128, 128, dk, dv, dt, hkv, 128, prefix, chunk, bs)
        gpu.attention(q=dq32, q_dtype=F32, q_tok_stride=hq * 128, q_head_stride=128, out=out32, out_dtype=F32,
                      out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=chunk, num_heads=hq,
                      num_kv_heads=hkv, head_dim=128, scale=c.scale, k_cache=dk, v_cache=dv, cache_len=total,
                      block_table=dt, block_size=bs, mask_mode=MASK_CAUSAL, start_pos=prefix)

    if FLOAT_QUERY_LEG:
        ms32, _, kern32 = Timer(gpu).run(step_f32, warmup, steps)
        res["float_queries"] = {"ms_per_step": round(ms32, 4), "TFLOPs": round(flops / (ms32 * 1e-3) / 1e12, 2),
                                "kernels_ms": {k: round(v[0], 4) for k, v in kern32.items()}}
        step()
        gpu.sync()
    if cpu:
        import oracle_bind
        oracle = oracle_bind.load()
        # runs of 32 query rows through the reference-shaped paged path: every call gathers the
        # keys it can see out of the pool and widens them to float first, as the reference's
        # CPU attention does on every call (transformer.mm:1750-1763)
        pool_k = dk.read(np.uint16, c.k_pool.shape)   # the pools with the chunk appended
        pool_v = dv.read(np.uint16, c.v_pool.shape)
        got = out.read(np.float16, (chunk, hq, 128)).astype(np.float32)
        got_lse = lse.read(np.float32, (hq, chunk))
        t0 = time.perf_counter()
        err = lerr = 0.0
        sample_flops = 0
        done = 0
        for r0 in (0, 480, 240, 112, 368, 176, 304, 48, 432):
            if done >= 2 and time.perf_counter() - t0 > CPU_SAMPLE_SECONDS:
                break
            n = 32
            want, wl = oracle.attention_paged(c.q[None, r0:r0 + n].astype(np.float32), pool_k, pool_v,
                                              c.block_table, bs, prefix + r0 + n, prefix + r0, c.scale)
            sample_flops += 4 * hq * 128 * (n * (prefix + r0) + n * (n + 1) // 2)
            err = max(err, max_err(got[r0:r0 + n], want[0]))
            lerr = max(lerr, max_err(got_lse[:, r0:r0 + n], wl[0]))
            done += 1
        cpu_s = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": round(sample_flops / cpu_s / 1e12, 5), "unit": "TFLOP/s",
                               "cores": oracle.lib.go_get_num_threads(), "kind": "port",
                               "seconds": round(cpu_s, 2),
                               "sample": f"{done} runs of 32 query rows (of 512) x {hq} heads, each incl. the "
                                         f"gather of the keys it sees"}
        res["parity"] = {"max_abs_err": err, "max_lse_err": lerr}
    return res


def bench_tree(gpu, steps, warmup, cpu):
    from granite_amd import F32, MASK_TREE, DeviceBuffer, workloads as W
    dev = DeviceBuffer.from_numpy
    c = W.make_tree()
    hq, hkv, n = c.num_heads, c.num_kv_heads, c.num_nodes
    b = dict(q=dev(c.q), k=dev(c.k_pool), v=dev(c.v_pool), t=dev(c.block_table), kt=dev(c.k_tree),
             vt=dev(c.v_tree), p=dev(c.parents))
    out, lse = dev(np.zeros((hq, n, 128), np.float32)), dev(np.zeros((hq, n), np.float32))

    def step():
        gpu.attention(q=b["q"], q_dtype=F32, q_tok_stride=128, q_head_stride=n * 128, out=out, out_dtype=F32,
                      out_tok_stride=128, out_head_stride=n * 128, lse=lse, seq_q=n, num_heads=hq,
                      num_kv_heads=hkv, head_dim=128, scale=c.scale, k_cache=b["k"], v_cache=b["v"],
                      cache_len=c.prefix_len, block_table=b["t"], block_size=c.block_size, k_extra=b["kt"],
                      v_extra=b["vt"], extra_len=n, parents=b["p"], mask_mode=MASK_TREE)

    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    res = {
        "workload": "tree_prefix4096_nodes64_hq32_hkv8_d128_bs16", "metric": "tree_attn_latency_us", "unit": "us",
        "value": round(ms * 1e3, 2), "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall_ms, 4),
        "flops": c.flops(), "algorithmic_bytes": c.algorithmic_bytes(),
        "GBps": round(c.algorithmic_bytes() / (ms * 1e-3) / 1e9, 1),
        "TFLOPs": round(c.flops() / (ms * 1e-3) / 1e12, 2),
        "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
        "note": "launch/latency bound (19 MB, 4.3 GFLOP); reported, no roofline target",
    }
    if cpu:
        import oracle_bind
        oracle = oracle_bind.load()
        q = np.transpose(c.q, (1, 0, 2))[None]
        kt = np.transpose(c.k_tree, (1, 0, 2))[None].astype(np.float32)
        vt = np.transpose(c.v_tree, (1, 0, 2))[None].astype(np.float32)
        passes, t0 = 0, time.perf_counter()
        while passes == 0 or time.perf_counter() - t0 < CPU_SAMPLE_SECONDS / 2:
            ctx, wl = oracle.attention_tree(q, c.k_pool, c.v_pool, kt, vt, c.parents, c.prefix_len, c.scale,
                                            table=c.block_table, block_size=c.block_size)
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        res["cpu_baseline"] = {"value": round(cpu_s * 1e6, 1), "unit": "us",
                               "cores": oracle.lib.go_get_num_threads(), "kind": "port",
                               "sample": f"the whole workload, mean of {passes} passes (incl. the prefix gather)"}
        res["parity"] = {"max_abs_err": max_err(out.read(np.float32, (hq, n, 128)), np.transpose(ctx[0], (1, 0, 2))),
                         "max_lse_err": max_err(lse.read(np.float32, (hq, n)), wl[0])}
    return res


def bench_decode_contiguous(gpu, steps, warmup, cpu):
    from granite_amd import F32, DeviceBuffer, workloads as W
    dev = DeviceBuffer.from_numpy
    c = W.make_decode_contiguous()
    dq, dk, dv = dev(c.q), dev(c.k_cache), dev(c.v_cache)
    out, lse = dev(np.zeros((32, 128), np.float32)), dev(np.zeros(32, np.float32))

    def step():
        gpu.decode_attention(q=dq, q_dtype=F32, k_cache=dk, v_cache=dv, out=out, lse=lse, batch_size=1,
                             num_heads=32, num_kv_heads=8, head_dim=128, scale=c.scale, max_seq=c.max_seq,
                             fixed_seq_len=c.seq_kv)

    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    res = {
        "workload": "decode_contiguous_ctx512_hq32_hkv8_d128", "metric": "decode_attn_latency_us", "unit": "us",
        "value": round(ms * 1e3, 2), "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall_ms, 4),
        "algorithmic_bytes": c.algorithmic_bytes(), "GBps": round(c.algorithmic_bytes() / (ms * 1e-3) / 1e9, 1),
        "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
        "note": "2 MB of traffic: launch-latency bound and cache resident; reported, no roofline target",
    }
    if cpu:
        import oracle_bind
        oracle = oracle_bind.load()
        reps, t0 = 0, time.perf_counter()
        while reps < 20 or time.perf_counter() - t0 < CPU_SAMPLE_SECONDS / 2:
            want, wl = oracle.attention_cached(c.q[None, None], c.k_cache, c.v_cache, c.seq_kv, c.seq_kv - 1,
                                               c.scale)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": round(cpu_s * 1e6, 1), "unit": "us",
                               "cores": oracle.lib.go_get_num_threads(), "kind": "port",
                               "sample": f"the whole workload, mean of {reps} passes (incl. the cache gather)"}
        res["parity"] = {"max_abs_err": max_err(out.read(np.float32, (32, 128)), want[0, 0]),
                         "max_lse_err": max_err(lse.read(np.float32, (32,)), wl[0, :, 0])}
    return res


def bench_copy_calibration(gpu, steps, warmup, cpu):
    """A plain copy of known size: the block-table gather with an identity
    table moves 2 x 128 MiB in and 2 x 128 MiB out.  Run under
    `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` it gives the factor between a
    counter's reading and real HBM bytes.  Not part of `--workload all`."""
    from granite_amd import DeviceBuffer
    hkv, d, bs, n_tok = 8, 128, 16, 65536
    rng = np.random.default_rng(7)
    pool = rng.integers(0, 1 << 16, size=(n_tok, hkv, d), dtype=np.uint16)
    table = np.arange(n_tok // bs, dtype=np.int32)
    dk, dv, dt = (DeviceBuffer.from_numpy(x) for x in (pool, pool[::-1].copy(), table))
    ok = DeviceBuffer.from_numpy(np.zeros((hkv, n_tok, d), np.uint16))
    ov = DeviceBuffer.from_numpy(np.zeros((hkv, n_tok, d), np.uint16))

    def step():
        gpu.paged_kv_gather(ok, ov, dk, dv, dt, hkv, d, n_tok, bs, n_tok)

    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    moved = 2 * pool.nbytes
    got = ok.read(np.uint16, (hkv, n_tok, d))
    return {"workload": "copy_calibration_gather_identity_65536tok_hkv8_d128", "metric": "copy_GBps",
            "unit": "GB/s", "value": round(2 * moved / (ms * 1e-3) / 1e9, 1), "ms_per_step": round(ms, 4),
            "wall_ms_per_step": round(wall_ms, 4), "bytes_read": moved, "bytes_written": moved,
            "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
            "parity": {"bit_exact": bool(np.array_equal(got, np.transpose(pool, (1, 0, 2))))}}


def bench_mfma_calibration(gpu, steps, warmup, cpu):
    """What the matrix cores reach on register operands (libgranite_hip_calibration.so, a
    measurement aid beside the attention library): zeros (the part keeps its peak clock)
    against normally distributed fp16 values (the power limit holds the clock down), both MFMA
    shapes, and then with the other instructions an attention inner loop issues per MFMA
    beside them -- float FMAs, exponentials, 16-byte LDS operand reads, scalar instructions --
    with one and with two waves per SIMD.  The mixes are given per pair of MFMAs; two of them
    are what the hardware counters report for the two prefill kernels (profiles/
    chunked_prefill.md: vector, LDS and scalar instructions per MFMA), so the rate of such a
    row is what that kernel's instruction mix leaves of the matrix cores with no tile staging,
    no barrier and no masks.  Not part of `--workload all`."""
    from granite_amd import DeviceBuffer, calibration
    rng = np.random.default_rng(11)
    n = 1 << 20
    data = {"zeros": np.zeros(n, np.float16),
            "normal": (0.05 * rng.standard_normal(n, dtype=np.float32)).astype(np.float16)}
    bufs = {k: DeviceBuffer.from_numpy(v) for k, v in data.items()}
    iterations = 20000

    def rate(kind, shape, waves, per_pair):
        best = 0.0
        for _ in range(max(1, min(steps, 3))):
            flops, ms = calibration.mfma_mix(bufs[kind], n, iterations, shape=shape, waves_per_simd=waves,
                                             per_pair=per_pair)
            best = max(best, flops / (ms * 1e-3) / 1e12)
        return round(best, 1)

    rates = {f"{kind}_{shape}": rate(kind, shape, 2, (0, 0, 0, 0)) for kind in data for shape in (32, 16)}
    mixes = {"mfma_only": (0, 0, 0, 0), "4_fma": (8, 0, 0, 0), "8_fma": (16, 0, 0, 0), "1_exp": (0, 2, 0, 0),
             "3_fma_1_exp": (6, 2, 0, 0), "1_lds_read": (0, 0, 2, 0), "3_fma_1_exp_1_lds_read": (6, 2, 2, 0),
             "3_fma_1_exp_half_lds_read": (6, 2, 1, 0),
             "3_fma_1_exp_1.5_lds_reads": (6, 2, 3, 0),
             "tiles_dma_kernel_mix_3_fma_1_exp_1.5_lds_2_salu": (6, 2, 3, 4),
             "tiles_kernel_mix_4_fma_1_exp_1.5_lds_3_salu": (8, 2, 3, 6),
             "rows64_mix_3.5_fma_1_exp_0.5_lds_1_salu": (7, 2, 1, 2)}
    mix_rates = {name: {f"{w}_wave_per_simd": rate("normal", 32, w, mix) for w in (1, 2)}
                 for name, mix in mixes.items()}
    return {"workload": "mfma_calibration_register_operands_one_workgroup_per_cu", "metric": "mfma_TFLOPs",
            "unit": "TFLOP/s", "value": rates["normal_32"], "ms_per_step": 0.0,
            "rates_TFLOPs": {"zeros_32x32x16": rates["zeros_32"], "zeros_16x16x32": rates["zeros_16"],
                             "normal_32x32x16": rates["normal_32"], "normal_16x16x32": rates["normal_16"]},
            "instruction_mix_per_pair_of_mfma": {k: list(v) for k, v in mixes.items()},
            "instruction_mix_TFLOPs_32x32x16_normal": mix_rates,
            "peak_TFLOPs": 2500.0}


def bench_rope_append(gpu, steps, warmup, cpu):
    """The step in front of the attention path: rotate Q and K (the reference's cos/sin tables
    as input) and append the rotated K and V to the paged cache in the same pass.  Shape: a
    prefill of 8192 tokens, 64 query heads, 8 KV heads, block 32 (the chunk of the chunked
    prefill config, 512 tokens at position 32768, is timed beside it: it is launch bound)."""
    from granite_amd import DeviceBuffer, ROUND_NEAREST
    dev = DeviceBuffer.from_numpy
    hq, hkv, d, bs = 64, 8, 128, 32
    import oracle_bind
    oracle = oracle_bind.load() if cpu else None

    def make(seq, start, seed):
        rng = np.random.default_rng(seed)
        q = rng.standard_normal((seq, hq, d), dtype=np.float32)
        k = rng.standard_normal((seq, hkv, d), dtype=np.float32)
        v = rng.standard_normal((seq, hkv, d), dtype=np.float32)
        positions = start + seq
        i = np.arange(d // 2, dtype=np.float32)
        freq = (1.0 / np.float32(10000.0) ** (2 * i / np.float32(d))).astype(np.float32)
        ang = (np.arange(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32)
        # the timed kernel's tables: built here (the angle in float as RoPECache does, src/llm/rope.cpp:5-22),
        # not taken from the checker; both sides of the parity leg below read these same arrays
        cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
        nblk = (positions + bs - 1) // bs
        table = rng.permutation(nblk).astype(np.int32)
        bufs = dict(q=dev(q), k=dev(k), v=dev(v), cos=dev(cos), sin=dev(sin), t=dev(table),
                    pk=dev(np.zeros((nblk * bs, hkv, d), np.uint16)),
                    pv=dev(np.zeros((nblk * bs, hkv, d), np.uint16)))
        host = dict(q=q, k=k, v=v, cos=cos, sin=sin, table=table, nblk=nblk)

        def step():
            gpu.rope_append(seq_len=seq, head_dim=d, start_pos=start, q=bufs["q"], num_heads_q=hq,
                            k=bufs["k"], num_heads_k=hkv, v=bufs["v"], cache_k=bufs["pk"], cache_v=bufs["pv"],
                            block_table=bufs["t"], block_size=bs, cos_table=bufs["cos"], sin_table=bufs["sin"],
                            table_positions=positions, write_k_back=False, rounding=ROUND_NEAREST)
        # Q read and written, K and V read, two half cache rows written, the cos/sin rows read
        nbytes = seq * (2 * hq * d * 4 + 2 * hkv * d * 4 + 2 * hkv * d * 2 + 2 * (d // 2) * 4)
        return step, bufs, host, nbytes

    step, bufs, host, nbytes = make(8192, 0, 21)
    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    c_step, _, _, c_bytes = make(512, 32768, 22)
    c_ms, _, c_kern = Timer(gpu).run(c_step, warmup, steps)
    res = {
        "workload": "rope_append_s8192_hq64_hkv8_d128_bs32", "metric": "rope_append_GBps", "unit": "GB/s",
        "value": round(nbytes / (ms * 1e-3) / 1e9, 1), "ms_per_step": round(ms, 4),
        "wall_ms_per_step": round(wall_ms, 4), "algorithmic_bytes": nbytes, "dtype": "f32 rotation, f16 cache",
        "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
        "chunk_512_at_32768": {"ms_per_step": round(c_ms, 4), "algorithmic_bytes": c_bytes,
                               "GBps": round(c_bytes / (c_ms * 1e-3) / 1e9, 1)},
        "note": "Q is rotated in place once per timed step (the values keep turning; the traffic is the same)",
    }
    res["roofline"] = roofline("hbm", nbytes, kern["rope_append"][0], profiled_traffic("rope_append", res["workload"]))
    res["roofline"]["kernel"] = "rope_append_kernel"
    if cpu:
        # parity on a fresh copy: one application against the oracle, bit for bit
        seq = 8192
        fresh_q, fresh_k = dev(host["q"]), dev(host["k"])
        gpu.rope_append(seq_len=seq, head_dim=d, start_pos=0, q=fresh_q, num_heads_q=hq, k=fresh_k,
                        num_heads_k=hkv, v=bufs["v"], cache_k=bufs["pk"], cache_v=bufs["pv"],
                        block_table=bufs["t"], block_size=bs, cos_table=bufs["cos"], sin_table=bufs["sin"],
                        table_positions=seq, write_k_back=True, rounding=ROUND_NEAREST)
        gpu.sync()
        passes, t0 = 0, time.perf_counter()
        while passes == 0 or time.perf_counter() - t0 < CPU_SAMPLE_SECONDS:
            want_q = oracle.rope_apply(host["q"], 0, host["cos"], host["sin"])
            want_k = oracle.rope_apply(host["k"], 0, host["cos"], host["sin"])
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        rows = host["table"][np.arange(seq) // bs] * bs + np.arange(seq) % bs
        pool_k = bufs["pk"].read(np.uint16, (host["nblk"] * bs, hkv, d))
        res["cpu_baseline"] = {"value": round(seq * (2 * hq * d * 4 + 2 * hkv * d * 4) / cpu_s / 1e9, 3), "unit": "GB/s",
                               "cores": 1, "kind": "port", "seconds": round(cpu_s * passes, 2),
                               "sample": f"the rotation of Q and K of the whole workload (no append), mean of {passes} passes"}
        res["parity"] = {"q_bit_exact": bool(np.array_equal(fresh_q.read(np.float32, host["q"].shape), want_q)),
                         "k_bit_exact": bool(np.array_equal(fresh_k.read(np.float32, host["k"].shape), want_k)),
                         "k_cache_bit_exact": bool(np.array_equal(pool_k[rows], want_k.astype(np.float16).view(np.uint16)))}
    return res


def bench_qkv_q4k(gpu, steps, warmup, cpu):
    """The projection in front of the attention path: Q, K and V of one decode token from
    Q4_K weights in one launch (hidden 4096, 32 query heads, 8 KV heads, D = 128), and the same
    for the 64 tokens of a batched decode step.  One pass over 14 MB of weights: at this size
    the launch itself is a good part of the time.  The timed steps walk through 32 copies of
    the weights (32 layers, 450 MB: more than the last-level cache holds), so every step reads
    its weights from HBM as a model's layers would; the figure with one set of weights re-read
    every step is reported beside it as cache resident."""
    from granite_amd import DeviceBuffer, workloads as W
    dev = DeviceBuffer.from_numpy
    c = W.make_qkv_projection(batch=64)
    K, nq, nkv = c.K, c.Nq, c.Nkv
    layers = 32
    dx = dev(c.x)
    weights_dev = [(dev(c.wq), dev(c.wk), dev(c.wv)) for _ in range(layers)]
    dwq, dwk, dwv = weights_dev[0]
    yq, yk, yv = (dev(np.zeros((64, n), np.float32)) for n in (nq, nkv, nkv))
    turn = [0]

    def next_layer():
        turn[0] = (turn[0] + 1) % layers
        return weights_dev[turn[0]]

    def step():
        wq, wk, wv = next_layer()
        gpu.fused_qkv_matvec_q4k(dx, wq, wk, wv, yq, yk, yv, K, nq, nkv)

    def step_resident():
        gpu.fused_qkv_matvec_q4k(dx, dwq, dwk, dwv, yq, yk, yv, K, nq, nkv)

    def step64():
        wq, wk, wv = next_layer()
        gpu.fused_qkv_matvec_q4k(dx, wq, wk, wv, yq, yk, yv, K, nq, nkv, batch=64)

    ms, wall_ms, kern = Timer(gpu).run(step, warmup, steps)
    ms_res, _, kern_res = Timer(gpu).run(step_resident, warmup, steps)
    ms64, _, kern64 = Timer(gpu).run(step64, warmup, steps)
    weights = c.wq.nbytes + c.wk.nbytes + c.wv.nbytes
    nbytes = weights + K * 4 + (nq + 2 * nkv) * 4
    res = {
        "workload": "fused_qkv_matvec_q4k_k4096_hq32_hkv8_d128_weights_of_32_layers_in_turn",
        "metric": "qkv_q4k_GBps", "unit": "GB/s",
        # the kernel's own duration (events around the launch), which is what the roofline below uses;
        # back-to-back steps overlap a launch's start-up with the previous kernel's tail, so the step
        # time can be the shorter of the two
        "value": round(nbytes / (kern["matvec_q4k"][0] * 1e-3) / 1e9, 1), "ms_per_step": round(ms, 4),
        "wall_ms_per_step": round(wall_ms, 4), "algorithmic_bytes": nbytes, "flops": 2 * K * (nq + 2 * nkv),
        "dtype": "4-bit weights, f32 accumulate", "kernels_ms": {k: round(v[0], 4) for k, v in kern.items()},
        "cache_resident": {"ms_per_step": round(ms_res, 4),
                           "kernels_ms": {k: round(v[0], 4) for k, v in kern_res.items()},
                           "GBps": round(nbytes / (kern_res["matvec_q4k"][0] * 1e-3) / 1e9, 1),
                           "note": "one set of weights re-read every step: served by the last-level cache, not HBM"},
        "batch_64": {"ms_per_step": round(ms64, 4), "kernels_ms": {k: round(v[0], 4) for k, v in kern64.items()},
                     "weights_GBps": round(weights / (ms64 * 1e-3) / 1e9, 1),
                     "note": "64 tokens on the matrix cores: one launch whose workgroups take two tiles of 32 "
                             "tokens through each unpacked weight, and a launch that adds the eight chunks of K"},
    }
    res["roofline"] = roofline("hbm", nbytes, kern["matvec_q4k"][0], profiled_traffic("qkv_q4k", res["workload"]))
    res["roofline"]["kernel"] = "matvec_q4k_kernel"
    if cpu:
        import oracle_bind
        oracle = oracle_bind.load()
        passes, t0 = 0, time.perf_counter()
        while passes == 0 or time.perf_counter() - t0 < CPU_SAMPLE_SECONDS / 2:
            want = [oracle.matvec_q4k(c.x[:1], w) for w in (c.wq, c.wk, c.wv)]
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        step_resident()
        gpu.sync()
        got = [b.read(np.float32, (1, n)) for b, n in ((yq, nq), (yk, nkv), (yv, nkv))]
        res["cpu_baseline"] = {"value": round(nbytes / cpu_s / 1e9, 3), "unit": "GB/s",
                               "cores": oracle.lib.go_get_num_threads(), "kind": "port",
                               "seconds": round(cpu_s * passes, 2),
                               "sample": f"the whole workload (dequantise every row, then the dot products), "
                                         f"mean of {passes} passes"}
        res["parity"] = {"max_abs_err": max(max_err(g, w) for g, w in zip(got, want))}
    return res


WORKLOADS = {
    "paged_decode": bench_paged_decode,
    "prefill": bench_prefill,
    "chunked_prefill": bench_chunked_prefill,
    "tree": bench_tree,
    "decode_contiguous": bench_decode_contiguous,
    "rope_append": bench_rope_append,
    "qkv_q4k": bench_qkv_q4k,
}
EXTRA_WORKLOADS = {"copy_calibration": bench_copy_calibration, "mfma_calibration": bench_mfma_calibration}


def main() -> int:
    global CLOCK_RAMP_MS, FLOAT_QUERY_LEG
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", choices=["all", *WORKLOADS, *EXTRA_WORKLOADS])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / parity leg")
    ap.add_argument("--no-float-queries", action="store_true",
                    help="prefill workloads: skip the second timing with float queries (profiling passes, so "
                         "that every counter belongs to the half-query kernel)")
    ap.add_argument("--ramp-ms", type=float, default=CLOCK_RAMP_MS,
                    help="untimed work in front of every measurement (0 for counter passes)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on exactly one GPU (--gpus 1); the attention path has no "
              "cross-GPU step (it would shard by KV head or by sequence).", file=sys.stderr)
        return 2

    CLOCK_RAMP_MS = args.ramp_ms
    FLOAT_QUERY_LEG = not args.no_float_queries
    from granite_amd import get_hip_compute
    gpu = get_hip_compute(0)
    info = gpu.device_info()
    log(f"device: {info.name.decode()} {info.arch.decode()} CUs={info.compute_units} clock={info.clock_khz} kHz")

    names = list(WORKLOADS) if args.workload == "all" else [args.workload]
    results = {}
    for name in names:
        t0 = time.perf_counter()
        fn = WORKLOADS.get(name) or EXTRA_WORKLOADS[name]
        results[name] = fn(gpu, args.steps, args.warmup, not args.no_cpu)
        log(f"[{name}] {results[name]['value']} {results[name]['unit']} "
            f"({results[name]['ms_per_step']} ms/step; {time.perf_counter() - t0:.1f}s total)")

    head = results.get("paged_decode") or results[names[0]]
    line = {
        "metric": head["metric"], "value": head["value"], "unit": head["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": head["unit"] != "us", "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": head["workload"], "q_dtype": head.get("q_dtype", "f16"),
                   "device": info.name.decode() or info.arch.decode(),
                   "arch": info.arch.decode(),
                   "compute_units": info.compute_units},
    }
    if "roofline" in head:
        line["roofline"] = head["roofline"]
    if "cpu_baseline" in head:
        line["cpu_baseline"] = head["cpu_baseline"]
    if "parity" in head:
        line["parity"] = head["parity"]
    line["workloads"] = results
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
