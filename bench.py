#!/usr/bin/env python3
"""Benchmark of the paged-attention decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--partition-size N]
    python bench.py --workload kv_write | kv_quantize      (the KV-cache write kernels, the step before the path)

A step is one call of the op (partition kernel + reduce kernel on one stream) on one batch of
synthetic input that is already resident in HBM.  Consecutive steps use different KV pools so the
256 MB Infinity Cache cannot serve the KV stream.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

METRIC = "µs/call + achieved KV HBM GB/s (% peak), FP8 KV, B=64 GQA8 ctx=4k"
HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the partition kernel from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what
# the counter reads for a plain copy of known size (profiles/pa_partition_kernel_c2_hbm_traffic.md,
# profiles/pa_partition_shared_kernel_c5_hbm_traffic.md); keyed by (workload, partition size) because the
# partial-output traffic depends on the partitioning
HBM_TRAFFIC_BYTES = {("c2_fp8_b64_ctx4k", 4096): 541_400_000, ("c5_ragged_mix", 7424): 2_050_400_000}


def _partition_kernel_name(wl):
    """The kernel the library launches for this workload: more than 16 query rows per kv head over an FP8
    cache go to the kernel whose row tiles share one pass over the pages."""
    ge = wl.q_len * (wl.num_q_heads // wl.num_kv_heads)
    fp8 = wl.key_cache.element_size() == 1
    return "pa_partition_shared_kernel" if (fp8 and ge > 16) else "pa_partition_kernel"


def _cpu_baseline(wl_cpu_sample, n_seq_sample, target_seconds=20.0):
    """The torch restatement of the reference's own oracle (oracle/pa_oracle.py, following
    test_pa_mtp.py:223-291) timed on the host cores over a few sequences of the same workload."""
    import torch

    from oracle import pa_oracle as O

    wl = wl_cpu_sample
    threads = torch.get_num_threads()

    def run(ids):
        return O.paged_attention_decode_oracle(
            wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
            wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, seq_ids=ids)

    run([0])  # warm-up
    t0, done = time.perf_counter(), 0
    while time.perf_counter() - t0 < target_seconds / 2:  # whole passes over the sample, >= 10 s in all
        for b in range(n_seq_sample):
            run([b])
            done += 1
    dt = time.perf_counter() - t0
    per_seq_bytes = wl.kv_bytes() / wl.batch
    return {
        "value": round(done * per_seq_bytes / dt / 1e9, 4),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "us_per_call_extrapolated": round(dt / done * 1e6 * _FULL_BATCH[0], 1),
        "sample": f"{done} single-sequence calls over the first {n_seq_sample} of {_FULL_BATCH[0]} sequences of "
                  f"the same workload, f32 torch ops, {dt:.1f} s wall on {threads} threads",
    }


_FULL_BATCH = [0]


def _bench_kv_cache(a) -> int:
    """The step before the decode path: `kv_write` appends 64 prompts of 4096 tokens (8 kv heads, head 128, bf16
    rows) to an FP8 paged cache with per-token scales in one call; `kv_quantize` converts the c2 cache pool
    (20480 pages of 16 tokens) from bf16 to FP8 with per-token scales.  Bytes counted: rows or cache read once,
    cache and scales written once."""
    import torch

    import triton_op_amd as T
    from triton_op_amd import _cabi
    from triton_op_amd import kv_layout as L

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    _cabi.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    h, d, bs = 8, 128, 16
    gen = torch.Generator(device=dev).manual_seed(7)
    if a.workload == "kv_write":
        ntok = 64 * 4096
        nblk = ntok // bs
        key = torch.randn(ntok, h, d, device=dev, generator=gen).to(torch.bfloat16)
        value = torch.randn(ntok, h, d, device=dev, generator=gen).to(torch.bfloat16)
        perm = torch.randperm(nblk, device=dev, generator=gen)
        slots = (perm.repeat_interleave(bs) * bs + torch.arange(ntok, device=dev) % bs).to(torch.int64)
        kc = torch.zeros(nblk, h, d // 16, bs, 16, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        vc = torch.zeros(nblk, h, d, bs, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        ks = torch.zeros(nblk, h, bs, 1, device=dev)
        vs = torch.zeros(nblk, h, bs, 1, device=dev)
        nbytes = ntok * h * (2 * d * 2 + 2 * d + 8)
        kernel, name = "kv_cache_write_tile_kernel", "kv_write_64x4096_fp8_token_scales"

        def step():
            T.kv_cache_write(key, value, kc, vc, slots, ks, vs)

        def cpu_sample():
            n = 4096
            k16 = L.tokens_to_key_cache(key[:n].cpu().view(n // bs, bs, h, d))
            v16 = L.tokens_to_value_cache(value[:n].cpu().view(n // bs, bs, h, d))
            t0 = time.perf_counter()
            L.quantize_kv_cache_per_token(k16, v16)
            return n * h * (2 * d * 2 + 2 * d + 8), time.perf_counter() - t0, f"{n} tokens"
    else:
        nblk = 20480
        kc16 = torch.randn(nblk, h, d // 8, bs, 8, device=dev, generator=gen).to(torch.bfloat16)
        vc16 = torch.randn(nblk, h, d, bs, device=dev, generator=gen).to(torch.bfloat16)
        nbytes = nblk * bs * h * (2 * d * 2 + 2 * d + 8)
        kernel, name = "quantize_kv_cache_tile_kernel", "kv_quantize_c2_pool"

        def step():
            T.quantize_kv_cache_symmetric(kc16, vc16, torch.float8_e4m3fn)

        def cpu_sample():
            n = 256
            k16, v16 = kc16[:n].cpu(), vc16[:n].cpu()
            t0 = time.perf_counter()
            L.quantize_kv_cache_per_token(k16, v16)
            return n * bs * h * (2 * d * 2 + 2 * d + 8), time.perf_counter() - t0, f"{n} pages"
    stream = torch.cuda.current_stream(dev)
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]
    t0 = time.perf_counter()
    for e0, e1 in evs:
        e0.record(stream)
        step()
        e1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / a.steps
    us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in evs)
    us_median = us[len(us) // 2]
    achieved = nbytes / (us_median * 1e-6) / 1e9
    result = {
        "metric": "KV-cache write GB/s (rows read + FP8 cache and scales written)", "value": round(achieved, 1),
        "unit": "GB/s", "us_per_call": round(us_median, 2), "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 in, fp8_e4m3fn + f32 scales out", "data": "synthetic",
        "config": {"workload": name, "kv_heads": h, "head_size": d, "block_size": bs, "bytes_per_call": nbytes},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None},
    }
    if not a.no_cpu_baseline:
        cpu_sample()  # warm-up
        tot_b, tot_dt, reps = 0, 0.0, 0
        while tot_dt < 10.0:  # a bounded sample, about 10 s of host work
            b, dt, what = cpu_sample()
            tot_b, tot_dt, reps = tot_b + b, tot_dt + dt, reps + 1
        result["cpu_baseline"] = {"value": round(tot_b / tot_dt / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(),
                                  "kind": "port",
                                  "sample": f"the torch formulas of kv_layout, {reps} passes over {what}, {tot_dt:.1f} s"}
    print(json.dumps(result, ensure_ascii=False))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--partition-size", type=int, default=0, help="0 = let the tuning layer choose")
    ap.add_argument("--pools", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--batch", type=int, default=0, help="override the batch size (debugging only)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the op shards by kv head or "
              "by sequence with no exchange); run with --gpus 1", file=sys.stderr)
        return 2

    if a.workload in ("kv_write", "kv_quantize"):
        return _bench_kv_cache(a)

    import torch

    import triton_op_amd as T
    from triton_op_amd import _cabi
    from triton_op_amd import workloads as W

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _cabi.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)

    # ---- workload: `pools` independent copies (different seeds) ----------------------------------------
    plans, wls = [], []
    for i in range(a.pools):
        wl = W.make_config(a.workload, device=dev, batch=a.batch or None)
        if i:
            # same shapes, different page contents and block tables
            cfg = dict(name=wl.name, seed=wl.meta["seed"] + 100 * i, batch=wl.batch, num_q_heads=wl.num_q_heads,
                       num_kv_heads=wl.num_kv_heads, block_size=wl.block_size, context_lens=wl.context_lens.cpu(),
                       q_len=wl.q_len, q_lens=None if wl.q_lens is None else wl.q_lens.cpu(),
                       kv_dtype=wl.meta["kv_dtype"], scale_mode=wl.meta["scale_mode"], device=dev)
            wl = W.make_decode_workload(**cfg)
        out = torch.empty_like(wl.query)
        ps = a.partition_size or None
        plan = T.plan_decode(out, wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                             wl.softmax_scale, wl.q_len, wl.max_context_len, torch.bfloat16, None, wl.key_scale,
                             wl.value_scale, partition_size=ps, query_lens=wl.q_lens)
        plans.append(plan)
        wls.append(wl)
    wl0 = wls[0]
    _FULL_BATCH[0] = wl0.batch
    kv_bytes = wl0.kv_bytes()
    stream = torch.cuda.current_stream(dev)
    sh = C.c_void_p(stream.cuda_stream)
    n = len(plans)

    def step(i):
        p = plans[i % n]
        rc = lib.pa_decode(C.byref(p.args), sh)
        if rc:
            _cabi.check(rc, "pa_decode")

    # ---- whole-op timing ---------------------------------------------------------------------------------
    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / a.steps

    # per-call device time from events on the launch stream (median is the headline µs/call)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]
    for i in range(a.steps):
        evs[i][0].record(stream)
        step(i)
        evs[i][1].record(stream)
    torch.cuda.synchronize()
    call_us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in evs)
    us_median = call_us[len(call_us) // 2]
    us_mean = sum(call_us) / len(call_us)

    # ---- the dominant kernel alone (roofline) --------------------------------------------------------------
    # Its average duration from HIP events on the launch stream.  When the partition kernel is the whole call
    # (one partition per sequence: c2), one event pair brackets the region of `steps`
    # back-to-back launches, which is what a kernel trace's average sees; otherwise other kernels run in
    # between and every launch gets an event pair of its own (which also brackets its dispatch).
    solo = plans[0].args.max_num_partitions == 1
    if solo:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(a.steps):
            rc = lib.pa_decode_partition(C.byref(plans[i % n].args), sh)
            if rc:
                _cabi.check(rc, "pa_decode_partition")
        e1.record(stream)
        torch.cuda.synchronize()
        k_us_avg = e0.elapsed_time(e1) * 1e3 / a.steps
        k_timing = f"one event pair around {a.steps} back-to-back launches"
    else:
        kevs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(a.steps)]
        for i in range(a.steps):
            p = plans[i % n]
            kevs[i][0].record(stream)
            rc = lib.pa_decode_partition(C.byref(p.args), sh)
            kevs[i][1].record(stream)
            if rc:
                _cabi.check(rc, "pa_decode_partition")
            if p.args.max_num_partitions > 1:
                lib.pa_decode_reduce(C.byref(p.args), sh)
        torch.cuda.synchronize()
        k_us = [e0.elapsed_time(e1) * 1e3 for e0, e1 in kevs]
        k_us_avg = sum(k_us) / len(k_us)
        k_timing = "an event pair around every launch (planning kernel included when the launch uses one)"
    achieved = kv_bytes / (k_us_avg * 1e-6) / 1e9

    # ---- a plain device copy, for scale -------------------------------------------------------------------
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(10):
        dst.copy_(src)
    e1.record(stream)
    torch.cuda.synchronize()
    copy_gbps = 10 * 2 * (1 << 30) / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst

    traffic = HBM_TRAFFIC_BYTES.get((wl0.name, int(plans[0].args.partition_size)))

    result = {
        "metric": METRIC,
        "value": round(kv_bytes / (us_median * 1e-6) / 1e9, 1),
        "unit": "GB/s (KV bytes / median µs per call)",
        "us_per_call": round(us_median, 2),
        "us_per_call_mean": round(us_mean, 2),
        "pct_of_hbm_peak": round(kv_bytes / (us_median * 1e-6) / 1e9 / HBM_PEAK_GBPS * 100, 2),
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn KV on FP8 MFMA (bf16 Q and P carried as two FP8 terms), f32 accumulate and softmax, bf16 out",
        "data": "synthetic",
        "config": {
            "workload": wl0.name,
            "batch": wl0.batch, "q_heads": wl0.num_q_heads, "kv_heads": wl0.num_kv_heads,
            "head_size": wl0.head_size, "q_len": wl0.q_len, "block_size": wl0.block_size,
            "context_len_max": wl0.max_context_len, "partition_size": int(plans[0].args.partition_size),
            "kv_bytes_per_call": kv_bytes, "kv_pools_rotated": n, "device": props.name,
            "compute_units": props.multi_processor_count,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": _partition_kernel_name(wl0),
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "kernel_us_avg": round(k_us_avg, 2),
            "kernel_timing": k_timing,
            "algorithmic_bytes_per_launch": kv_bytes,
            "device_copy_GBps": round(copy_gbps, 1),
        },
    }
    if not a.no_cpu_baseline:
        # a bounded sample: the first sequences of pool 0, copied to the host
        nsamp = min(wl0.batch, 16)
        result["cpu_baseline"] = _cpu_baseline(wl0.to("cpu"), nsamp)
    print(json.dumps(result, ensure_ascii=False))
    return 0


if __name__ == "__main__":
    sys.exit(main())
