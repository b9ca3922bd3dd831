#!/usr/bin/env python3
"""Benchmark of the paged-attention decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]            the headline (c2) plus c2 and c4 at the reference's
                                                                     256-token partitions, c3, c4 and c5 in `configs`
    python bench.py --workload c1|c2|c3|c4|c5 [--partition-size N]   one configuration
    python bench.py --workload ref:B,Hq,Hkv,bs,qlen[,transv][,ctx=N]  one row of the reference harness's sweep
    python bench.py --workload custom:b=..,hq=..,hkv=..,q=..,ctx=..[,bs=..,scale=token|tensor,kv=fp8|bf16,qdtype=bf16|fp8,transv=0|1,hd=64|128|256]
                               [,lens=c5[,cap=N][,qlens=c5|N][,pick=one|rest]]   c5's draw of context lengths (and of new tokens per sequence)
    python bench.py --workload probe_gather                          read-only probe of c2's page-gather pattern
    python bench.py --workload probe_gather:c5                       ... of another workload's (plain order, four-wave workgroups)
    python bench.py --workload probe_stream42:c5                     the pages read by workgroups whose waves share each step
                                                                     (depth 4 steps in registers, 2 workgroups per CU)
    python bench.py --workload probe_issue                           issue cost of the decode step's instructions
    python bench.py --workload trace:c5                              where a workgroup slot's time goes (measuring build)
    python bench.py --workload kv_write | kv_quantize                the KV-cache write kernels, the step before the path

A step is one call of the op (partition kernel + reduce kernel on one stream) on one batch of synthetic input
that is already resident in HBM.  Consecutive steps use different KV pools so the 256 MB last-level cache
cannot serve the KV stream.  Prints ONE JSON line.

`ref:` builds the inputs the reference harness builds (test_pa_mtp.py:660-722,763-783): uniform(-1,1) bf16 query
and cache, a pool of 16384 tokens' worth of pages per sequence, block tables drawn with replacement, the cache
quantised per (block, head, token), the query per row (FP8 query with per-row scales: the Gluon entry point's
contract), context length 4096 unless given.  Every decode line also carries the reference's own bandwidth figure
(test_pa_mtp.py:937-945: K, V, query and output bytes over the time, in units of 1.024^4 * 1e12 B/s).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

METRIC = "µs/call + achieved KV HBM GB/s (% peak), FP8 KV, B=64 GQA8 ctx=4k"
HBM_PEAK_GBPS = 8000.0
SETTLE_CALLS = 100  # untimed calls before anything is measured (clocks and power state settle), not part of --warmup

# HBM bytes per launch of the partition kernel from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what the
# counter reads for a plain copy of known size.  An entry holds for ONE (workload, partition size, launch) as
# pa_decode_launch_info names it: when the launch layer or a kernel's instantiation changes, the figure is stale and
# the line carries null and a note instead.
HBM_TRAFFIC = {
    ("c2_fp8_b64_ctx4k", 4096): {
        "bytes": 541_400_000, "launch": "pa_partition_kernel<fp8, bs16, 4 waves> x 512",
        "profile": "profiles/pa_partition_kernel_c2_hbm_traffic.md"},
    ("c2_fp8_b64_ctx4k", 256): {
        "bytes": 557_700_000,
        "launch": "pa_partition_kernel<fp8, bs16, 1 waves> x 512, teams of 4 waves, 4 partitions per wave, no reduce kernel",
        "profile": "profiles/pa_partition_kernel_c2_hbm_traffic.md"},
    ("c3_fp8_mtp2_bs1024", 8192): {
        "bytes": 4_437_300_000, "launch": "pa_partition_kernel<fp8, strided, 4 waves> x 4096, sorted items",
        "profile": "profiles/pa_partition_kernel_c3_c4_hbm_traffic.md"},
    ("c4_fp8_ctx128k", 8192): {
        "bytes": 1_077_200_000, "launch": "pa_partition_kernel<fp8, bs16, 4 waves> x 512",
        "profile": "profiles/pa_partition_kernel_c3_c4_hbm_traffic.md"},
    ("c4_fp8_ctx128k", 256): {
        "bytes": 1_110_800_000, "launch": "pa_partition_kernel<fp8, bs16, 1 waves> x 2048, 8 partitions per workgroup",
        "profile": "profiles/pa_partition_kernel_c3_c4_hbm_traffic.md"},
    ("c5_ragged_mix", 7424): {
        "bytes": 1_991_300_000,
        "launch": "pa_partition_shared_kernel<fp8 per-token, bs16, 3 ring slots, 3 workgroups per CU> x 8192, sorted items, "
                  "an item's heads on one XCD",
        "profile": "profiles/pa_partition_shared_kernel_c5_hbm_traffic.md"},
    ("c5_ragged_mix", 7424, "output_only"): {
        "bytes": 1_943_700_000,
        "launch": "pa_partition_shared_kernel<fp8 per-token, bs16, 3 ring slots, 3 workgroups per CU> x 8192, sorted items, "
                  "an item's heads on one XCD",
        "profile": "profiles/pa_partition_shared_kernel_c5_hbm_traffic.md"},
}


# ---------------------------------------------------------------------------------------------------------------
# workloads
# ---------------------------------------------------------------------------------------------------------------
def _parse_kv(text):
    out = {}
    for item in text.split(","):
        if not item:
            continue
        k, _, v = item.partition("=")
        out[k.strip()] = v.strip()
    return out


def _make_ref_workload(spec, device, seed):
    """One row of the reference harness's sweep, inputs made as the harness makes them."""
    import torch

    import triton_op_amd as T
    from triton_op_amd import kv_layout as L
    from triton_op_amd.workloads import Workload

    parts = spec.split(",")
    b, hq, hkv, bs, qlen = (int(x) for x in parts[:5])
    transv, ctx = False, 4096
    for x in parts[5:]:
        if x == "transv":
            transv = True
        elif x.startswith("ctx="):
            ctx = int(x[4:])
        else:
            raise ValueError(f"ref: unknown field {x!r}")
    d = 128
    blocks_per_seq = (ctx + bs - 1) // bs
    total_blocks = ((16384 + bs - 1) // bs) * b
    gen = torch.Generator(device=device).manual_seed(seed)
    kc16, vc16 = L.create_kv_cache(total_blocks, bs, hkv, d, torch.bfloat16, generator=gen, device=device)
    kq, _, vq, _, ks, vs = T.quantize_kv_cache_symmetric(kc16, vc16, torch.float8_e4m3fn)
    del kc16, vc16
    if transv:
        vq = L.shuffle_value_cache_layout(vq)
    q_tok = torch.empty(b * qlen, hq, d, device=device).uniform_(-1.0, 1.0, generator=gen).to(torch.bfloat16)
    q8, q8s = L.pertoken_quant(L.mtp_pack(q_tok, b, qlen, hkv).contiguous().float())
    bt = torch.randint(0, total_blocks, (b, blocks_per_seq), generator=gen, device=device, dtype=torch.int32)
    return Workload(
        name=f"ref_b{b}_h{hq}x{hkv}_bs{bs}_q{qlen}{'_transv' if transv else ''}_ctx{ctx}", query=q8, key_cache=kq,
        value_cache=vq, context_lens=torch.full((b,), ctx, dtype=torch.int32, device=device), block_tables=bt,
        softmax_scale=1.0 / math.sqrt(d), q_len=qlen, q_lens=None, key_scale=ks, value_scale=vs, partition_size=256,
        num_kv_heads=hkv, num_q_heads=hq, head_size=d, block_size=bs, max_context_len=ctx,
        meta={"seed": seed, "pool_blocks": total_blocks, "kv_dtype": "fp8", "scale_mode": "token",
              "query_scale": q8s.contiguous(), "distribution": "uniform(-1,1), block tables with replacement"})


def _make_custom_workload(spec, device, seed):
    import torch

    from triton_op_amd import kv_layout as L
    from triton_op_amd import workloads as W

    kv = _parse_kv(spec)
    b, hq, hkv = int(kv.get("b", 64)), int(kv.get("hq", 64)), int(kv.get("hkv", 8))
    q, ctx, bs = int(kv.get("q", 1)), int(kv.get("ctx", 4096)), int(kv.get("bs", 16))
    scale, kvd, qd = kv.get("scale", "tensor"), kv.get("kv", "fp8"), kv.get("qdtype", "bf16")
    transv = kv.get("transv", "0") == "1"
    hd = int(kv.get("hd", 128))  # head size: 128 on the tuned kernels, 64 / 256 on the generic ones
    unknown = set(kv) - {"b", "hq", "hkv", "q", "ctx", "bs", "scale", "kv", "qdtype", "transv", "lens", "qlens", "pick", "hd", "cap"}
    if unknown:
        raise ValueError(f"custom: unknown keys {sorted(unknown)}")
    ctx_lens, q_lens, tag = torch.full((b,), ctx, dtype=torch.int32), None, f"ctx{ctx}"
    if kv.get("lens") == "c5":
        # the ragged configuration's own draw of context lengths (and of new tokens per sequence: qlens=c5), for
        # experiments that vary one thing about it; qlens=N gives every sequence N new tokens in buffers padded to q
        gen = W._gen("cpu", 5, 9)
        ctx_lens = W._lognormal_ctx(b, 2048, 1.0, 16, 65536, gen)
        drawn = torch.randint(1, 5, (b,), generator=gen, dtype=torch.int32)
        tag = "c5lens"
        if "cap" in kv:  # cap=N: no context longer than N tokens
            ctx_lens = torch.clamp(ctx_lens, max=int(kv["cap"]))
            tag += f"_cap{kv['cap']}"
        if "qlens" in kv:
            q_lens = drawn if kv["qlens"] == "c5" else torch.full((b,), int(kv["qlens"]), dtype=torch.int32)
            q_lens = torch.clamp(q_lens, max=q)
            ctx_lens = torch.maximum(ctx_lens, q_lens)
            tag += f"_qlens{kv['qlens']}"
        if "pick" in kv:  # pick=one: only the sequences that drew one new token; pick=rest: the others
            keep = (drawn == 1) if kv["pick"] == "one" else (drawn != 1)
            ctx_lens, b = ctx_lens[keep], int(keep.sum())
            q_lens = None if q_lens is None else q_lens[keep]
            tag += f"_pick{kv['pick']}"
    elif "lens" in kv or "qlens" in kv:
        raise ValueError("custom: lens=c5 is the only length distribution on offer; qlens needs it")
    wl = W.make_decode_workload(
        name=f"custom_b{b}_h{hq}x{hkv}_bs{bs}_q{q}_{tag}_{kvd}_{scale}_{qd}q{'_transv' if transv else ''}{'' if hd == 128 else f'_hd{hd}'}",
        seed=seed, batch=b, num_q_heads=hq, num_kv_heads=hkv, block_size=bs, head_size=hd,
        context_lens=ctx_lens, q_len=q, q_lens=q_lens, kv_dtype=kvd,
        scale_mode="none" if kvd == "bf16" else scale, device=device, transposed_v=transv)
    if qd == "fp8":
        q8, q8s = L.pertoken_quant(wl.query.float())
        wl.query = q8
        wl.meta["query_scale"] = q8s.contiguous()
    return wl


def _make_workload(name, device, pool_index, batch=None):
    from triton_op_amd import workloads as W

    if name.startswith("ref:"):
        return _make_ref_workload(name[4:], device, 1234 + 100 * pool_index)
    if name.startswith("custom:"):
        return _make_custom_workload(name[7:], device, 77 + 100 * pool_index)
    wl = W.make_config(name, device=device, batch=batch)
    if pool_index:
        # same shapes, different page contents and block tables
        wl = W.make_decode_workload(
            name=wl.name, seed=wl.meta["seed"] + 100 * pool_index, batch=wl.batch, num_q_heads=wl.num_q_heads,
            num_kv_heads=wl.num_kv_heads, block_size=wl.block_size, context_lens=wl.context_lens.cpu(), q_len=wl.q_len,
            q_lens=None if wl.q_lens is None else wl.q_lens.cpu(), kv_dtype=wl.meta["kv_dtype"],
            scale_mode=wl.meta["scale_mode"], device=device)
    return wl


def _reference_bandwidth_tbps(wl, us):
    """The reference harness's bandwidth figure (test_pa_mtp.py:937-945):
    B*D*(2*ctx*Hkv*sizeof(kv) + 2*qlen*Hq*sizeof(q)) / (us * 1e6 * 1.024**4); sums over the batch when ragged."""
    import torch

    tokens = int(wl.context_lens.to(torch.int64).sum())
    q_rows = int(wl.q_lens.to(torch.int64).sum()) if wl.q_lens is not None else wl.batch * wl.q_len
    nbytes = wl.head_size * (2 * tokens * wl.num_kv_heads * wl.key_cache.element_size() +
                             2 * q_rows * wl.num_q_heads * wl.query.element_size())
    return nbytes / (us * 1e6 * 1.024 ** 4)


def _dtype_text(wl):
    kv = "fp8_e4m3fn" if wl.key_cache.element_size() == 1 else "bf16"
    q = "fp8_e4m3fn" if wl.query.element_size() == 1 else "bf16"
    if kv == "bf16":
        return "bf16 KV and Q on bf16 MFMA, f32 accumulate and softmax, bf16 out"
    return (f"{kv} KV on FP8 MFMA ({q} Q" + (" and P" if q != "bf16" else " and P, each") +
            " carried as FP8 head + residual), f32 accumulate and softmax, bf16 out")


# ---------------------------------------------------------------------------------------------------------------
# timing of one decode configuration
# ---------------------------------------------------------------------------------------------------------------
class _Config:
    """`pools` independent copies of one workload with their validated plans."""

    def __init__(self, name, dev, pools, partition_size=None, batch=None, shared_from=None, output_only=False):
        import torch

        import triton_op_amd as T

        self.wls = shared_from.wls if shared_from is not None else [
            _make_workload(name, dev, i, batch) for i in range(pools)]
        self.plans = []
        # The KV pools rotate from call to call (a decode step reads every layer's cache once); the output, the
        # partition buffers and the workspace are the same memory in every call, as in an engine that reuses its
        # activation buffers from layer to layer (with buffers of their own per pool, c5's 70 MB of partial results
        # and outputs per call cost it 5 %: re-written lines stay in the last-level cache, fresh ones go to HBM).
        out = torch.empty(self.wls[0].query.shape, dtype=torch.bfloat16, device=dev)
        shared = {}
        for wl in self.wls:
            # the two context-length statistics a serving engine has on the host: the longest and the sum
            plan = T.plan_decode(
                out, wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
                wl.q_len, wl.max_context_len, torch.bfloat16, wl.meta.get("query_scale"), wl.key_scale, wl.value_scale,
                partition_size=partition_size or None, query_lens=wl.q_lens,
                total_context_tokens=int(wl.context_lens.to(torch.int64).sum()), output_only=output_only, **shared)
            if not shared:
                shared = dict(max_logits=plan.max_logits, exp_sums=plan.exp_sums, tmp_output=plan.tmp_output,
                              workspace=plan.workspace)
            self.plans.append(plan)
        self.wl0 = self.wls[0]
        self.kv_bytes = self.wl0.kv_bytes()
        self.partition_size = int(self.plans[0].args.partition_size)
        self.output_only = output_only
        self.launch = self.plans[0].launch_info()
        self.kernel = self.launch.split("<")[0]


def _time_config(lib, cfg, stream, steps, warmup, settle):
    """Returns the timings of one configuration.  Order: `settle` untimed calls; the partition kernel alone
    (roofline); `warmup` untimed calls and exactly `steps` calls between two synchronisations (ms_per_step); the same
    `steps` calls again with an event pair around each (median µs per call)."""
    import torch

    from triton_op_amd import _cabi

    sh = C.c_void_p(stream.cuda_stream)
    plans, n = cfg.plans, len(cfg.plans)

    def call(i):
        rc = lib.pa_decode(C.byref(plans[i % n].args), sh)
        if rc:
            _cabi.check(rc, "pa_decode")

    for i in range(settle):
        call(i)
    torch.cuda.synchronize()

    # ---- the dominant kernel alone.  When the partition kernel is the whole call (one partition per sequence), one
    # event pair brackets `steps` back-to-back launches, which is what a kernel trace's average sees; otherwise other
    # kernels run in between and every launch gets an event pair of its own (which also brackets its dispatch).
    # (a launch in teams merges in the partition kernel: pa_decode is that one kernel, pa_decode_partition another launch)
    team = "no reduce kernel" in cfg.launch
    solo = plans[0].args.max_num_partitions == 1 or team
    if "own partitions of " in cfg.launch:  # (output-only: the library's own cut of the partition axis; one partition?)
        own = int(cfg.launch.split("own partitions of ")[1].split()[0])
        solo = solo or own >= plans[0].args.max_num_partitions * plans[0].args.partition_size
    r_us_avg = None
    if solo:
        k_launches = max(steps, 100)  # (a short run's 20 launches would mostly measure the first one's ramp)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(k_launches):
            rc = (lib.pa_decode if team else lib.pa_decode_partition)(C.byref(plans[i % n].args), sh)
            if rc:
                _cabi.check(rc, "pa_decode_partition")
        e1.record(stream)
        torch.cuda.synchronize()
        k_us_avg = e0.elapsed_time(e1) * 1e3 / k_launches
        k_timing = f"one event pair around {k_launches} back-to-back launches"
    else:
        kevs = [tuple(torch.cuda.Event(enable_timing=True) for _ in range(3)) for _ in range(steps)]
        for i in range(steps):
            p = plans[i % n]
            kevs[i][0].record(stream)
            rc = lib.pa_decode_partition(C.byref(p.args), sh)
            kevs[i][1].record(stream)
            if rc:
                _cabi.check(rc, "pa_decode_partition")
            lib.pa_decode_reduce(C.byref(p.args), sh)
            kevs[i][2].record(stream)
        torch.cuda.synchronize()
        k_us = [e0.elapsed_time(e1) * 1e3 for e0, e1, _ in kevs]
        k_us_avg = sum(k_us) / len(k_us)
        # (stage 2 over every sequence, as pa_decode_reduce runs it alone; inside pa_decode it skips the sequences
        # stage 1 has finished)
        r_us_avg = sum(e1.elapsed_time(e2) * 1e3 for _, e1, e2 in kevs) / len(kevs)
        k_timing = "an event pair around every launch (planning kernel included when the launch uses one)"

    # ---- the whole op
    for i in range(warmup):
        call(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        call(i)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i in range(steps):
        evs[i][0].record(stream)
        call(i)
        evs[i][1].record(stream)
    torch.cuda.synchronize()
    call_us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in evs)
    return {"us_median": call_us[len(call_us) // 2], "us_mean": sum(call_us) / len(call_us), "wall_ms": wall_ms,
            "kernel_us_avg": k_us_avg, "kernel_timing": k_timing, "reduce_us_avg": r_us_avg}


def _sample_power(lib, cfg, stream, seconds):
    """Keeps the configuration's call running back to back for `seconds` and, from the third second on, reads the
    board's socket power (amd-smi) and shader clock (rocm-smi) once a second in child processes: what the kernels
    are given to run on once the power management has settled.  Returns None where the tools give nothing."""
    import re
    import subprocess
    import threading

    import torch

    from triton_op_amd import _cabi

    sh = C.c_void_p(stream.cuda_stream)
    plans, n = cfg.plans, len(cfg.plans)
    samples = {"socket_power_W": [], "sclk_MHz": []}
    stop = threading.Event()

    def tool(cmd, pattern):
        try:
            out = subprocess.run(cmd, capture_output=True, text=True, timeout=10).stdout
        except (OSError, subprocess.TimeoutExpired):
            return None
        m = re.search(pattern, out)
        return float(m.group(1)) if m else None

    def sampler():
        if stop.wait(2.0):
            return
        while not stop.is_set():
            w = tool(["amd-smi", "metric", "-p"], r"SOCKET_POWER:\s*([0-9.]+)\s*W")
            c = tool(["rocm-smi", "--showclocks"], r"sclk clock level: \d+: \(([0-9.]+)Mhz\)")
            if w is not None:
                samples["socket_power_W"].append(w)
            if c is not None:
                samples["sclk_MHz"].append(c)
            stop.wait(1.0)

    th = threading.Thread(target=sampler, daemon=True)
    th.start()
    t0, calls = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for i in range(200):
            rc = lib.pa_decode(C.byref(plans[(calls + i) % n].args), sh)
            if rc:
                _cabi.check(rc, "pa_decode")
        calls += 200
        torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    stop.set()
    th.join(15.0)
    cap = tool(["rocm-smi", "--showmaxpower"], r"Max Graphics Package Power \(W\):\s*([0-9.]+)")
    if not samples["socket_power_W"] and not samples["sclk_MHz"]:
        return None
    return {"seconds": round(dt, 1), "calls": calls, "us_per_call_wall": round(dt / calls * 1e6, 2),
            "socket_power_W": samples["socket_power_W"], "sclk_MHz": samples["sclk_MHz"], "power_cap_W": cap,
            "how": "amd-smi metric -p and rocm-smi --showclocks, once a second from the third second of a back-to-back loop"}


def _traffic(cfg):
    entry = HBM_TRAFFIC.get((cfg.wl0.name, cfg.partition_size, "output_only") if cfg.output_only
                            else (cfg.wl0.name, cfg.partition_size))
    if entry is None:
        return None, "no rocprofv3 FETCH_SIZE/WRITE_SIZE measurement on record for this workload and partition size"
    if entry["launch"] != cfg.launch:
        return None, (f"the figure on record ({entry['profile']}) was measured on '{entry['launch']}', "
                      f"this run launches '{cfg.launch}'")
    return entry["bytes"], entry["profile"]


def _config_line(cfg, t):
    """The short record of a configuration for the `configs` array of the headline line."""
    achieved = cfg.kv_bytes / (t["kernel_us_avg"] * 1e-6) / 1e9
    return {
        "workload": cfg.wl0.name, "partition_size": cfg.partition_size,
        # PA_DECODE_FLAG_OUTPUT_ONLY: the caller reads only the real query rows of `output` (include/pa_decode.h)
        "output_only": cfg.output_only, "us_per_call": round(t["us_median"], 2),
        "kv_GBps": round(cfg.kv_bytes / (t["us_median"] * 1e-6) / 1e9, 1), "kernel": cfg.kernel, "launch": cfg.launch,
        "kernel_us_avg": round(t["kernel_us_avg"], 2), "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "reduce_us_avg": None if t["reduce_us_avg"] is None else round(t["reduce_us_avg"], 2),
        "partitions_per_sequence": int(cfg.plans[0].args.max_num_partitions),
        "algorithmic_bytes_per_launch": cfg.kv_bytes,
        "traffic": _traffic(cfg)[0],  # HBM bytes per launch of the partition kernel by FETCH_SIZE + WRITE_SIZE (profiles/)
        "reference_formula_TBps": round(_reference_bandwidth_tbps(cfg.wl0, t["us_median"]), 3),
    }


def _cpu_baseline(wl, n_seq_sample, full_batch, target_seconds=20.0):
    """The torch restatement of the reference's own oracle (oracle/pa_oracle.py, following
    test_pa_mtp.py:223-291) timed on the host cores over a few sequences of the same workload."""
    import torch

    from oracle import pa_oracle as O

    threads = torch.get_num_threads()

    def run(ids):
        return O.paged_attention_decode_oracle(
            wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
            wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, seq_ids=ids,
            query_scale=wl.meta.get("query_scale"))

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
        "us_per_call_extrapolated": round(dt / done * 1e6 * full_batch, 1),
        "sample": f"{done} single-sequence calls over the first {n_seq_sample} of {full_batch} sequences of "
                  f"the same workload, f32 torch ops, {dt:.1f} s wall on {threads} threads",
    }


def _device_copy_gbps(dev, stream):
    import torch

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
    return 10 * 2 * (1 << 30) / (e0.elapsed_time(e1) * 1e-3) / 1e9


def _bench_decode(a) -> int:
    import torch

    from triton_op_amd import _cabi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _cabi.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    stream = torch.cuda.current_stream(dev)

    headline = a.workload or "c2"
    cfg = _Config(headline, dev, a.pools, a.partition_size, a.batch or None, output_only=a.output_only)
    t = _time_config(lib, cfg, stream, a.steps, a.warmup, a.settle)
    wl0 = cfg.wl0
    achieved = cfg.kv_bytes / (t["kernel_us_avg"] * 1e-6) / 1e9
    traffic, traffic_note = _traffic(cfg)
    value = cfg.kv_bytes / (t["us_median"] * 1e-6) / 1e9
    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s (KV bytes / median µs per call)",
        "us_per_call": round(t["us_median"], 2),
        "us_per_call_mean": round(t["us_mean"], 2),
        "pct_of_hbm_peak": round(value / HBM_PEAK_GBPS * 100, 2),
        "reference_formula_TBps": round(_reference_bandwidth_tbps(wl0, t["us_median"]), 3),
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "settle_calls": a.settle,
        "ms_per_step": round(t["wall_ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": _dtype_text(wl0),
        "data": "synthetic",
        "config": {
            "workload": wl0.name,
            "batch": wl0.batch, "q_heads": wl0.num_q_heads, "kv_heads": wl0.num_kv_heads,
            "head_size": wl0.head_size, "q_len": wl0.q_len, "block_size": wl0.block_size,
            "context_len_max": wl0.max_context_len, "partition_size": cfg.partition_size,
            "kv_bytes_per_call": cfg.kv_bytes, "kv_pools_rotated": len(cfg.plans), "device": props.name,
            "compute_units": props.multi_processor_count,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": cfg.kernel,
            "launch": cfg.launch,
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_note": traffic_note,
            "kernel_us_avg": round(t["kernel_us_avg"], 2),
            "kernel_timing": t["kernel_timing"],
            "algorithmic_bytes_per_launch": cfg.kv_bytes,
        },
    }

    # ---- the other configurations, driver-visible in the same line (the default run only) ----------------------
    if not a.workload and not a.no_configs:
        lines = []
        # c2 at the configuration's literal partition size 256 (the reference's constant): same pools
        c2_256 = _Config("c2", dev, a.pools, 256, shared_from=cfg)
        lines.append(_config_line(c2_256, _time_config(lib, c2_256, stream, min(a.steps, 100), 10, a.settle)))
        # ... and the same reference-shaped buffers as scratch (PA_DECODE_FLAG_OUTPUT_ONLY): the library cuts the
        # partition axis its own way inside them
        c2_256_lean = _Config("c2", dev, a.pools, 256, shared_from=c2_256, output_only=True)
        lines.append(_config_line(c2_256_lean, _time_config(lib, c2_256_lean, stream, min(a.steps, 100), 10, a.settle)))
        del c2_256, c2_256_lean
        for name in ("c3", "c4", "c5"):
            other = _Config(name, dev, 1)  # each of them streams far more than the last-level cache holds
            lines.append(_config_line(other, _time_config(lib, other, stream, min(a.steps, 100), 10, a.settle)))
            if name == "c4":
                # ... and at the configuration's literal partition size: 512 partitions per sequence, the merge of
                # which is what the configuration is there to stress
                c4_256 = _Config("c4", dev, 1, 256, shared_from=other)
                lines.append(_config_line(c4_256, _time_config(lib, c4_256, stream, min(a.steps, 100), 10, a.settle)))
                c4_256_lean = _Config("c4", dev, 1, 256, shared_from=c4_256, output_only=True)
                lines.append(_config_line(c4_256_lean, _time_config(lib, c4_256_lean, stream, min(a.steps, 100), 10, a.settle)))
                del c4_256, c4_256_lean
            if name == "c5":
                # ... and as an engine calls it that reads only the real query rows of `output`: no partition-buffer
                # entries for the sequences stage 1 finishes, no zeros for the rows beyond a sequence's query length
                c5_lean = _Config("c5", dev, 1, shared_from=other, output_only=True)
                lines.append(_config_line(c5_lean, _time_config(lib, c5_lean, stream, min(a.steps, 100), 10, a.settle)))
                del c5_lean
            del other
            torch.cuda.empty_cache()
        result["configs"] = lines

    result["roofline"]["device_copy_GBps"] = round(_device_copy_gbps(dev, stream), 1)
    if a.power_seconds > 0:
        result["power"] = _sample_power(lib, cfg, stream, a.power_seconds)
    if not a.no_cpu_baseline:
        # a bounded sample: the first sequences of pool 0, copied to the host
        nsamp = min(wl0.batch, 16)
        result["cpu_baseline"] = _cpu_baseline(wl0.to("cpu"), nsamp, wl0.batch)
    print(json.dumps(result, ensure_ascii=False))
    return 0


# ---------------------------------------------------------------------------------------------------------------
# the read-only probe of c2's gather pattern
# ---------------------------------------------------------------------------------------------------------------
def _load_probe_library():
    """libpa_probe.so: the two measuring kernels (tests/native/pa_probe.h), a library of their own beside the
    operator's; built by `python -m triton_op_amd.build`."""
    from triton_op_amd import _cabi

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "native", "libpa_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `python -m triton_op_amd.build`")
    lib = C.CDLL(path)
    lib.pa_probe_gather.restype = C.c_int
    lib.pa_probe_gather.argtypes = [C.POINTER(_cabi.PaDecodeArgs), C.c_void_p, C.c_void_p]
    lib.pa_probe_stream.restype = C.c_int
    lib.pa_probe_stream.argtypes = [C.POINTER(_cabi.PaDecodeArgs), C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.pa_probe_issue.restype = C.c_int
    lib.pa_probe_issue.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    return lib


def _bench_probe_gather(a) -> int:
    """Reads exactly the pages c2's partition kernel reads, in the same order and grouping (one workgroup of four
    waves per (sequence, kv head), each wave every fourth 64-token step, 16 bytes per lane, non-temporal), and does
    no arithmetic: what the memory system gives this access pattern."""
    import torch

    from triton_op_amd import _cabi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _load_probe_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev)
    sh = C.c_void_p(stream.cuda_stream)
    of = a.workload.partition(":")[2] or "c2"  # probe_gather:c5, probe_gather:custom:... = that workload's pages
    cfg = _Config(of, dev, a.pools, a.partition_size, a.batch or None)
    sink = torch.zeros(64, dtype=torch.int32, device=dev)

    # probe_gather | probe_stream42 (depth 4, 2 workgroups per CU) | probe_stream42v1 (+ variant: 1 no barrier, 2 no scales)
    shape, _, variant = a.workload.partition(":")[0].partition("v")

    def call(i):
        args = C.byref(cfg.plans[i % len(cfg.plans)].args)
        if shape == "probe_gather":
            rc = lib.pa_probe_gather(args, C.c_void_p(sink.data_ptr()), sh)
        else:
            rc = lib.pa_probe_stream(args, int(shape[-2]), int(shape[-1]), int(variant or 0), C.c_void_p(sink.data_ptr()), sh)
        if rc:
            _cabi.check(rc, shape)

    for i in range(a.settle):
        call(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for i in range(a.steps):
        call(i)
    e1.record(stream)
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / a.steps
    gbps = cfg.kv_bytes / (us * 1e-6) / 1e9
    print(json.dumps({
        "metric": "read-only gather probe of %s's page pattern (no arithmetic)" % of, "value": round(gbps, 1), "unit": "GB/s",
        "us_per_call": round(us, 2), "n_gpus": 1, "steps": a.steps, "warmup": a.settle, "ms_per_step": round(us / 1e3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "probe_gather_" + cfg.wl0.name, "bytes_per_call": cfg.kv_bytes,
                   "kv_pools_rotated": len(cfg.plans)},
        "roofline": {"bound": "hbm", "kernel": "pa_gather_probe_kernel" if shape == "probe_gather" else "pa_stream_probe_kernel", "achieved": round(gbps, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None},
    }, ensure_ascii=False))
    return 0


def _bench_trace(a) -> int:
    """`--workload trace:W`: W (a workload of pa_partition_shared_kernel) through the measuring build of the library
    (tests/native/libpa_decode_trace.so, -DPA_DECODE_TRACE): one wave of every workgroup leaves timestamps of the
    100 MHz wall clock at its entry, after it has requested its first steps, when its query operands are ready, when
    the first step has landed, after its last step and at its end.  Prints where a workgroup slot's time goes."""
    here = os.path.dirname(os.path.abspath(__file__))
    os.environ["PA_DECODE_LIB"] = os.path.join(here, "tests", "native", "libpa_decode_trace.so")  # before the first load
    import numpy as np
    import torch

    from triton_op_amd import _cabi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _cabi.load_library()
    lib.pa_decode_trace_read.argtypes = [C.c_void_p, C.c_ulonglong]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev)
    sh = C.c_void_p(stream.cuda_stream)
    cfg = _Config(a.workload.partition(":")[2] or "c5", dev, 1, a.partition_size, a.batch or None, output_only=a.output_only)
    if cfg.kernel != "pa_partition_shared_kernel":
        print(f"trace: only pa_partition_shared_kernel leaves timestamps; this workload launches {cfg.launch}", file=sys.stderr)
        return 2
    plan = cfg.plans[0]
    for _ in range(a.settle):
        _cabi.check(lib.pa_decode(C.byref(plan.args), sh), "pa_decode")
    torch.cuda.synchronize()
    _cabi.check(lib.pa_decode_trace_clear(), "pa_decode_trace_clear")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    _cabi.check(lib.pa_decode(C.byref(plan.args), sh), "pa_decode")
    e1.record(stream)
    torch.cuda.synchronize()
    words = np.zeros(16384 * 8, dtype=np.uint64)
    _cabi.check(lib.pa_decode_trace_read(words.ctypes.data, words.nbytes), "pa_decode_trace_read")
    t = words.reshape(-1, 8).astype(np.float64)
    xcd_of = (np.arange(len(t)) & 7)[t[:, 5] > 0]  # workgroup ids go round the eight XCDs
    t = t[t[:, 5] > 0]
    us = 0.01  # per tick
    ent, req, qry, first, last, end, steps = [t[:, i] for i in range(7)]
    where = words.reshape(-1, 8)[:, 7][words.reshape(-1, 8)[:, 5] > 0]
    rows = (where & np.uint64(0xffff)).astype(np.float64)
    hw_id, xcc_id = ((where >> np.uint64(16)) & np.uint64(0xffff)).astype(np.int64), ((where >> np.uint64(32)) & np.uint64(0xf)).astype(np.int64)
    # HW_ID: cu_id bits 8-11, sh_id bit 12, se_id bits 13-15: one number per CU of the GPU
    cu_of = xcc_id * 4096 + ((hw_id >> 8) & 0xff)
    start, span = ent.min(), (end.max() - ent.min()) * us
    slots = int(plan.launch_info().split(" workgroups per CU")[0].split()[-1]) * torch.cuda.get_device_properties(dev).multi_processor_count

    def stat(x):
        return {"mean_us": round(float(x.mean() * us), 2), "p10_us": round(float(np.percentile(x, 10) * us), 2),
                "p90_us": round(float(np.percentile(x, 90) * us), 2), "per_slot_us": round(float(x.sum() * us / slots), 1)}

    ev = np.concatenate([np.stack([ent, np.ones_like(ent)], 1), np.stack([end, -np.ones_like(end)], 1)])
    ev = ev[np.argsort(ev[:, 0], kind="stable")]
    active, when = np.cumsum(ev[:, 1]), (ev[:, 0] - start) * us
    tail_from = float(when[np.where(active >= 0.9 * slots)[0][-1]]) if (active >= 0.9 * slots).any() else 0.0
    print(json.dumps({
        "metric": "where a workgroup slot's time goes (per-workgroup timestamps, measuring build)", "workload": cfg.wl0.name,
        "launch": cfg.launch, "call_us": round(e0.elapsed_time(e1) * 1e3, 1), "live_workgroups": int(len(t)),
        "workgroup_slots": slots, "launch_span_us": round(float(span), 1),
        "entry_to_first_steps_requested": stat(req - ent), "entry_to_query_ready": stat(qry - ent),
        "entry_to_first_step_landed": stat(first - ent), "main_loop": stat(last - first),
        "per_step_in_loop": stat((last - first) / np.maximum(steps, 1)), "epilogue": stat(end - last),
        "whole_workgroup": stat(end - ent),
        "slot_time_used": round(float((end - ent).sum() * us / (slots * span)), 3),
        "last_time_nine_tenths_of_the_slots_are_busy_us": round(tail_from, 1),
        # per XCD: when its last workgroup ended, and the sum of its workgroups' times over its share of the slots
        "xcd_end_us": [round(float((end[xcd_of == x].max() - start) * us), 1) for x in range(8)],
        "xcd_busy_per_slot_us": [round(float((end - ent)[xcd_of == x].sum() * us / (slots / 8)), 1) for x in range(8)],
        "xcd_per_step_us": [round(float((((last - first) / np.maximum(steps, 1))[(xcd_of == x) & (steps >= 16)]).mean() * us), 3) for x in range(8)],
        # per CU: the mean time of a step over the CU's workgroups (16 steps or more): slowest, median and fastest CU
        "cu_per_step_us": (lambda v: {"cus": len(v), "min": round(min(v), 3), "median": round(sorted(v)[len(v) // 2], 3),
                                      "max": round(max(v), 3)})(
            [float((((last - first) / np.maximum(steps, 1))[(cu_of == c) & (steps >= 16)]).mean() * us)
             for c in np.unique(cu_of) if ((cu_of == c) & (steps >= 16)).any()]),
        "cu_busy_us": (lambda v: {"min": round(min(v), 1), "median": round(sorted(v)[len(v) // 2], 1), "max": round(max(v), 1)})(
            [float((end - ent)[cu_of == c].sum() * us / (slots / torch.cuda.get_device_properties(dev).multi_processor_count))
             for c in np.unique(cu_of)]),
        "per_step_us_by_live_rows": {str(r): round(float((((last - first) / steps)[(rows > r - 16) & (rows <= r) & (steps >= 16)]).mean() * us), 2)
                                     for r in (16, 32, 48, 64) if ((rows > r - 16) & (rows <= r) & (steps >= 16)).any()},
    }, ensure_ascii=False))
    return 0


def _bench_probe_issue(a) -> int:
    """What the instructions of the decode step cost a SIMD's issue port (pa_probe_issue): nanoseconds per
    instruction per wave with one and with three waves on every SIMD, and how far the matrix pipe runs beside the
    vector ALU."""
    import torch

    from triton_op_amd import _cabi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    lib = _load_probe_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev)
    sh = C.c_void_p(stream.cuda_stream)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.zeros(64, dtype=torch.int32, device=dev)
    iters = 2000
    names = {0: "v_fma_f32", 1: "v_mfma_f32_16x16x128_f8f6f4", 2: "16 MFMA + 128 v_fma_f32 interleaved (per iteration)",
             3: "v_exp_f32", 4: "v_cvt_pk_fp8_f32", 5: "v_permlane32_swap"}
    per_iter = {0: 128, 1: 16, 2: 1, 3: 128, 4: 128, 5: 128}
    out = {}
    for mode in range(6):
        for waves in (1, 3):
            def call():
                _cabi.check(lib.pa_probe_issue(mode, iters, cus * waves, C.c_void_p(sink.data_ptr()), sh), "probe")
            call()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            call()
            e1.record(stream)
            torch.cuda.synchronize()
            ns = e0.elapsed_time(e1) * 1e6 / (iters * per_iter[mode]) / waves
            out[f"{names[mode]}, {waves} wave(s) per SIMD"] = round(ns, 2)
    fma = out["v_fma_f32, 3 wave(s) per SIMD"]
    print(json.dumps({
        "metric": "issue cost of the decode step's instructions, ns per instruction per wave", "value": fma, "unit": "ns (v_fma_f32)",
        "n_gpus": 1, "steps": iters, "warmup": 1, "ms_per_step": 0.0, "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32 / fp8", "data": "synthetic", "config": {"workload": "probe_issue"},
        "ns_per_instruction_per_wave": out,
        "note": "a full-rate wave64 VALU instruction takes 4 shader cycles; the interleaved line is per iteration of "
                "16 MFMAs + 128 fmas: max(MFMA alone, fma alone) if the matrix pipe ran entirely beside the vector ALU, "
                "their sum if not at all"}, ensure_ascii=False))
    return 0


# ---------------------------------------------------------------------------------------------------------------
# the KV-cache write kernels
# ---------------------------------------------------------------------------------------------------------------
def _bench_kv_cache(a) -> int:
    """The step before the decode path: `kv_write` appends 64 prompts of 4096 tokens (8 kv heads, head 128, bf16
    rows) to an FP8 paged cache with per-token scales in one call; `kv_quantize` converts the c2 cache pool
    (20480 pages of 16 tokens) from bf16 to FP8 with per-token scales.  Bytes counted: rows or cache read once,
    cache and scales written once.  These kernels read and write in about equal parts, and a plain device copy
    (hipMemcpyDtoD, the same mix) is the bound they are held against: `roofline.peak` stays the published 8 TB/s,
    `roofline.frac_of_device_copy` is the fraction of the copy rate measured in the same process."""
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
    copy_gbps = _device_copy_gbps(dev, stream)
    result = {
        "metric": "KV-cache write GB/s (rows read + FP8 cache and scales written)", "value": round(achieved, 1),
        "unit": "GB/s", "us_per_call": round(us_median, 2), "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 in, fp8_e4m3fn + f32 scales out", "data": "synthetic",
        "config": {"workload": name, "kv_heads": h, "head_size": d, "block_size": bs, "bytes_per_call": nbytes},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "device_copy_GBps": round(copy_gbps, 1), "frac_of_device_copy": round(achieved / copy_gbps, 4),
                     "bound_note": "mixed read/write stream: the measured rate of a plain device copy (read + write "
                                   "bytes) is the practical bound, the published peak is a read-stream figure"},
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
    ap.add_argument("--workload", default="", help="default: c2 as the headline plus c2@256, c3, c4, c5 in `configs`")
    ap.add_argument("--partition-size", type=int, default=0, help="0 = let the tuning layer choose")
    ap.add_argument("--pools", type=int, default=3)
    ap.add_argument("--output-only", action="store_true",
                    help="call with PA_DECODE_FLAG_OUTPUT_ONLY (the caller reads only the real query rows of `output`)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="default run: the headline only")
    ap.add_argument("--power-seconds", type=float, default=0.0,
                    help="also loop the workload for this long and sample socket power and shader clock (amd-smi, rocm-smi)")
    ap.add_argument("--batch", type=int, default=0, help="override the batch size (debugging only)")
    ap.add_argument("--settle", type=int, default=SETTLE_CALLS,
                    help="untimed calls before anything is measured (profiling runs lower it)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the op shards by kv head or "
              "by sequence with no exchange); run with --gpus 1", file=sys.stderr)
        return 2
    if a.workload in ("kv_write", "kv_quantize"):
        return _bench_kv_cache(a)
    if a.workload.partition(":")[0] == "probe_gather" or a.workload.startswith("probe_stream"):
        return _bench_probe_gather(a)
    if a.workload.startswith("trace:") or a.workload == "trace":
        return _bench_trace(a)
    if a.workload == "probe_issue":
        return _bench_probe_issue(a)
    return _bench_decode(a)


if __name__ == "__main__":
    sys.exit(main())
