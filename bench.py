#!/usr/bin/env python3
"""Benchmark of the Liger hot path on one MI355X.

A step is one pass of the launch vector of one GLM-130B-shaped TP=2 layer shard over one prefill batch
(BASELINE config 2: hidden 12288, 48 of 96 heads x 128, FFN 16384 of 32768, batch 8 x seq 512, causal, fp16).
Prints one JSON line; `value` is milliseconds per layer-shard with inputs and weights resident in HBM.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

CFG2 = dict(hidden=12288, heads_global=96, d=128, ffn_global=32768, world_size=2, batch=8, seq=512)
CFG3 = dict(batch=32, cache_len=1024)


def measured_traffic(label, weight_layout=2):
    """HBM bytes per launch of `label` from the committed rocprofv3 counter runs (FETCH_SIZE + WRITE_SIZE, calibrated
    against a copy kernel of known size; see profiles/).  None when no measurement is on file for this weight layout."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            j = json.load(f)
        base = j.get("weight_layout", 1)
        suffix = "" if weight_layout == base else {0: "[in,out]", 1: "[out,in]", 2: "[tiled]"}[weight_layout]
        k = j["kernels"].get(label + suffix)
        if k is None and "gemm" not in label and "ffn" not in label and "proj" not in label:
            k = j["kernels"].get(label)    # kernels that read no weights
        return int(k["fetch_bytes"] + k["write_bytes"]) if k else None
    except (OSError, KeyError, ValueError):
        return None


def gemm_flops_cfg2():
    M, H, Hl, F = 4096, 12288, 6144, 16384
    return {"q": 2 * M * H * Hl, "k": 2 * M * H * Hl, "v": 2 * M * H * Hl, "out": 2 * M * Hl * H, "ffn1": 2 * M * H * F, "ffn2": 2 * M * F * H}


def cpu_baseline(po, sample_batch=4, sample_seq=512):
    """Times the CPU oracle (OpenMP C) on a bounded sample of the cfg2 layer: same shard shapes, M = sample rows,
    and scales linearly to M = 4096 (GEMM time is linear in M; attention at this size is < 1 % of the work)."""
    import numpy as np
    H, h, d, F = 12288, 48, 128, 16384
    Hl = h * d
    w = {}
    tid = 1
    for name, shape, std, mean in (("wq", (H, Hl), 0.02, 0), ("wk", (H, Hl), 0.02, 0), ("wv", (H, Hl), 0.02, 0), ("bq", (Hl,), 0.02, 0),
                                   ("bk", (Hl,), 0.02, 0), ("bv", (Hl,), 0.02, 0), ("wo", (Hl, H), 0.02, 0), ("ln1_g", (H,), 0.1, 1),
                                   ("ln1_b", (H,), 0.1, 0), ("w1", (H, F), 0.02, 0), ("b1", (F,), 0.02, 0), ("w2", (F, H), 0.02, 0),
                                   ("ln2_g", (H,), 0.1, 1), ("ln2_b", (H,), 0.1, 0)):
        n = int(np.prod(shape))
        w[name] = po.fill_normal(n, 0, tid, mean, std, po.F16).reshape(shape)
        tid += 1
    M = sample_batch * sample_seq
    x = po.fill_normal(M * H, 0, 99, 0.0, 1.0, po.F16).reshape(M, H)
    shape = dict(batch=sample_batch, seq=sample_seq, hidden=H, head_num=h, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=po.F16)
    t0 = time.perf_counter()
    po.encoder_forward(shape, w, x)
    dt = time.perf_counter() - t0
    scale = 4096.0 / M
    return {"value": dt * 1e3 * scale, "unit": "ms/layer-shard", "cores": po.lib().lo_num_threads(), "kind": "port",
            "sample": "cfg2 layer shard with batch %d x seq %d (M=%d of 4096 rows): %.2f s measured, scaled x%.0f" % (
                sample_batch, sample_seq, M, dt, scale)}


def kernel_only(args, capi, host, model, x, y, B, S, H, stream):
    """Launches one kernel repeatedly so that a profiler sees only it (same shapes and buffers as the bench)."""
    import ctypes as C
    import torch
    name = args.kernel_only
    if name == "copy":
        # calibration kernel of known traffic: the transpose-back kernel moving 128 MiB in and 128 MiB out
        src = torch.empty(1, 64, 8192, 128, device="cuda", dtype=torch.float16)
        capi.call("lg_fill_normal_f16", src.data_ptr(), src.numel(), 0, 5, 0.0, 1.0, None)
        dst = torch.empty_like(src)
        for _ in range(args.iters):
            capi.call("lg_transpose_f16", dst.data_ptr(), src.data_ptr(), 1, 8192, 64, 128, C.c_void_p(stream))
        capi.call("lg_stream_synchronize", stream)
        print(json.dumps({"kernel": "copy", "bytes_read": src.numel() * 2, "bytes_written": src.numel() * 2, "iters": args.iters}))
        return
    decode = args.decode or name in ("attn_decode", "kv_append") or name.endswith("(decode)")
    if decode:
        Bd, L = CFG3["batch"], CFG3["cache_len"]
        xd = torch.empty(Bd, H, device="cuda", dtype=torch.float16)
        capi.call("lg_fill_normal_f16", xd.data_ptr(), xd.numel(), 0, 98, 0.0, 1.0, None)
        yd = torch.empty_like(xd)
        desc = model.describe(Bd, 1, decode_past=L - 1)
        idx = [e["idx"] for e in desc if e["label"] == name]
        if not idx:
            sys.exit("no launch-vector entry named %r; have %s" % (name, [e["label"] for e in desc]))
        ms = host.lib.lgh_model_time_one(model.h, xd.data_ptr(), yd.data_ptr(), Bd, 1, L - 1, 0, idx[0], args.iters)
    else:
        desc = model.describe(B, S)
        idx = [e["idx"] for e in desc if e["label"] == name]
        if not idx:
            sys.exit("no launch-vector entry named %r; have %s" % (name, [e["label"] for e in desc]))
        ms = host.lib.lgh_model_time_one(model.h, x.data_ptr(), y.data_ptr(), B, S, -1, -1, idx[0], args.iters)
    print(json.dumps({"kernel": name, "iters": args.iters, "avg_ms_hip_events": round(ms, 5)}))


def bench_cfg4(capi, host, weight_layout, factors=(1, 2, 4, 8), shares=(0, 32, 64, 96, 128), repeats=3, decode_steps=8):
    """BASELINE config 4: a prefill request (batch 4 x seq 512) is decomposed by `factors` (token rows) and interleaved on two
    streams with a decode batch (32 sequences, 1024 cached positions, `decode_steps` steps: 8 steps hold the whole prefill in
    their window, 4 do not, so that a GEMM has to be split); makespan against sequential launch of the same two requests.  The decode batch is the primary request (its HBM-bound kernels open the windows), the prefill's MFMA-bound
    GEMMs are the ones split to fit them.  `shares` = compute units given to the HBM-bound side in co-running rounds (0: both
    streams on the whole chip, as the reference runs them).  Each request has its own context (buffers, workspace, cache slots)."""
    c = CFG2
    out = []
    model = host.Model(capi.F16, 64, 512, c["heads_global"], c["d"], layer_num=1, world_size=c["world_size"], ffn_inner=c["ffn_global"],
                       causal=True, fused=True, max_cache_len=1024 + 64, weight_layout=weight_layout, seed=0)
    partition = {}
    for factor in factors:
        sched = host.Scheduler(model, schedule_deep=6, contention_factor=0.8, policy=host.POLICY_RESOURCE,
                               axis=host.SPLIT_TOKEN_ROWS, seq_bucket=64, ignore_num=0, pool_count=2, ctx_batch=32)
        sched.set_factor(factor)
        sched.profile(4, 512, 512, 1, 10)
        sched.profile_decode(32, 1024, 10)
        res = {"factor": factor, "streams_verified_concurrent": sched.streams_concurrent}

        def best_of(mode):
            best = None
            for _ in range(repeats):
                sched.serve_decode(32, 1000, decode_steps)
                sched.serve(4, 512, 0)
                r = sched.run_queued(mode)
                if best is None or r["total_duration_ms"] < best["total_duration_ms"]:
                    best = r
            return {"makespan_ms": round(best["total_duration_ms"], 4), "secondary_launches": best["secondary_launches"],
                    "splits": best["splits"], "rounds": best["rounds"], "partition_rounds": best["partition_rounds"]}

        sched.set_merge_minor(False)
        res["sequential"] = best_of(host.MODE_SEQUENTIAL)
        res["interleaved"] = best_of(host.MODE_LIGER)
        sched.set_merge_minor(True)
        res["interleaved_minor_merged"] = best_of(host.MODE_LIGER)
        for share in shares:
            if share == 0:
                continue
            sched.enable_partition(share)
            meas = sched.profile_partition(4, 512, 32, 1024)
            partition[share] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in meas.items()}
            partition[share]["streams_verified_concurrent"] = sched.partition_streams_concurrent
            key = "partitioned_%d_hbm_cus" % share
            if sched.partition_factor(1, 0) <= 0:
                res[key] = {"skipped": ("a partitioned co-run does not beat back-to-back execution (gain %.3f)" % meas["gain"])
                            if sched.partition_streams_concurrent else "the partition's streams could not be made to overlap"}
                continue
            res[key] = best_of(host.MODE_LIGER)
            res[key]["speedup"] = round(res["sequential"]["makespan_ms"] / res[key]["makespan_ms"], 4)
        sched.enable_partition(0)
        print("cfg4: factor %d done" % factor, file=sys.stderr, flush=True)
        res["speedup"] = round(res["sequential"]["makespan_ms"] / res["interleaved"]["makespan_ms"], 4)
        res["speedup_minor_merged"] = round(res["sequential"]["makespan_ms"] / res["interleaved_minor_merged"]["makespan_ms"], 4)
        out.append(res)
        sched.close()   # gives its streams back: hardware queues that pile up make later streams share one
    model.close()
    return {"workload": "cfg4: prefill B4 S512 (split by token rows) || decode B32 L1024 x %d steps, one layer shard" % decode_steps,
            "partition_measurement": {"what": "MFMA-bound kernels of the prefill layer on 256 - n compute units || decode steps on n, "
                                              "against both back to back on the whole chip", "by_hbm_cus": partition},
            "results": out}


def bench_corun_one(capi, host, weight_layout, dec_bs):
    """One process of --corun-variants: the MFMA-bound kernels of a prefill layer shard (batch 4 x seq 512) next to decode steps
    (`dec_bs` sequences, 1024 cached positions) with both streams on the whole chip, and with the HBM-bound side on 64 / 128
    compute units, each against the same work back to back on the whole chip.  The pipelined GEMM's tile width follows
    LG_GEMM_TILE_WIDTH (unset: chosen by shape, 256 x 256 here; 2: 256 x 128, which leaves room for other waves on the CU)."""
    c = CFG2
    model = host.Model(capi.F16, 64, 512, c["heads_global"], c["d"], layer_num=1, world_size=c["world_size"], ffn_inner=c["ffn_global"],
                       causal=True, fused=True, max_cache_len=1024 + 64, weight_layout=weight_layout, seed=0)
    sched = host.Scheduler(model, schedule_deep=6, contention_factor=0.8, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS,
                           seq_bucket=64, ignore_num=0, pool_count=2, ctx_batch=32)
    out = {"tile_width": os.environ.get("LG_GEMM_TILE_WIDTH", "auto"), "decode_batch": dec_bs}
    w = sched.profile_contention(4, 512, dec_bs, 1024)
    w["gain"] = (w["main_ms"] + w["sub_ms"]) / w["both_ms"]
    out["whole_chip"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in w.items()}
    for share in (64, 128):
        sched.enable_partition(share)
        meas = sched.profile_partition(4, 512, dec_bs, 1024)
        out["hbm_cus_%d" % share] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in meas.items()}
    sched.enable_partition(0)
    sched.close()
    model.close()
    return out


def bench_corun_variants(weight_layout):
    """GEMM variant x CU share: one child process per (tile width, decode batch), because the library reads the tile width once."""
    import subprocess
    rows = []
    for width in ("", "2"):
        for dec_bs in (32, 16):
            env = dict(os.environ)
            env.pop("LG_GEMM_TILE_WIDTH", None)
            if width:
                env["LG_GEMM_TILE_WIDTH"] = width
            r = subprocess.run([sys.executable, os.path.abspath(__file__), "--corun-one", str(dec_bs), "--weight-layout", str(weight_layout)],
                               env=env, stdout=subprocess.PIPE, text=True, timeout=300)
            if r.returncode != 0:
                raise RuntimeError("co-run measurement (tile width %s, decode batch %d) failed with status %d" % (width or "auto", dec_bs, r.returncode))
            rows.append(json.loads(r.stdout.strip().splitlines()[-1]))
            print("corun: tile width %s, decode batch %d done" % (width or "auto", dec_bs), file=sys.stderr, flush=True)
    return {"workload": "prefill B4 S512 MFMA-bound kernels || decode steps at 1024 cached positions, one layer shard", "rows": rows}


def bench_cfg5(capi, host, weight_layout, n_requests, rates=(8.0, 16.0, 24.0, 32.0), shares=(128,), runs=1, decode_steps_ahead=2, short=False,
               packed_qkv=False):
    """BASELINE config 5: Poisson arrivals at 8 and 16 req/s -- and at 24 and 32 req/s, which is at and beyond what one request
    at a time can serve (about 28 req/s; at the reference's 4 req/s nothing ever queues on this device) -- through 4 stacked
    layer shards; prompts U[128, 1024] (rounded to 64), 32 decode
    tokens each; mean and p99 request latency with interleaving on and off.  `runs` > 1 repeats every (rate, mode) and reports
    the mean and the spread of the mean latency over the runs."""
    c = CFG2
    pool = 16
    model = host.Model(capi.F16, pool + 1, 1024, c["heads_global"], c["d"], layer_num=4, world_size=c["world_size"], ffn_inner=c["ffn_global"],
                       causal=True, fused=True, max_cache_len=1024 + 64, weight_layout=weight_layout, factor=8, seed=0, packed_qkv=packed_qkv)
    sched = host.Scheduler(model, schedule_deep=6, contention_factor=0.8, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS,
                           seq_bucket=64, ignore_num=5, pool_count=pool, ctx_batch=1)
    t0 = time.perf_counter()
    sched.profile(1, 64, 1024, 64, 5)     # from 64 tokens: the last chunk of a chunked prefill may be that short
    for past in range(128, 1024 + 64 + 1, 64):
        sched.profile_decode(1, min(past, 1024 + 63), 5)
    # batched decode steps: a few batch sizes on a coarser grid of cached positions (looked up at or below the batch)
    for bs in (2, 3, 4, 6, 8, 12, 16):
        for past in range(128, 1024 + 64 + 1, 64):
            sched.profile_decode(bs, min(past, 1024 + 63), 3)
    prof_s = time.perf_counter() - t0
    print("cfg5: profiled in %.1f s" % prof_s, file=sys.stderr, flush=True)
    # measured contention: the MFMA-bound kernels of a 512-token prefill next to batch-1 decode steps at 512 cached positions
    meas = sched.profile_contention(1, 512, 1, 512)
    table = {"mfma_main_hbm_sub": sched.contention(0, 1), "hbm_main_mfma_sub": sched.contention(1, 0)}
    part_meas = {}
    part_factor = {}
    for share in shares:
        sched.enable_partition(share)
        pm = sched.profile_partition(1, 512, 1, 512)
        part_meas[share] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in pm.items()}
        part_meas[share]["streams_verified_concurrent"] = sched.partition_streams_concurrent
        part_factor[share] = (sched.partition_factor(0, 1), sched.partition_factor(1, 0))
    sched.enable_partition(0)
    # (mode, name, measured contention, minor kernels merged, HBM-side compute units of partitioned rounds, batched decode)
    modes = [(host.MODE_SEQUENTIAL, "scheduling_off", False, False, 0, False), (host.MODE_LIGER, "scheduling_on", False, False, 0, False),
             (host.MODE_LIGER, "scheduling_on_measured_contention", True, False, 0, False),
             (host.MODE_LIGER, "scheduling_on_minor_kernels_merged", False, True, 0, False)]
    for share in shares:
        if part_factor[share][0] > 0:
            modes.append((host.MODE_LIGER, "scheduling_on_partitioned_%d_hbm_cus" % share, False, True, share, False))
    if short:   # off / on / on with batched decode steps (the default bench run)
        modes = [modes[0], modes[3]]
    modes.append((host.MODE_SEQUENTIAL, "batched_decode_without_interleaving", False, True, 0, True))
    modes.append((host.MODE_LIGER, "scheduling_on_batched_decode", False, True, 0, True))
    for share in shares:
        if part_factor[share][0] > 0:
            modes.append((host.MODE_LIGER, "scheduling_on_batched_decode_partitioned_%d_hbm_cus" % share, False, True, share, True))
    # prompts longer than 256 (512) tokens prefilled in chunks of that many, the batched decode step taking the turn between two
    # chunks (full sweep only)
    if not short:
        for chunk in (256, 512):
            modes.append((host.MODE_SEQUENTIAL, "batched_decode_chunked_prefill_%d_without_interleaving" % chunk, False, True, 0, chunk))
            modes.append((host.MODE_LIGER, "scheduling_on_batched_decode_chunked_prefill_%d" % chunk, False, True, 0, chunk))
    out = []
    for lam in rates:
        trace = host.make_poisson_trace(lam, n_requests, 1, 128, 1024, 64, 32, 0)
        row = {"lambda_req_s": lam, "requests": n_requests}
        for mode, name, measured, merge_minor, share, batched in modes:
            sched.set_contention(0, 1, table["mfma_main_hbm_sub"] if measured else -1.0)
            sched.set_contention(1, 0, table["hbm_main_mfma_sub"] if measured else -1.0)
            sched.set_merge_minor(merge_minor)
            sched.enable_batch_decode(bool(batched), decode_steps_ahead)
            sched.set_prefill_chunk(batched if batched not in (True, False) else 0)
            sched.enable_partition(share)
            if share:
                sched.set_partition_factor(0, 1, part_factor[share][0])
                sched.set_partition_factor(1, 0, part_factor[share][1])
            if share:
                sched.run_trace(trace, mode)   # untimed: the partition feedback settles on what this workload's rounds deliver
            reps = [sched.run_trace(trace, mode) for _ in range(runs)]
            r = reps[0]
            print("cfg5: lambda %.0f %s: mean %.2f ms" % (lam, name, sum(x["avg_e2e_ms"] for x in reps) / len(reps)), file=sys.stderr, flush=True)
            # latency = arrival -> completion on one clock; the reference's sum (first launch - arrival) + (start event -> stop
            # event) is kept beside it: it under-counts when a start event is held up on the device
            means = [x["avg_e2e_ms"] for x in reps]
            row[name] = {"mean_latency_ms": round(sum(means) / len(means), 3), "p99_latency_ms": round(sum(x["p99_e2e_ms"] for x in reps) / len(reps), 3),
                         "mean_latency_runs_ms": [round(v, 3) for v in means], "mean_latency_spread_ms": round(max(means) - min(means), 3),
                         "mean_cpu_plus_gpu_ms": round(r["avg_latency_ms"], 3),
                         "mean_gpu_ms": round(r["avg_gpu_ms"], 3), "mean_queue_ms": round(r["avg_queue_ms"], 3),
                         "throughput_req_s": round(r["throughput"], 3), "records": r["records"],
                         "secondary_launches": r["secondary_launches"], "splits": r["splits"], "profile_misses": r["profile_misses"],
                         "partition_rounds": r["partition_rounds"],
                         "partition_feedback": sched.partition_feedback_state() if share else None,
                         "batched_steps": r["batched_steps"], "chunking": sched.chunk_counters() if batched not in (True, False) else None,
                         "rows_per_batched_step": round(r["batched_rows"] / r["batched_steps"], 2) if r["batched_steps"] else None}
        out.append(row)
    sched.enable_partition(0)
    sched.set_prefill_chunk(0)
    sched.enable_batch_decode(False)
    concurrent = sched.streams_concurrent
    sched.close()
    model.close()
    return {"workload": "cfg5: 4 layer shards, Poisson arrivals, prompts U[128,1024] rounded to 64, 32 decode tokens; Q, K and V weights "
                        + ("packed as one [H, 3 Hl] matrix (the layout of GLM checkpoints)" if packed_qkv else "stored separately"),
            "profile_seconds": round(prof_s, 1),
            "streams_verified_concurrent": concurrent,
            "contention_measurement": {k: (round(v, 4) if isinstance(v, float) else v) for k, v in meas.items()},
            "contention_table": {k: round(v, 4) for k, v in table.items()},
            "partition_measurement": part_meas, "results": out}


def measured_ceilings(capi, iters=3000, read_mib=2048, traffic_variants=False):
    """What this device sustains, measured now with the library's two probe kernels (lg_probe_mfma_f16, lg_probe_read):
    a register-only loop of the GEMM's matrix instruction on its wave tile with operands distributed like the bench's data
    (N(0,1) x N(0,0.02) products are what the layer's GEMMs multiply; both operand sets here are N(0,1) halves, which toggle
    at least as many bits) and with all-zero operands, and a single-pass read of a buffer eight times the memory-side cache."""
    import ctypes as C
    import torch
    n = 1 << 20
    ops = torch.empty(n, device="cuda", dtype=torch.float16)
    scratch = torch.zeros(64, device="cuda", dtype=torch.float32)
    out = {}
    ms, tf, ghz = C.c_float(), C.c_float(), C.c_float()
    for name in ("random_operands", "zero_operands"):
        if name == "random_operands":
            capi.call("lg_fill_normal_f16", ops.data_ptr(), n, 0, 77, 0.0, 1.0, None)
        else:
            ops.zero_()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            capi.call("lg_probe_mfma_f16", ops.data_ptr(), n, scratch.data_ptr(), 256, iters, C.byref(ms), C.byref(tf), C.byref(ghz), None)
            if best is None or tf.value > best[0]:
                best = (tf.value, ghz.value, ms.value)
        out["mfma_f16_" + name] = {"TFLOPs": round(best[0], 1), "shader_clock_GHz": round(best[1], 3), "kernel_ms": round(best[2], 3),
                                   "frac_of_published_peak": round(best[0] / PEAK_FP16_TFLOPS, 4)}
    # the same instruction stream with the operands travelling L2 -> LDS -> registers at the pipelined GEMM's rate (random data)
    capi.call("lg_fill_normal_f16", ops.data_ptr(), n, 0, 77, 0.0, 1.0, None)
    torch.cuda.synchronize()
    def streamed(loads, reads):
        best = None
        for _ in range(3):
            capi.call("lg_probe_mfma_stream_f16", ops.data_ptr(), n, scratch.data_ptr(), 256, iters // 2, loads, reads, C.byref(ms), C.byref(tf), C.byref(ghz), None)
            if best is None or tf.value > best[0]:
                best = (tf.value, ghz.value, ms.value)
        return {"TFLOPs": round(best[0], 1), "shader_clock_GHz": round(best[1], 3), "kernel_ms": round(best[2], 3),
                "frac_of_published_peak": round(best[0] / PEAK_FP16_TFLOPS, 4)}
    out["mfma_f16_random_operands_streamed_through_lds"] = streamed(8, 12)
    if traffic_variants:
        # what half or none of either kind of operand traffic would leave (per wave and k-tile: L2 -> LDS loads of 1 KiB, LDS -> register
        # reads of 1 KiB per k-step)
        out["mfma_f16_streamed_traffic_variants"] = {"loads_%d_reads_%d" % (l, r): streamed(l, r)["TFLOPs"]
                                                     for l, r in ((8, 12), (4, 12), (0, 12), (8, 6), (8, 0), (4, 6), (0, 0))}
    del ops
    buf = torch.empty(read_mib << 20, device="cuda", dtype=torch.uint8)
    capi.call("lg_fill_normal_f16", buf.data_ptr(), buf.numel() // 2, 0, 78, 0.0, 1.0, None)
    torch.cuda.synchronize()
    gb = C.c_float()
    for nt in (0, 1):
        capi.call("lg_probe_read", buf.data_ptr(), buf.numel(), scratch.data_ptr(), 5, nt, C.byref(ms), C.byref(gb), None)
        out["read_%d_MiB%s" % (read_mib, "_nontemporal" if nt else "")] = {"GBps": round(gb.value, 1), "ms_per_pass": round(ms.value, 4),
                                                                          "frac_of_published_peak": round(gb.value / PEAK_HBM_GBS, 4)}
    del buf
    torch.cuda.empty_cache()
    out["what"] = ("lg_probe_mfma_f16: 1024 blocks x 8 waves x %d rounds of 32 v_mfma_f32_16x16x32_f16, operands in registers; "
                   "lg_probe_mfma_stream_f16: %d rounds of 64, per round 8 KiB per wave L2 -> LDS and 24 KiB LDS -> registers (the pipelined GEMM's "
                   "operand traffic, nothing else of it); lg_probe_read: one pass over %d MiB per launch, 16-byte loads" % (iters, iters // 2, read_mib))
    return out


def bench_weight_relay(capi, host, weight_layout):
    """One-off cost of taking the cfg2 layer shard's six weight matrices over from plain [in, out] device arrays (the layout the
    reference's (N,N) GEMM call implies) into the layer's storage layout: lgh_model_load_param, one kernel per matrix."""
    import torch
    c = CFG2
    model = host.Model(capi.F16, 1, 64, c["heads_global"], c["d"], layer_num=1, world_size=c["world_size"], ffn_inner=c["ffn_global"],
                       causal=True, fused=True, weight_layout=weight_layout, seed=0)
    srcs = {}
    for name, i in model.param_info().items():
        if i["rows"] > 1:
            t = torch.empty(i["rows"] * i["cols"], device="cuda", dtype=torch.float16)
            capi.call("lg_fill_normal_f16", t.data_ptr(), t.numel(), 0, 5, 0.0, 0.02, None)
            srcs[name] = t
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        for name, t in srcs.items():
            model.load_param(name, t.data_ptr(), 0)
        capi.call("lg_stream_synchronize", model.stream)
        dt = (time.perf_counter() - t0) * 1e3
        best = dt if best is None else min(best, dt)
    nbytes = sum(t.numel() * 2 for t in srcs.values())
    model.close()
    del srcs
    torch.cuda.empty_cache()
    return {"what": "lgh_model_load_param on the %d weight matrices of one cfg2 layer shard, sources [in, out]" % 6, "ms": round(best, 3),
            "weight_MB": round(nbytes / 1e6, 1), "read_plus_write_GBps": round(2 * nbytes / (best * 1e-3) / 1e9, 1)}


def bench_fp32(capi, host):
    """The fp32 instantiation (the reference builds every layer for float as well, context.h:49-55): BASELINE config 1 (hidden 256,
    4 heads x 64, FFN 1024, pre-LayerNorm, batch 2 x seq 32) as one launch vector, and the fp32 GEMM on the matrix cores at a
    size that fills the chip, against the published fp32 matrix peak."""
    import ctypes as C
    import torch
    m = host.Model(capi.F32, 2, 32, 4, 64, layer_num=1, ffn_inner=1024, norm_mode=host.PRE_LN_RESID, causal=False, fused=False, seed=0)
    x = torch.empty(64, 256, device="cuda", dtype=torch.float32)
    capi.call("lg_fill_normal_f32", x.data_ptr(), x.numel(), 0, 99, 0.0, 1.0, None)
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    for _ in range(5):
        m.run(x.data_ptr(), y.data_ptr(), 2, 32, None, m.stream)
    capi.call("lg_stream_synchronize", m.stream)
    t0 = time.perf_counter()
    for _ in range(200):
        m.run(x.data_ptr(), y.data_ptr(), 2, 32, None, m.stream)
    capi.call("lg_stream_synchronize", m.stream)
    cfg1_ms = (time.perf_counter() - t0) * 1e3 / 200
    launches = m.kernels_per_layer()
    m.close()
    out = {"cfg1_layer_ms": round(cfg1_ms, 4), "cfg1_launches": launches}
    n = 4096
    a = torch.empty(n, n, device="cuda", dtype=torch.float32)
    b = torch.empty(n, n, device="cuda", dtype=torch.float32)
    c = torch.empty(n, n, device="cuda", dtype=torch.float32)
    capi.call("lg_fill_normal_f32", a.data_ptr(), a.numel(), 0, 5, 0.0, 0.02, None)
    capi.call("lg_fill_normal_f32", b.data_ptr(), b.numel(), 0, 6, 0.0, 1.0, None)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for transa, name in ((0, "[in, out]"), (1, "[out, in]")):
        for _ in range(2):
            capi.call("lg_gemm_f32", transa, 0, n, n, n, a.data_ptr(), n, b.data_ptr(), n, c.data_ptr(), n, None)
        e0.record()
        for _ in range(10):
            capi.call("lg_gemm_f32", transa, 0, n, n, n, a.data_ptr(), n, b.data_ptr(), n, c.data_ptr(), n, None)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 10
        out["gemm_4096_cubed_weights_" + name] = {"ms": round(ms, 4), "TFLOPs": round(2 * n ** 3 / ms / 1e9, 1),
                                                  "frac_of_fp32_matrix_peak": round(2 * n ** 3 / ms / 1e9 / 157.3, 4)}
    return out


def derived_peaks(info):
    """Roofline denominators re-derived from the device properties: matrix peak = CUs x 4096 fp16 flop per clock and CU x
    engine clock; memory peak = bus width x reported memory clock x 4 transfers per pin and clock (the runtime reports 2.0 GHz
    for HBM3E pins that run at 8 Gb/s; with 2 transfers per clock the "peak" would be 4.1 TB/s, below the 5.9 TB/s the
    decode attention kernel measures, so the reported clock is a quarter of the pin rate)."""
    flops = info["cu_count"] * 4096 * info["clock_khz"] * 1e3 / 1e12
    gbs = info["bus_width_bits"] / 8 * info["mem_clock_khz"] * 1e3 * 4 / 1e9
    return {"fp16_mfma_TFLOPs": round(flops, 1), "hbm_GBps": round(gbs, 1),
            "formula": "%d CUs x 4096 flop/clk x %.3f GHz; %d bit x %.3f GHz x 4" % (info["cu_count"], info["clock_khz"] / 1e6,
                                                                                     info["bus_width_bits"], info["mem_clock_khz"] / 1e6)}


def time_layer(capi, host, weight_layout, fused, steps, warmup, packed_qkv=False):
    """Times the cfg2 prefill layer shard and the cfg3 decode step in one weight layout; returns (model, x, y, results)."""
    import torch
    c = CFG2
    B, S, H = c["batch"], c["seq"], c["hidden"]
    M = B * S
    model = host.Model(capi.F16, 32, S, c["heads_global"], c["d"], layer_num=1, world_size=c["world_size"], ffn_inner=c["ffn_global"],
                       norm_mode=host.POST_NORESID, causal=True, fused=fused, max_cache_len=CFG3["cache_len"] + 32 if fused else 0,
                       weight_layout=weight_layout, seed=0, packed_qkv=packed_qkv)
    x = torch.empty(M, H, device="cuda", dtype=torch.float16)
    capi.call("lg_fill_normal_f16", x.data_ptr(), x.numel(), 0, 99, 0.0, 1.0, None)
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    stream = model.stream
    for _ in range(warmup):
        model.run(x.data_ptr(), y.data_ptr(), B, S, None, stream)
    capi.call("lg_stream_synchronize", stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        model.run(x.data_ptr(), y.data_ptr(), B, S, None, stream)
    capi.call("lg_stream_synchronize", stream)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps
    # per-kernel durations: HIP events on the launch stream, 2 warm-ups + 20 launches, min of 3 (the reference's profiler protocol)
    desc = model.describe(B, S)
    times = model.time_kernels(x.data_ptr(), y.data_ptr(), B, S)
    kernels = [{"idx": e["idx"], "kernel": e["label"], "class": e["class"], "ms": round(t, 4)} for e, t in zip(desc, times)]
    decode = None
    if fused:
        Bd, L = CFG3["batch"], CFG3["cache_len"]
        xd = torch.empty(Bd, H, device="cuda", dtype=torch.float16)
        capi.call("lg_fill_normal_f16", xd.data_ptr(), xd.numel(), 0, 98, 0.0, 1.0, None)
        yd = torch.empty_like(xd)
        torch.cuda.synchronize()
        ddesc = model.describe(Bd, 1, decode_past=L - 1)
        dtimes = model.time_kernels(xd.data_ptr(), yd.data_ptr(), Bd, 1, decode_past=L - 1, cache_slot=0)
        # the step as a whole, timed like the prefill step: every step streams the whole weight shard and KV cache (2.2 GB), so
        # nothing is served from what an earlier launch of the same kernel left in the 256 MB memory-side cache, which the
        # per-kernel loops above allow for the smaller weights
        for _ in range(max(warmup, 3)):
            model.run_decode(xd.data_ptr(), yd.data_ptr(), Bd, L - 1, 0, None, stream)
        capi.call("lg_stream_synchronize", stream)
        torch.cuda.synchronize()
        dsteps = max(steps, 20)
        t0 = time.perf_counter()
        for _ in range(dsteps):
            model.run_decode(xd.data_ptr(), yd.data_ptr(), Bd, L - 1, 0, None, stream)
        capi.call("lg_stream_synchronize", stream)
        torch.cuda.synchronize()
        step_ms = (time.perf_counter() - t0) * 1e3 / dsteps
        # and every entry where it runs inside the step (an event between every two entries; run time + the gap before it)
        in_step = model.time_step(xd.data_ptr(), yd.data_ptr(), Bd, 1, decode_past=L - 1, cache_slot=0, reps=20)
        decode = {"kernels": [{"idx": e["idx"], "kernel": e["label"], "ms": round(t, 4), "in_step_ms": round(u, 4)}
                              for e, t, u in zip(ddesc, dtimes, in_step)],
                  "ms_per_layer_shard": round(step_ms, 4), "sum_kernel_ms": round(sum(dtimes), 4)}
    return model, x, y, {"ms_per_step": ms_per_step, "kernels": kernels, "sum_kernel_ms": sum(times), "decode": decode}


def timed_only(capi, host, args, fused):
    """The bench's timed region and nothing else: `warmup` untimed and `steps` timed launches of the cfg2 prefill layer shard (or,
    with --decode, of the cfg3 decode step), the same calls `time_layer` times.  Every launch-vector entry is one kernel dispatch,
    so a kernel trace of this run holds (warmup + steps) x len(entries) dispatches after the set-up fills, in launch order."""
    import torch
    c = CFG2
    B, S, H = c["batch"], c["seq"], c["hidden"]
    model = host.Model(capi.F16, 32, S, c["heads_global"], c["d"], layer_num=1, world_size=c["world_size"], ffn_inner=c["ffn_global"],
                       norm_mode=host.POST_NORESID, causal=True, fused=fused, max_cache_len=CFG3["cache_len"] + 32 if fused else 0,
                       weight_layout=args.weight_layout, seed=0, packed_qkv=fused and not args.separate_qkv)
    stream = model.stream
    if args.decode:
        Bd, L = CFG3["batch"], CFG3["cache_len"]
        x = torch.empty(Bd, H, device="cuda", dtype=torch.float16)
        desc = model.describe(Bd, 1, decode_past=L - 1)
        step = lambda: model.run_decode(x.data_ptr(), y.data_ptr(), Bd, L - 1, 0, None, stream)
    else:
        x = torch.empty(B * S, H, device="cuda", dtype=torch.float16)
        desc = model.describe(B, S)
        step = lambda: model.run(x.data_ptr(), y.data_ptr(), B, S, None, stream)
    capi.call("lg_fill_normal_f16", x.data_ptr(), x.numel(), 0, 99, 0.0, 1.0, None)
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    capi.call("lg_stream_synchronize", stream)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    capi.call("lg_stream_synchronize", stream)
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    return {"timed_only": "cfg3 decode step" if args.decode else "cfg2 prefill layer shard", "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 4), "entries": [e["label"] for e in desc], "weight_layout": args.weight_layout}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--unfused", action="store_true", help="time the reference-shaped 14-entry assembly instead")
    ap.add_argument("--no-scheduler", action="store_true", help="skip the short config-4 / config-5 scheduler records")
    ap.add_argument("--cfg4", action="store_true", help="run the full decomposition sweep (BASELINE config 4) instead of the short record")
    ap.add_argument("--cfg5", action="store_true", help="run the full mixed request trace (BASELINE config 5; minutes) instead of the short record")
    ap.add_argument("--cfg5-requests", type=int, default=60)
    ap.add_argument("--cfg5-runs", type=int, default=3)
    ap.add_argument("--separate-qkv", "--cfg5-separate-qkv", dest="separate_qkv", action="store_true",
                    help="three separate Q / K / V weights (9 launch-vector entries per fused layer) instead of the packed [H, 3 Hl] one of GLM "
                         "checkpoints (7 entries: the three projections are one entry, for which the library picks the launches that fill the "
                         "rounds of workgroups best: the cfg2 batch 1.3 %% faster, prompts of 384-768 tokens 7-13 %%)")
    ap.add_argument("--corun-variants", action="store_true",
                    help="GEMM tile width (chosen by shape / 256 x 128) x CU share: prefill MFMA kernels next to decode steps, one JSON line")
    ap.add_argument("--corun-one", type=int, default=0, help=argparse.SUPPRESS)
    ap.add_argument("--kernel-only", default=None,
                    help="launch only the named launch-vector entry (e.g. 'ffn1+bias+gelu', 'attn_decode', 'layer_norm') or "
                         "'copy' (a plain 128 MiB read + 128 MiB write kernel) --iters times; for rocprofv3 runs.  "
                         "'mfma_ceiling' / 'read_ceiling' run the library's probe kernels and print what the device sustains")
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--timed-only", action="store_true",
                    help="run nothing but the warm-up steps and the timed steps of the prefill layer shard (with --decode: of the decode "
                         "step) and print their launch vector; for rocprofv3 runs whose rows are then the timed dispatches alone")
    ap.add_argument("--decode", action="store_true",
                    help="with --kernel-only: take the entry from the decode step's launch vector (batch 32, 1024 cached positions); "
                         "needed for the entries whose name the prefill vector has too (ffn1+bias+gelu, ffn2, layer_norm)")
    ap.add_argument("--weight-layout", type=int, default=2, choices=[0, 1, 2],
                    help="0: weights stored [in, out] (the reference's cuBLAS (N,N) layout); 1: stored [out, in]; "
                         "2 (default): [out, in] in 16 x 32 fragment blocks, the layout a layer re-lays weights into when it takes them over "
                         "(lgh_model_load_param -> lg_weight_tile_f16; cost in the weight_relay_at_load record)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs one GPU's tensor-parallel shard on one GPU; --gpus %d is not supported "
              "(the all-reduce between GPUs is out of scope)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    if args.corun_variants:
        print(json.dumps(bench_corun_variants(args.weight_layout)), flush=True)
        return
    import torch
    liger = importlib.import_module("24ppopp-liger_amd")
    host = importlib.import_module("24ppopp-liger_amd.host")
    capi = liger.capi
    torch.cuda.set_device(0)
    info = capi.device_info()
    c = CFG2
    B, S, H = c["batch"], c["seq"], c["hidden"]
    M = B * S
    fused = not args.unfused

    if args.corun_one:
        print(json.dumps(bench_corun_one(capi, host, args.weight_layout, args.corun_one)), flush=True)
        return
    if args.kernel_only in ("mfma_ceiling", "read_ceiling"):
        m = measured_ceilings(capi, traffic_variants=args.kernel_only == "mfma_ceiling")
        print(json.dumps({"kernel": args.kernel_only, **{k: v for k, v in m.items() if k == "what" or k.startswith("mfma" if args.kernel_only == "mfma_ceiling" else "read")}}))
        return
    if args.timed_only:
        print(json.dumps(timed_only(capi, host, args, fused)))
        return
    if args.kernel_only:
        model = host.Model(capi.F16, 32, S, c["heads_global"], c["d"], layer_num=1, world_size=c["world_size"], ffn_inner=c["ffn_global"],
                           norm_mode=host.POST_NORESID, causal=True, fused=fused, max_cache_len=CFG3["cache_len"] + 32 if fused else 0,
                           weight_layout=args.weight_layout, seed=0, packed_qkv=fused and not args.separate_qkv)
        x = torch.empty(M, H, device="cuda", dtype=torch.float16)
        capi.call("lg_fill_normal_f16", x.data_ptr(), x.numel(), 0, 99, 0.0, 1.0, None)
        y = torch.empty_like(x)
        torch.cuda.synchronize()
        kernel_only(args, capi, host, model, x, y, B, S, H, model.stream)
        return

    packed = fused and not args.separate_qkv
    model, x, y, res = time_layer(capi, host, args.weight_layout, fused, args.steps, args.warmup, packed_qkv=packed)
    ms_per_step, kernels = res["ms_per_step"], res["kernels"]
    fl = gemm_flops_cfg2()
    label_flops = {"q_gemm": fl["q"], "k_gemm": fl["k"], "v_gemm": fl["v"], "out_proj": fl["out"], "ffn1": fl["ffn1"], "ffn2": fl["ffn2"],
                   "q_gemm+bias+heads": fl["q"], "k_gemm+bias+heads": fl["k"], "v_gemm+bias+heads": fl["v"], "ffn1+bias+gelu": fl["ffn1"],
                   "qkv_gemm+bias+heads": fl["q"] + fl["k"] + fl["v"]}
    gemm_ms = 0.0
    gemm_fl = 0.0
    for k in kernels:
        if k["kernel"] in label_flops:
            k["tflops"] = round(label_flops[k["kernel"]] / (k["ms"] * 1e-3) / 1e12, 1)
            k["traffic"] = measured_traffic(k["kernel"], args.weight_layout)
            gemm_ms += k["ms"]
            gemm_fl += label_flops[k["kernel"]]
    # dominant kernel = FFN-1 (with FFN-2 the largest share of the step's flops; always the same one, so that the counter
    # traffic on file belongs to it)
    dom = [k for k in kernels if k["kernel"] in ("ffn1+bias+gelu", "ffn1")][0]
    dom_fl = label_flops[dom["kernel"]]
    achieved = dom_fl / (dom["ms"] * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": dom["kernel"], "achieved": round(achieved, 1), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_FP16_TFLOPS, 4), "traffic": measured_traffic(dom["kernel"], args.weight_layout),
                "all_gemms_tflops": round(gemm_fl / (gemm_ms * 1e-3) / 1e12, 1),
                "all_gemms_frac": round(gemm_fl / (gemm_ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 4)}
    ln = [k for k in kernels if k["kernel"] == "layer_norm"]
    ln_gbs = (2 * M * H * 2) / (min(k["ms"] for k in ln) * 1e-3) / 1e9 if ln else None

    # decode step of the same shard (BASELINE config 3): batch 32, one token, 1024 cached positions
    decode = None
    if res["decode"]:
        Bd, L = CFG3["batch"], CFG3["cache_len"]
        dk = res["decode"]["kernels"]
        step_ms = res["decode"]["ms_per_layer_shard"]
        attn = [k for k in dk if k["kernel"] == "attn_decode"][0]
        kv_bytes = 2 * Bd * 48 * L * 128 * 2
        w_bytes = (3 * H * 6144 + 6144 * H + 2 * H * 16384) * 2
        is_gemm = lambda k: "gemm" in k["kernel"] or "proj" in k["kernel"] or "ffn" in k["kernel"]
        gemm_dec_ms = sum(k["ms"] for k in dk if is_gemm(k))
        gemm_in_step_ms = sum(k["in_step_ms"] for k in dk if is_gemm(k))
        decode = {"workload": "cfg3: batch 32, 1 new token, 1024 cached positions", "ms_per_layer_shard": step_ms,
                  "sum_kernel_ms": res["decode"]["sum_kernel_ms"],
                  "tokens_per_s": round(Bd / (step_ms * 1e-3), 1), "kernels": dk,
                  "hbm_floor_ms": round((w_bytes + kv_bytes) / (PEAK_HBM_GBS * 1e9) * 1e3, 4),
                  "roofline_attn_decode": {"bound": "hbm", "achieved": round(kv_bytes / (attn["ms"] * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                                           "unit": "GB/s", "frac": round(kv_bytes / (attn["ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                           "in_step_frac": round(kv_bytes / (attn["in_step_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                           "traffic": measured_traffic("attn_decode")},
                  "skinny_gemms": {"ms": round(gemm_dec_ms, 4), "weight_GBps": round(w_bytes / (gemm_dec_ms * 1e-3) / 1e9, 1),
                                   "frac": round(w_bytes / (gemm_dec_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                   # the same GEMMs timed where they run inside whole steps (launch gaps included, nothing
                                   # re-read from the memory-side cache by a repeated launch)
                                   "in_step_ms": round(gemm_in_step_ms, 4),
                                   "in_step_frac": round(w_bytes / (gemm_in_step_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}}

    out = {
        "metric": "ms/layer-shard prefill (GLM-130B TP=2 shard, B8 S512, causal, fp16)",
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "cfg2 prefill: hidden 12288, 48/96 heads x 128, FFN 16384/32768, batch 8 x seq 512, causal; "
                               + (("fused assembly, Q / K / V as one packed weight (7 launch-vector entries/layer)" if packed else
                                   "fused assembly, separate Q / K / V weights (9 launch-vector entries/layer)") if fused
                                  else "reference-shaped assembly (14 launches/layer)")
                               + "; weights stored " + {0: "[in, out]", 1: "[out, in]", 2: "[out, in] in 16 x 32 fragment blocks"}[args.weight_layout]},
        "tokens_per_s": round(M / (ms_per_step * 1e-3), 1),
        "roofline": roofline,
        "layer_norm_GBps": round(ln_gbs, 1) if ln_gbs else None,
        "kernels": kernels,
        "sum_kernel_ms": round(res["sum_kernel_ms"], 4),
        "decode": decode,
        "device": info,
        "peaks": {"fp16_mfma_TFLOPs": PEAK_FP16_TFLOPS, "hbm_GBps": PEAK_HBM_GBS, "source": "published MI355X figures (the roofline denominators)",
                  "derived_from_device_properties": derived_peaks(info)},
    }
    del model, x, y
    torch.cuda.empty_cache()
    # what a kernel that does nothing else sustains on this device, measured in this run: the power-limited matrix ceiling on
    # data like the bench's, and the memory read ceiling
    out["peaks"]["measured"] = measured_ceilings(capi)
    mc = out["peaks"]["measured"]["mfma_f16_random_operands"]["TFLOPs"]
    out["roofline"]["frac_of_measured_mfma_ceiling"] = round(out["roofline"]["achieved"] / mc, 4) if mc > 0 else None
    ms_ = out["peaks"]["measured"]["mfma_f16_random_operands_streamed_through_lds"]["TFLOPs"]
    out["roofline"]["frac_of_measured_mfma_ceiling_with_operand_traffic"] = round(out["roofline"]["achieved"] / ms_, 4) if ms_ > 0 else None
    # the same layer (prefill and decode step) in the other weight layouts: 0 = [in, out], the layout the reference's (N,N)
    # cuBLAS call implies; 1 = [out, in]; 2 = [out, in] re-laid into 16 x 32 fragment blocks
    names = {0: ("reference_layout", "[in, out]"), 1: ("out_in_layout", "[out, in]"), 2: ("tiled_layout", "[out, in] in 16 x 32 fragment blocks")}
    for other in (0, 1, 2):
        if other == args.weight_layout:
            continue
        m2, x2, y2, r2 = time_layer(capi, host, other, fused, max(5, args.steps // 2), 2, packed_qkv=packed)
        out[names[other][0]] = {
            "weights": names[other][1], "ms_per_layer_shard_prefill": round(r2["ms_per_step"], 4),
            "ms_per_layer_shard_decode": r2["decode"]["ms_per_layer_shard"] if r2["decode"] else None,
            "prefill_gemm_tflops": {k["kernel"]: round(label_flops[k["kernel"]] / (k["ms"] * 1e-3) / 1e12, 1) for k in r2["kernels"] if k["kernel"] in label_flops},
            "decode_kernels_ms": {k["kernel"]: k["ms"] for k in r2["decode"]["kernels"]} if r2["decode"] else None,
            "decode_kernels_in_step_ms": {k["kernel"]: k["in_step_ms"] for k in r2["decode"]["kernels"]} if r2["decode"] else None}
        del m2, x2, y2
        torch.cuda.empty_cache()
    if fused:
        # the reference-shaped assembly (bert.h:59-79: 14 launches per layer, three batched-GEMM / softmax / transpose kernels
        # instead of the fused attention, separate bias kernels) on the same shard and weights layout: what a maintainer who binds
        # the C ABI entry by entry gets before adopting the fused entries
        m3, x3, y3, r3 = time_layer(capi, host, args.weight_layout, False, max(5, args.steps // 2), 2)
        out["reference_assembly"] = {"launches_per_layer": len(r3["kernels"]), "ms_per_layer_shard_prefill": round(r3["ms_per_step"], 4),
                                     "kernels_ms": {"%d:%s" % (k["idx"], k["kernel"]): k["ms"] for k in r3["kernels"]}}
        del m3, x3, y3
        torch.cuda.empty_cache()
    if fused:
        # the same shard with the other storage of the Q, K and V projections: packed as ONE [H, 3 Hl] weight (the layout of GLM
        # checkpoints) they are one launch-vector entry, for which the library picks the launches that fill the rounds of workgroups
        # best (at cfg2: Q and K as one launch of three full rounds, V as a full round and a round of 128-wide tiles); stored
        # separately they are three entries of two rounds of 192-wide tiles each
        m4, x4, y4, r4 = time_layer(capi, host, args.weight_layout, True, max(5, args.steps // 2), 2, packed_qkv=not packed)
        out["separate_qkv" if packed else "packed_qkv"] = {
            "launches_per_layer": len(r4["kernels"]), "ms_per_layer_shard_prefill": round(r4["ms_per_step"], 4),
            "ms_per_layer_shard_decode": r4["decode"]["ms_per_layer_shard"] if r4["decode"] else None,
            "kernels_ms": {"%d:%s" % (k["idx"], k["kernel"]): k["ms"] for k in r4["kernels"]}}
        del m4, x4, y4
        torch.cuda.empty_cache()
    out["weight_relay_at_load"] = bench_weight_relay(capi, host, args.weight_layout)
    out["fp32"] = bench_fp32(capi, host)
    if not args.no_cpu_baseline:
        from oracle import pyoracle as po
        out["cpu_baseline"] = cpu_baseline(po)
    if fused and not args.no_scheduler:
        # scheduler records: the decomposition sweep against a decode batch (config 4) and the mixed trace (config 5); short
        # versions by default so that the whole run stays within minutes, the full sweeps with --cfg4 / --cfg5
        if args.cfg4:
            out["cfg4"] = bench_cfg4(capi, host, args.weight_layout)
            out["cfg4_split_forced"] = bench_cfg4(capi, host, args.weight_layout, decode_steps=4)
        else:
            out["cfg4"] = bench_cfg4(capi, host, args.weight_layout, factors=(1, 8), shares=(0, 128), repeats=3)
            out["cfg4_split_forced"] = bench_cfg4(capi, host, args.weight_layout, factors=(8,), shares=(0, 128), repeats=3, decode_steps=4)
        torch.cuda.empty_cache()
        if args.cfg5:
            out["cfg5"] = bench_cfg5(capi, host, args.weight_layout, args.cfg5_requests, runs=args.cfg5_runs, packed_qkv=not args.separate_qkv)
        else:
            out["cfg5"] = bench_cfg5(capi, host, args.weight_layout, 40, rates=(16.0, 32.0), shares=(128,), runs=3, short=True,
                                     packed_qkv=not args.separate_qkv)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
