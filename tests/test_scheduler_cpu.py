"""Unit tests of the launch-vector runtime (layer assembly, Sample, Scheduler, profile JSON, report) on the CPU.

The runtime is the shipped C++ code; only the device library underneath is replaced by tests/fake_backend, which
records every launch with virtual timestamps.  Expected launch sequences are derived by hand from the policy the
reference implements (src/schedule.h:221-278, src/init.h:121-259); the fake's cost model is
    gemm: 0.003 + 2*m*n*k / 1e9 ms      memory kernels: 0.003 + bytes / 1e6 ms      host launch cost 0.002 ms.
"""
import json
import os

import numpy as np
import pytest

from tests.fake_util import Fake

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture()
def fake():
    f = Fake()
    f.set_rates(1.0e9, 1.0e6, 0.002)
    f.reset()
    yield f
    f.close()


def small_model(host, fused=True, factor=4, layers=1, max_batch=4, cache=128):
    return host.Model(1, max_batch, 64, 4, 64, layer_num=layers, ffn_inner=512, causal=True, fused=fused,
                      max_cache_len=cache if fused else 0, factor=factor, seed=0)


def fake_trace_of(fake, model, batch, seq):
    """Launch records of one plain run of the model on the virtual-time backend."""
    fake.reset()
    model.run(0x10000, 0x20000000, batch, seq)   # the backend never dereferences "device" pointers
    return fake.trace()


def test_launch_vector_shapes_and_order(fake):
    host = fake.host
    m = small_model(host, fused=False, cache=0)
    d = m.describe(2, 32)
    assert [e["label"] for e in d] == ["q_gemm", "k_gemm", "v_gemm", "qkv_bias_transpose", "qk_gemm", "softmax", "pv_gemm",
                                       "transpose_back", "out_proj", "layer_norm", "ffn1", "bias+gelu", "ffn2", "layer_norm"]
    # only the six weight GEMMs are type GEMM (decomposable), as in the reference (bert_layer.h:145-163 tags the batched ones COMPUTATION)
    assert [e["type"] for e in d].count("GEMM") == 6
    assert m.kernels_per_layer() == 14
    mf = small_model(host, fused=True)
    assert mf.kernels_per_layer() == 9 and mf.kernels_per_layer(decode=True) == 7   # one grouped Q/K/V launch whose epilogues append the K/V rows
    assert [e["label"] for e in mf.describe(2, 1, decode_past=10)][:3] == ["qkv_gemm(decode)", "attn_decode", "out_proj(decode)"]
    assert all(e["class"] == "HBM_BOUND" for e in mf.describe(2, 1, decode_past=10))
    mg = host.Model(1, 2, 32, 4, 64, ffn_inner=512, fused=True, ffn_act=host.FFN_GEGLU)
    # fused GeGLU: the product is formed in FFN-1's epilogue; the reference-shaped assembly keeps the separate kernel
    assert [e["label"] for e in mg.describe(2, 32)][-3:] == ["ffn1+bias+geglu", "ffn2", "layer_norm"]
    gate_up = [e for e in fake_trace_of(fake, mg, 2, 32) if e["name"].startswith("gemm")][-2]
    assert (gate_up["m"], gate_up["n"], gate_up["k"]) == (1024, 64, 256)      # FFN-1 produces 2 F columns
    assert mg.param_info()["layer0.w1"]["interleave16"] == 1 and mg.param_info()["layer0.b1"]["interleave16"] == 1
    mu = host.Model(0, 2, 32, 4, 64, ffn_inner=512, ffn_act=host.FFN_GEGLU)
    assert [e["label"] for e in mu.describe(2, 32)][-4:] == ["ffn1(gate+up)", "bias+geglu", "ffn2", "layer_norm"]
    assert mu.param_info()["layer0.w1"]["interleave16"] == 0
    mp = host.Model(0, 2, 32, 4, 64, packed_qkv=True)
    assert [e["label"] for e in mp.describe(2, 32)][:3] == ["qkv_gemm", "fused_qkv_bias_transpose", "qk_gemm"]
    assert mp.kernels_per_layer() == 12
    mpf = host.Model(1, 2, 32, 4, 64, fused=True, packed_qkv=True, max_cache_len=40)
    assert [e["label"] for e in mpf.describe(2, 32)][:3] == ["qkv_gemm+bias+heads", "attn_prefill_fused", "out_proj"]
    assert mpf.kernels_per_layer() == 7 and sorted(mpf.param_info()) == sorted(mp.param_info())
    assert [e["label"] for e in mpf.describe(2, 1, decode_past=10)][0] == "qkv_gemm(decode)"
    assert mg.kernels_per_layer() == 9
    m2 = host.Model(0, 2, 32, 4, 64, layer_num=3, norm_mode=host.PRE_LN_RESID)
    assert len(m2.describe(2, 32)) == 3 * 15
    with pytest.raises(host.capi.LigerError):
        host.Model(1, 2, 32, 5, 64, world_size=2)      # heads not divisible by the TP degree
    with pytest.raises(host.capi.LigerError):
        host.Model(0, 2, 32, 4, 64, fused=True)        # fused assembly is fp16 only


def test_entries_timed_inside_whole_steps_add_up_to_the_step(fake):
    """time_step launches the whole vector (two untimed passes + reps) with an event between every two entries: every entry is
    launched once per pass in vector order, and on the virtual-time backend the per-entry means equal the looped per-kernel
    times plus the host launch cost that separates two entries."""
    host = fake.host
    m = small_model(host)
    n = m.kernels_per_layer()
    fake.reset()
    per_entry = m.time_step(0x10000, 0x20000000, 2, 64, reps=3)
    launches = [e for e in fake.trace() if e["name"] not in ("event_record",)]
    assert len(per_entry) == n and all(t > 0 for t in per_entry)
    one_pass = [e["name"] for e in fake_trace_of(fake, m, 2, 64)]
    assert [e["name"] for e in launches] == one_pass * 5            # 2 untimed passes + 3 timed ones
    looped = m.time_kernels(0x10000, 0x20000000, 2, 64, iters=2, trials=1)
    assert per_entry == pytest.approx(looped, abs=0.01)             # virtual durations; 0.002 ms launch cost per entry


def test_sequential_run_launches_every_entry_once_in_order(fake):
    host = fake.host
    m = small_model(host)
    s = host.Scheduler(m, pool_count=3, ctx_batch=1)
    fake.reset()
    s.serve(1, 64)
    s.serve(1, 48)
    r = s.run_queued(host.MODE_SEQUENTIAL)
    t = fake.trace()
    assert r["records"] == 2 and r["secondary_launches"] == 0 and r["rounds"] == 2
    assert len({e["stream"] for e in t}) == 1
    names = ["gemm_fused"] * 3 + ["attn_prefill", "gemm", "layer_norm", "gemm_fused", "gemm", "layer_norm"]
    assert [e["name"] for e in t] == names * 2
    assert [e["n"] for e in t if e["name"] == "gemm"] == [64, 64, 48, 48]
    assert all(b["start"] >= a["end"] - 1e-12 for a, b in zip(t, t[1:]))


def test_classic_policy_degenerates_to_sequential_without_communication(fake):
    """With COMMUNICATION vs rest as the only classes and no all-reduce entry in a one-GPU vector, nothing may be
    launched on the secondary stream."""
    host = fake.host
    m = small_model(host)
    s = host.Scheduler(m, policy=host.POLICY_CLASSIC, pool_count=3, ctx_batch=1)
    s.profile(1, 64, 64, 1, 2)
    fake.reset()
    s.serve(1, 64)
    s.serve(1, 64)
    r = s.run_queued(host.MODE_LIGER)
    assert r["secondary_launches"] == 0 and r["splits"] == 0
    assert len({e["stream"] for e in fake.trace()}) == 1


def test_resource_policy_worked_example(fake):
    """Two identical prefill requests A (primary) and B.  Fused vector: [q k v attn out](MFMA) [ln](HBM) [ffn1 ffn2](MFMA) [ln](HBM).
    Scheduling window 1: A launches q,k,v,attn,out; B's next is MFMA -> same class -> nothing on stream 1.
    Scheduling window 2: A launches ln (0.0695 ms window, x0.8 = 0.0556).  B: q,k,v (0.0124 each), attn (0.0082) fit -> 0.0102 left;
             out_proj (0.0124) does not fit -> split with profiled fractions [0.0061, 0.0082, 0.0103] -> 2/4 fits ->
             first piece (128 of 256 output columns) goes to stream 1, remainder (128 columns) stays queued.
    Scheduling window 3: A launches ffn1, ffn2 (MFMA); B's next (remainder of out_proj) is MFMA -> nothing.
    Scheduling window 4: A launches its last ln; B's remainder fits the window and runs on stream 1; B's ln is HBM -> stop.
    Then B becomes primary and finishes alone on stream 0."""
    host = fake.host
    m = small_model(host, factor=4)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, pool_count=3, ctx_batch=1)
    s.profile(1, 64, 64, 1, 2)
    # profiled with 2 launches per timing: the first launch starts one host launch cost (0.002) after the start event,
    # so the per-launch figure is the kernel cost + 0.001
    assert abs(s.lookup(0, 1, 64) - (0.003 + 2 * 256 * 64 * 256 / 1e9 + 0.001)) < 1e-6
    assert abs(s.lookup(5, 1, 64) - (0.003 + 2 * 64 * 256 * 2 / 1e6 + 0.001)) < 1e-6
    sub = s.sub_lookup(4, 1, 64)
    assert len(sub) == 3 and all(abs(v - (0.003 + 2 * (64 * (i + 1)) * 64 * 256 / 1e9 + 0.001)) < 1e-6 for i, v in enumerate(sub))
    assert s.sub_lookup(5, 1, 64) is None  # only GEMM entries are decomposable
    fake.reset()
    s.serve(1, 64)
    s.serve(1, 64)
    r = s.run_queued(host.MODE_LIGER)
    t = fake.trace()
    s0 = min(e["stream"] for e in t)
    seq = [(e["stream"] - s0, e["name"], e["m"]) for e in t]
    A1 = [(0, "gemm_fused", 256)] * 3 + [(0, "attn_prefill", 4), (0, "gemm", 256), (0, "layer_norm", 64)]
    B1 = [(1, "gemm_fused", 256)] * 3 + [(1, "attn_prefill", 4), (1, "gemm", 128)]
    A2 = [(0, "gemm_fused", 512), (0, "gemm", 256), (0, "layer_norm", 64)]
    B2 = [(1, "gemm", 128)]
    B3 = [(0, "layer_norm", 64), (0, "gemm_fused", 512), (0, "gemm", 256), (0, "layer_norm", 64)]
    assert seq == A1 + B1 + A2 + B2 + B3
    assert r["secondary_launches"] == 6 and r["splits"] == 1 and r["records"] == 2
    # the two pieces of B's out_proj tile the output: same weights base + 128 columns (fp16), same activations, C + 128 columns
    p1, p2 = [e for e in t if e["name"] == "gemm" and e["m"] == 128]
    assert p2["A"] - p1["A"] == 128 * 2 and p2["C"] - p1["C"] == 128 * 2 and p1["B"] == p2["B"]
    # stream 1 is gated on the end of the previous primary round (device-side event wait)
    end_round1 = [e for e in t if e["stream"] == s0][4]["end"]
    first_b = [e for e in t if e["stream"] != s0][0]
    assert first_b["start"] >= end_round1 - 1e-12
    # budget: secondary work launched in a round never exceeds contention_factor x the primary window
    assert sum(e["end"] - e["start"] for e in t[6:11]) <= 0.8 * (t[5]["end"] - t[5]["start"]) + 1e-9
    # B moves from stream 1 to stream 0: its first kernel there starts after its last kernel on stream 1 has ended
    assert t[15]["start"] >= t[14]["end"] - 1e-12


@pytest.mark.parametrize("contention,expect_splits", [(0.8, False), (0.12, True), (0.05, True)])
def test_decode_request_fills_prefill_gemm_windows_and_splits_cover_exactly(fake, contention, expect_splits):
    """Primary = a prefill request (long MFMA rounds), secondary = a request with decode steps (HBM-bound kernels).
    Every kernel of every request is launched exactly once and per request in order; decomposed GEMM pieces of the
    decode request's skinny GEMMs are not produced (they fit), while a swapped case (decode primary, prefill secondary)
    produces splits whose pieces partition the columns."""
    host = fake.host
    m = small_model(host, factor=8)
    s = host.Scheduler(m, contention_factor=contention, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=3, ctx_batch=1)
    s.profile(1, 48, 64, 16, 2)
    for past in (48, 64, 80):
        s.profile_decode(1, past, 2)
    fake.reset()
    s.serve(1, 48, 3)   # A: prefill 48 + 3 decode steps
    s.serve(1, 64, 0)   # B: prefill only
    r = s.run_queued(host.MODE_LIGER)
    t = fake.trace()
    assert r["records"] == 2 and r["profile_misses"] == 0
    # B's GEMMs (token dimension 64) : total output columns per weight matrix must be covered exactly once
    weights = {n: (p, p + 2 * cnt) for n, (p, cnt) in m.params().items() if n.split(".")[1] in ("wq", "wk", "wv", "wo", "w1", "w2")}
    cover = {}
    for e in t:
        if e["name"] in ("gemm", "gemm_fused") and e["n"] == 64:
            owner = [n for n, (lo, hi) in weights.items() if lo <= e["A"] < hi]
            assert len(owner) == 1
            cover.setdefault(owner[0], []).append((e["C"], e["m"]))
    widths = {n.split(".")[1]: sum(m_ for _, m_ in v) for n, v in cover.items()}
    assert widths == {"wq": 256, "wk": 256, "wv": 256, "wo": 256, "w1": 512, "w2": 256}
    for n, v in cover.items():
        v.sort()
        if n.endswith(("wq", "wk", "wv")):
            continue  # head-transposed outputs: pieces are whole heads, checked by the width sum above
        for (c0, m0), (c1, _) in zip(v, v[1:]):
            assert c1 - c0 == m0 * 2              # contiguous fp16 column ranges: no gap, no overlap
    assert (r["splits"] > 0) == expect_splits
    # A's decode kernels: 3 steps x 7 entries, in order, attention lengths 49, 50, 51
    assert [e["n"] for e in t if e["name"] == "attn_decode"] == [49, 50, 51]
    assert r["secondary_launches"] > 0
    # per-request order in virtual time (n == tokens identifies the request for row-shaped kernels)
    for tokens in (48, 64):
        mine = [e for e in t if (e["name"] in ("gemm", "gemm_fused") and e["n"] == tokens) or (e["name"] == "layer_norm" and e["m"] == tokens)]
        assert all(b["start"] >= a["end"] - 1e-12 for a, b in zip(mine, mine[1:]))


MFMA, HBM = 0, 1   # resource classes (launch_context.h)


@pytest.mark.parametrize("speed", [1.0, 0.625, 0.4])
def test_measured_contention_matches_the_backend_model(fake, speed):
    """profile_contention runs prefill MFMA kernels on stream 0 next to repeated decode steps on stream 1.  On the
    virtual-time backend a kernel launched beside a busy stream runs at `speed`, so the concurrent run must take
    max(primary, secondary / speed) and the hidden fraction follows from the three times."""
    host = fake.host
    m = small_model(host)
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, pool_count=1, ctx_batch=1)
    assert s.contention(MFMA, HBM) == pytest.approx(0.8)      # unmeasured: the reference's constant
    fake.reset()                                               # also restores speed 1
    fake.set_corun_speed(speed)
    r = s.profile_contention(1, 64, 1, 64)
    launch_slack = 0.002 * 64                                  # host launch cost of the issued kernels (virtual ms)
    assert r["sub_repeats"] >= 1
    assert r["both_ms"] == pytest.approx(max(r["main_ms"], r["sub_ms"] / speed), abs=launch_slack)
    hidden = (r["main_ms"] + r["sub_ms"] - r["both_ms"]) / r["sub_ms"]
    assert r["hidden"] == pytest.approx(min(1.0, max(0.05, hidden)), rel=1e-5)
    assert s.contention(MFMA, HBM) == pytest.approx(r["hidden"])
    assert s.contention(HBM, MFMA) == pytest.approx(min(1.0, max(0.05, (r["main_ms"] + r["sub_ms"] - r["both_ms"]) / r["main_ms"])), rel=1e-5)
    assert s.contention(HBM, HBM) == pytest.approx(0.8)       # other pairs keep the constant
    # independent timelines (speed 1) hide most of the secondary (all but launch offsets and the rounding of the repeat
    # count); a slower co-run hides less
    limit = {1.0: (0.6, 1.0), 0.625: (0.2, 0.6), 0.4: (0.05, 0.2)}[speed]
    assert limit[0] <= r["hidden"] <= limit[1]
    s.set_contention(MFMA, HBM, -1.0)
    assert s.contention(MFMA, HBM) == pytest.approx(0.8)


def test_contention_table_sets_the_secondary_budget(fake):
    """The table entry for (primary class, secondary class) replaces the constant: a small entry admits fewer secondary
    launches per round than the default 0.8, a table entry equal to the constant changes nothing."""
    host = fake.host

    def run(entry):
        m = small_model(host, factor=8)
        s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=3, ctx_batch=1)
        s.profile(1, 48, 64, 16, 2)
        for past in (48, 64, 80):
            s.profile_decode(1, past, 2)
        if entry is not None:
            s.set_contention(HBM, MFMA, entry)
            s.set_contention(MFMA, HBM, entry)
        fake.reset()
        s.serve(1, 48, 3)
        s.serve(1, 64, 0)
        r = s.run_queued(host.MODE_LIGER)
        t = fake.trace()
        ids = sorted({e["stream"] for e in t})   # stream ids grow with every scheduler: compare their rank
        order = [(ids.index(e["stream"]), e["name"], e["m"], e["n"], e["k"]) for e in t]
        return r, order

    base, base_order = run(None)
    same, same_order = run(0.8)
    assert same_order == base_order and same["secondary_launches"] == base["secondary_launches"]
    tight, tight_order = run(0.05)
    assert tight["records"] == 2
    assert sorted(x[1:] for x in tight_order if not x[1].startswith("gemm")) == sorted(x[1:] for x in base_order if not x[1].startswith("gemm"))
    assert tight["rounds"] >= base["rounds"]
    assert tight_order != base_order


def test_missing_or_short_profile_never_splits_or_crashes(fake):
    host = fake.host
    m = small_model(host, factor=8)
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, pool_count=3, ctx_batch=1)
    # main durations only for the primary's ln (window) and a GEMM that is too long; sub profile shorter than factor-1
    for k in range(9):
        s.set_profile(k, 1, 64, 1.0 if k in (5, 8) else 5.0, sub=[0.1, 0.2] if k == 0 else None)
    fake.reset()
    s.serve(1, 64)
    s.serve(1, 64)
    r = s.run_queued(host.MODE_LIGER)
    assert r["records"] == 2 and r["splits"] == 0 and r["secondary_launches"] == 0
    # with no profile at all every lookup misses, durations are 0, windows are 0: still drains, sequentially
    s2 = host.Scheduler(m, policy=host.POLICY_RESOURCE, pool_count=3, ctx_batch=1)
    fake.reset()
    s2.serve(1, 64)
    s2.serve(1, 32)
    r2 = s2.run_queued(host.MODE_LIGER)
    assert r2["records"] == 2 and r2["profile_misses"] == 18 and r2["secondary_launches"] == 0


def test_profile_json_roundtrip_and_failure_paths(fake, tmp_path):
    host = fake.host
    m = small_model(host)
    s = host.Scheduler(m, pool_count=0)
    s.profile(1, 32, 64, 32, 2)
    a, b = str(tmp_path / "Main_1_64_4_1_64.json"), str(tmp_path / "Sub_1_64_4_1_64.json")
    s.save(a, b)
    main = json.load(open(a))
    sub = json.load(open(b))
    assert {tuple(sorted(e)) for e in main} == {("batch_size", "duration", "kernel_name", "seq_len")}   # utils.h:106-127 schema
    assert len(main) == 18 and len(sub) == 12 and all(len(e["duration"]) == 3 for e in sub)            # factor 4 -> 3 fractions
    s2 = host.Scheduler(m, pool_count=0)
    s2.load(a, b)
    for e in main:
        assert abs(s2.lookup(e["kernel_name"], e["batch_size"], e["seq_len"]) - e["duration"]) < 1e-6
    # a measured contention table travels in the main file as records with kernel_name -1 (same schema) and comes back
    s.set_contention(MFMA, HBM, 0.55)
    s.set_contention(HBM, MFMA, 0.25)
    s.save(a, b)
    main2 = json.load(open(a))
    extra = sorted((e["batch_size"], e["seq_len"], round(e["duration"], 6)) for e in main2 if e["kernel_name"] == -1)
    assert extra == [(MFMA, HBM, 0.55), (HBM, MFMA, 0.25)] and len(main2) == len(main) + 2
    s3 = host.Scheduler(m, contention_factor=0.8, pool_count=0)
    assert s3.contention(MFMA, HBM) == pytest.approx(0.8)          # unmeasured: the constant factor
    s3.load(a, b)
    assert s3.contention(MFMA, HBM) == pytest.approx(0.55) and s3.contention(HBM, MFMA) == pytest.approx(0.25)
    assert s3.lookup(-1, MFMA, HBM) == 0.0                         # not left behind as a kernel entry
    s.set_contention(MFMA, HBM, -1.0)
    s.set_contention(HBM, MFMA, -1.0)
    # a file in the reference's own writer format (trailing-comma-free, "duration": [ ... ] with a space)
    open(a, "w").write('[{"kernel_name":0,"batch_size":2,"seq_len":64,"duration":1.5},{"kernel_name":1,"batch_size":2,"seq_len":64,"duration":0.25}]')
    open(b, "w").write('[{"kernel_name":0,"batch_size":2,"seq_len":64,"duration": [0.2,0.4,0.6]}]')
    s2.load(a, b)
    assert s2.lookup(0, 2, 64) == 1.5 and s2.lookup(1, 2, 64) == 0.25 and s2.sub_lookup(0, 2, 64) == pytest.approx([0.2, 0.4, 0.6])
    for bad in ("", "[{\"kernel_name\":0}]", "{", "[{\"kernel_name\":0,\"batch_size\":1,\"seq_len\":2,\"duration\":[1,2]}]"):
        open(a, "w").write(bad)
        with pytest.raises(host.capi.LigerError):
            s2.load(a, b)
    with pytest.raises(host.capi.LigerError):
        s2.load(str(tmp_path / "missing.json"), b)


def test_report_arithmetic_reproduces_the_published_logs(fake):
    """Known-answer test: mean(CPU_Time + CUDA_Time) over the 131 request lines of the reference's published runs gives
    the printed Average Latency, and 1000 * records / Total_Duration the printed Throughput (schedule.h:325-348)."""
    host = fake.host
    logs = json.load(open(os.path.join(GOLD, "reference_logs.json")))
    for run, avg in (("baseline", 260.409698), ("liger", 199.714066)):
        d = logs[run]
        r = host.summarize(d["cpu_ms"], d["gpu_ms"], d["printed"]["Total_Duration"])
        assert r["records"] == d["printed"]["records"] == 131
        assert abs(r["avg_latency_ms"] - avg) < 2e-3 and abs(avg - d["printed"]["Average Latency"]) < 1e-9
        assert abs(r["throughput"] - d["printed"]["Throughput"]) < 1e-3
        lat = np.sort(np.array(d["cpu_ms"]) + np.array(d["gpu_ms"]))
        assert r["p99_latency_ms"] == pytest.approx(lat[int(np.ceil(0.99 * 131)) - 1])
    assert host.summarize([], [], 0.0)["records"] == 0


def test_poisson_trace_is_seeded_and_has_the_right_rate(fake):
    host = fake.host
    tr = host.make_poisson_trace(8.0, 4000, 1, 128, 1024, 64, 32, 7)
    assert tr == host.make_poisson_trace(8.0, 4000, 1, 128, 1024, 64, 32, 7)
    assert tr != host.make_poisson_trace(8.0, 4000, 1, 128, 1024, 64, 32, 8)
    arr = np.array([t["arrival_s"] for t in tr])
    gaps = np.diff(np.concatenate([[0.0], arr]))
    assert np.all(gaps > 0) and abs(gaps.mean() - 1 / 8.0) < 0.01 and abs(gaps.std() - 1 / 8.0) < 0.02   # exponential: mean == std
    seqs = np.array([t["seq"] for t in tr])
    assert seqs.min() >= 128 and seqs.max() <= 1024 and np.all(seqs % 64 == 0) and len(set(seqs)) == 15
    assert all(t["n_decode"] == 32 and t["batch"] == 1 for t in tr)


def test_realtime_trace_replay_drains(fake):
    """The threaded path (request thread + scheduler loop): arrivals in real time, all requests reported."""
    host = fake.host
    m = small_model(host)
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, pool_count=2, ctx_batch=1, ignore_num=0)
    s.profile(1, 64, 64, 1, 2)
    trace = [{"arrival_s": 0.002 * i, "batch": 1, "seq": 64, "n_decode": 0} for i in range(12)]
    for mode in (host.MODE_SEQUENTIAL, host.MODE_LIGER):
        fake.reset()
        r = s.run_trace(trace, mode)
        assert r["records"] == 12
        assert len([e for e in fake.trace() if e["name"] == "attn_prefill"]) == 12


def test_merged_minor_kernels_keep_a_prefill_in_one_run(fake):
    """RESOURCE policy with merge_minor: minor entries (the LayerNorms between a prefill's GEMMs, the row gather before the
    decode steps) take the class of the entry before them.  A prefill is then one run of MFMA-bound launches instead of four
    per layer, and a prefill that waits behind a request in its decode steps (HBM-bound) is interleaved past its first
    LayerNorm.  Every entry is still launched exactly once and every request keeps its own order."""
    host = fake.host
    m = small_model(host, layers=2)

    def run(merge, requests):
        s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=3, ctx_batch=1)
        s.profile(1, 48, 64, 16, 2)
        for past in (48, 64, 80):
            s.profile_decode(1, past, 2)
        s.set_merge_minor(merge)
        fake.reset()
        for r in requests:
            s.serve(*r)
        rep = s.run_queued(host.MODE_LIGER)
        return rep, fake.trace()

    # one prefill-only request: 2 layers x (5 MFMA, LN, 2 MFMA, LN) = 8 runs; one run when the LayerNorms are merged
    plain, t0 = run(False, [(1, 64, 0)])
    merged, t1 = run(True, [(1, 64, 0)])
    assert plain["rounds"] == 8 and merged["rounds"] == 1
    assert [e["name"] for e in t0] == [e["name"] for e in t1] and len(t1) == 2 * 9
    # A: prefill + 3 decode steps (one MFMA run, then one HBM run), B: prefill only, queued behind it
    reqs = [(1, 48, 3), (1, 64, 0)]
    plain, t0 = run(False, reqs)
    merged, t1 = run(True, reqs)
    assert plain["records"] == merged["records"] == 2
    assert sorted(e["name"] for e in t0) == sorted(e["name"] for e in t1)     # the same launches, each exactly once
    assert merged["rounds"] < plain["rounds"]
    # without merging B's interleaving stops at its first LayerNorm at the latest (5 launches); with it B goes on past it
    assert 0 < plain["secondary_launches"] <= 5
    assert merged["secondary_launches"] > 5
    b_rows = [e for e in t1 if (e["name"] in ("gemm", "gemm_fused") and e["n"] == 64) or (e["name"] == "layer_norm" and e["m"] == 64)]
    assert all(y["start"] >= x["end"] - 1e-12 for x, y in zip(b_rows, b_rows[1:]))   # B's own order is kept


def test_requests_that_exceed_the_contexts_are_refused_on_the_host(fake):
    """Shapes decide how far a launch vector writes into a request's buffers and KV-cache slots, so every entry point that
    builds one checks them first and launches nothing (no kernel may write outside its buffers)."""
    host = fake.host
    m = small_model(host, max_batch=4, cache=80)      # max_seq 64, cache 80 rows, 4 slots
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, pool_count=2, ctx_batch=2)
    s.profile(1, 64, 64, 1, 2)
    fake.reset()
    for bad in ((3, 64, 0),      # batch beyond the contexts' batch
                (1, 65, 0),      # sequence beyond max_seq_len
                (1, 64, 17),     # 64 + 17 decode steps do not fit 80 cache rows
                ):
        with pytest.raises(host.capi.LigerError):
            s.serve(*bad)
    with pytest.raises(host.capi.LigerError):
        s.serve_decode(1, 70, 11)                      # past + steps beyond the cache
    with pytest.raises(host.capi.LigerError):
        s.serve_decode(3, 10, 1)                       # batch beyond the contexts' batch
    with pytest.raises(host.capi.LigerError):
        s.profile_decode(1, 80)                        # position 80 is outside an 80-row cache
    with pytest.raises(host.capi.LigerError):
        s.profile_contention(1, 64, 3, 10)             # decode batch beyond the context
    with pytest.raises(host.capi.LigerError):
        m.run(0x1000, 0x2000, 2, 64, cache_slot=3)     # slots 3, 4 of 4
    with pytest.raises(host.capi.LigerError):
        m.run_decode(0x1000, 0x2000, 1, 80, cache_slot=0)
    with pytest.raises(host.capi.LigerError):
        m.time_kernels(0x1000, 0x2000, 5, 64)          # batch beyond max_batch
    with pytest.raises(host.capi.LigerError):
        m.time_kernels(0x1000, 0x2000, 1, 1, decode_past=80, cache_slot=0)
    with pytest.raises(host.capi.LigerError):
        m.time_step(0x1000, 0x2000, 5, 64)             # batch beyond max_batch
    nocache = small_model(host, cache=0, fused=False)
    s2 = host.Scheduler(nocache, pool_count=1, ctx_batch=1)
    with pytest.raises(host.capi.LigerError):
        s2.serve(1, 32, 1)                             # decode steps without a KV cache
    with pytest.raises(host.capi.LigerError):
        s2.serve_decode(1, 0, 1)
    assert fake.trace() == []                          # nothing was launched by any of the refused calls
    # what fits is still accepted afterwards
    s.serve(2, 64, 16)
    assert s.run_queued(host.MODE_SEQUENTIAL)["records"] == 1


def test_more_queued_requests_than_contexts_fail_instead_of_deadlocking(fake):
    host = fake.host
    m = small_model(host)
    s = host.Scheduler(m, pool_count=2, ctx_batch=1)
    s.serve(1, 32)
    s.serve(1, 32)
    with pytest.raises(host.capi.LigerError, match="no scheduler loop"):
        s.serve(1, 32)                                 # no loop is running that could return a context
    assert s.run_queued(host.MODE_LIGER)["records"] == 2
    s.serve(1, 32)                                     # contexts are back
    assert s.run_queued(host.MODE_LIGER)["records"] == 1


def test_interleaving_without_request_contexts_is_refused(fake):
    """Two requests on two streams that share the model's default buffers would race: run_stream_sync needs a pool."""
    host = fake.host
    m = small_model(host)
    s = host.Scheduler(m, schedule_deep=6, pool_count=0)
    s.serve(1, 32)
    s.serve(1, 32)
    with pytest.raises(host.capi.LigerError, match="per-request contexts"):
        s.run_queued(host.MODE_LIGER)
    s1 = host.Scheduler(m, schedule_deep=1, pool_count=0)   # one request in flight at a time: allowed
    s1.serve(1, 32)
    assert s1.run_queued(host.MODE_LIGER)["records"] == 1


def test_request_off_the_profile_grid_is_still_split(fake):
    """Durations are looked up at seq rounded up to the profile grid; the decomposition table must be looked up with the
    same key, or requests whose length is not itself a profiled key would never be split."""
    host = fake.host
    m = small_model(host, factor=4)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=3, ctx_batch=1)
    s.profile(1, 48, 64, 16, 2)
    fake.reset()
    s.serve(1, 64)
    s.serve(1, 52)            # looked up at 64
    r = s.run_queued(host.MODE_LIGER)
    assert r["records"] == 2 and r["profile_misses"] == 0 and r["sub_profile_misses"] == 0
    assert r["splits"] >= 1   # the worked example's split of B's out_proj happens for the off-grid request too
    pieces = [e for e in fake.trace() if e["name"] == "gemm" and e["n"] == 52 and e["m"] < 256]
    assert sum(e["m"] for e in pieces) == 256


def test_cu_mask_streams_need_every_die_and_report_their_share(fake):
    import ctypes as C
    lib = fake.lib
    st = C.c_void_p()
    mask = (C.c_uint * 8)(0xffffffff, 0xffffffff, 0, 0, 0, 0, 0, 0)       # 64 units
    assert lib.lg_stream_create_cu_mask(C.byref(st), mask, 8) == 0
    lib.lg_stream_cu_count.argtypes = [C.c_void_p]
    assert lib.lg_stream_cu_count(st) == 64 and lib.lg_stream_cu_count(None) == 256
    empty = (C.c_uint * 8)()
    assert lib.lg_stream_create_cu_mask(C.byref(st), empty, 8) != 0


def _partition_setup(fake, factor_hbm_main=None):
    host = fake.host
    m = small_model(host, factor=4, layers=2, max_batch=4, cache=128)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=3, ctx_batch=1)
    s.profile(1, 48, 64, 16, 2)
    for past in (48, 64, 80):
        s.profile_decode(1, past, 2)
    s.set_merge_minor(True)
    s.enable_partition(128)
    s.set_partition_feedback(False)     # these tests look at the partition mechanism itself, round by round
    if factor_hbm_main is not None:
        s.set_partition_factor(HBM, MFMA, factor_hbm_main)
        s.set_partition_factor(MFMA, HBM, 1.0 / factor_hbm_main)
    return host, m, s


def test_partitioned_rounds_run_only_while_the_other_class_has_work(fake):
    """Decode request A (HBM-bound, primary) and prefill request B (MFMA-bound, waiting).  With a partition, A's kernels run
    on the HBM side's compute units and B's on the MFMA side's for exactly as long as B has work; afterwards A is back on
    the whole chip (stream 0).  Every entry is launched once, each request in its own order."""
    host, m, s = _partition_setup(fake, factor_hbm_main=1.0)
    fake.reset()
    s.serve_decode(1, 48, 24)     # A: 24 decode steps x 2 layers x 7 kernels, one long HBM-bound run
    s.serve(1, 64, 0)             # B: two prefill layers, one MFMA-bound run (minor kernels merged)
    r = s.run_queued(host.MODE_LIGER)
    t = fake.trace()
    assert r["records"] == 2 and r["partition_rounds"] >= 1 and r["secondary_launches"] >= 18
    ids = sorted({e["stream"] for e in t})
    b_rows = [e for e in t if (e["name"] in ("gemm", "gemm_fused") and e["n"] == 64) or (e["name"] == "layer_norm" and e["m"] == 64) or e["name"] == "attn_prefill"]
    a_rows = [e for e in t if e not in b_rows]
    assert len(b_rows) == 18 + r["splits"] and len(a_rows) == 24 * 2 * 7
    # B ran on one masked stream only; A on another masked stream while B had work, on stream 0 (the lowest id) afterwards
    b_streams = {e["stream"] for e in b_rows}
    a_streams = [e["stream"] for e in a_rows]
    assert len(b_streams) == 1 and b_streams.isdisjoint(a_streams) and ids[0] not in b_streams
    assert a_streams[0] != ids[0] and a_streams[-1] == ids[0]
    switch = a_streams.index(ids[0])
    assert all(x == a_streams[0] for x in a_streams[:switch]) and all(x == ids[0] for x in a_streams[switch:])
    # the partitioned part of A is about as long as B's work divided by the factor (1.0): B's stand-alone time on the whole chip
    b_work = sum((e["end"] - e["start"]) / 2.0 for e in b_rows)          # measured on 128 of 256 units: twice the whole-chip cost
    a_part = sum((e["end"] - e["start"]) / 2.0 for e in a_rows[:switch])
    assert a_part == pytest.approx(b_work, rel=0.25)
    for rows in (a_rows, b_rows):
        assert all(y["start"] >= x["end"] - 1e-12 for x, y in zip(rows, rows[1:]))
    # no partition factor for the pair -> the same requests never leave the whole-chip streams
    s.set_partition_factor(HBM, MFMA, -1.0)
    fake.reset()
    s.serve_decode(1, 48, 24)
    s.serve(1, 64, 0)
    r2 = s.run_queued(host.MODE_LIGER)
    assert r2["partition_rounds"] == 0 and len({e["stream"] for e in fake.trace()}) <= 2


def test_a_failed_change_of_share_leaves_no_stream_behind_and_no_stale_pointer(fake):
    """enable_partition for a new share releases the streams of the old one before it creates its own.  Whatever goes wrong
    on the way, the scheduler must neither keep a pointer to a released stream (a later run synchronises the partition's
    streams) nor lose track of a stream it created (each holds a hardware queue and a workspace)."""
    host, m, s = _partition_setup(fake, factor_hbm_main=1.0)      # share 128 in use
    lib = fake.lib
    live = lib.fake_live_streams()
    # (1) an error recorded earlier (here: a refused request) is sticky and process-wide: the change is refused up front and
    #     the share in use stays usable
    assert lib.lgh_sched_serve(s.h, 99, 64, 0) != 0
    assert lib.lgh_sched_enable_partition(s.h, 64) != 0
    assert lib.fake_live_streams() == live
    lib.lgh_clear_error()
    s.serve_decode(1, 48, 8)
    s.serve(1, 64, 0)
    assert s.run_queued(host.MODE_LIGER)["partition_rounds"] >= 1
    # (2) the third of the four new streams cannot be created: the two that were are released again, the old share's four
    #     are gone, partitioning is off and runs use the two whole-chip streams only
    lib.fake_fail_cu_mask_streams_after(2)
    try:
        with pytest.raises(host.capi.LigerError):
            s.enable_partition(64)
    finally:
        lib.fake_fail_cu_mask_streams_after(-1)
    assert lib.fake_live_streams() == live - 4
    assert s.partition_factor(HBM, MFMA) == pytest.approx(1.0)      # the table is only reset by a successful change
    fake.reset()
    s.serve_decode(1, 48, 8)
    s.serve(1, 64, 0)
    r = s.run_queued(host.MODE_LIGER)
    assert r["records"] == 2 and r["partition_rounds"] == 0 and len({e["stream"] for e in fake.trace()}) <= 2
    # (3) and the share can be switched on again afterwards
    s.enable_partition(64)
    assert lib.fake_live_streams() == live
    s.set_partition_factor(HBM, MFMA, 1.0)
    s.serve_decode(1, 48, 8)
    s.serve(1, 64, 0)
    assert s.run_queued(host.MODE_LIGER)["partition_rounds"] >= 1
    s.close()
    assert lib.fake_live_streams() == live - 6


def test_the_streams_of_a_partitioned_round_are_probed_pair_by_pair(fake):
    """Two CU-masked streams may share a hardware queue and then take turns.  enable_partition probes both (primary,
    secondary) pairs, replaces a secondary that does not overlap with its primary (rejected candidates are released once
    a good one is found) and reports the outcome; a share whose pairs cannot be made to overlap gets no measured factor.
    The verification is opt-in (set_verify_partition_streams)."""
    host, m, s = _partition_setup(fake)                 # share 128, created without verification
    lib = fake.lib
    live = lib.fake_live_streams()
    assert s.partition_streams_concurrent is None
    s.set_verify_partition_streams(True)
    # the next three probes see streams that take turns: the first pair needs two replacements, the second pair one
    lib.fake_cu_mask_streams_created(1)
    lib.fake_serialise_probes(3)
    s.enable_partition(64)
    assert lib.fake_cu_mask_streams_created(1) == 4 + 3
    assert lib.fake_live_streams() == live             # the old share's four and the three rejected ones are gone
    assert s.partition_streams_concurrent
    fake.set_share_model(0.5, 0.2)                      # a backend on which a partition pays
    assert s.profile_partition(1, 48, 1, 48)["gain"] > 1.02 and s.partition_factor(MFMA, HBM) > 0
    # no candidate overlaps: the share is usable but flagged, and the measurement installs nothing
    lib.fake_serialise_probes(1000)
    s.enable_partition(32)
    lib.fake_serialise_probes(0)
    assert lib.fake_live_streams() == live
    assert s.partition_streams_concurrent is False
    assert s.profile_partition(1, 48, 1, 48)["gain"] > 1.02 and s.partition_factor(MFMA, HBM) < 0
    s.enable_partition(0)
    assert s.partition_streams_concurrent is None
    s.close()


@pytest.mark.parametrize("matrix_exp,memory_exp,corun,pays", [(1.0, 1.0, 1.0, False), (0.5, 0.2, 0.5, True)])
def test_partition_feedback_follows_what_the_rounds_deliver(fake, matrix_exp, memory_exp, corun, pays):
    """Prefill requests (MFMA-bound) and decode requests (HBM-bound) queued in turn, with a partition table that says every
    co-running round should be partitioned.  The backend decides what is true: (a) a share of the compute units costs in
    proportion and the whole chip overlaps two streams for free -> partitioned rounds deliver less than whole-chip rounds;
    (b) a share hurts less than in proportion and the whole chip only time-slices -> partitioned rounds deliver more.
    With feedback the scheduler runs both kinds of round in turn, then keeps the better kind (and probes the other now and
    then); without it every such round is partitioned, whatever it delivers."""
    host = fake.host
    m = host.Model(1, 41, 64, 4, 64, layer_num=2, ffn_inner=512, causal=True, fused=True, max_cache_len=128, factor=4, seed=0)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=40, ctx_batch=1)
    s.profile(1, 48, 64, 16, 2)
    for past in (48, 64, 80, 96, 112):
        s.profile_decode(1, past, 2)
    s.set_merge_minor(True)
    s.enable_partition(128)
    s.set_partition_factor(HBM, MFMA, 1.0)
    s.set_partition_factor(MFMA, HBM, 1.0)

    def run(feedback):
        s.set_partition_feedback(feedback, 3, 8, 1.02)
        fake.reset()
        fake.set_share_model(matrix_exp, memory_exp)
        fake.set_corun_speed(corun)
        for _ in range(20):
            s.serve(1, 64, 0)
            s.serve_decode(1, 48, 60)
        r = s.run_queued(host.MODE_LIGER)
        assert r["records"] == 40 and r["profile_misses"] == 0
        return r, s.partition_feedback_state()

    r, st = run(True)
    eligible = r["partition_rounds"] + st["declined"]
    assert eligible >= 15 and st["samples_whole_chip"] >= 3 and st["samples_partitioned"] >= 3
    if pays:
        assert st["rate_partitioned"] > 1.02 * st["rate_whole_chip"]
        assert r["partition_rounds"] >= 0.65 * eligible
    else:
        assert st["rate_partitioned"] < 1.02 * st["rate_whole_chip"]
        assert r["partition_rounds"] <= 0.45 * eligible
    # a second run starts from what the first one measured: no more turns, only the occasional probe of the other side
    r1, st1 = run(True)
    eligible1 = r1["partition_rounds"] + st1["declined"]
    assert (r1["partition_rounds"] >= 0.8 * eligible1) if pays else (r1["partition_rounds"] <= 0.2 * eligible1)
    r2, st2 = run(False)
    assert st2["declined"] == 0 and r2["partition_rounds"] >= 15
    s.close()
    m.close()


@pytest.mark.parametrize("matrix_exp,memory_exp,pays", [(1.0, 1.0, False), (0.5, 0.2, True)])
def test_measured_partition_follows_the_backend_model(fake, matrix_exp, memory_exp, pays):
    """profile_partition runs the prefill's MFMA-bound kernels on 128 of 256 compute units next to decode steps on the other
    128.  When a share costs in proportion (exponent 1) both sides take twice as long and nothing is gained: the table stays
    empty and rounds are never partitioned.  When a share hurts less than in proportion the co-run wins, and factor and gain
    follow from the model: matrix kernels 2^a times slower, memory kernels 2^b."""
    host, m, s = _partition_setup(fake)
    fake.reset()
    fake.set_share_model(matrix_exp, memory_exp)
    r = s.profile_partition(1, 64, 1, 64)
    slow_a, slow_b = 2.0 ** matrix_exp, 2.0 ** memory_exp
    assert r["main_part_ms"] == pytest.approx(r["main_ms"] * slow_a, rel=0.1)
    # a decode step mixes memory kernels with (tiny) matrix kernels: its slow-down lies between the two
    slow_sub = r["sub_part_ms"] / (r["sub_repeats"] * r["sub_ms"])
    assert min(slow_a, slow_b) * 0.9 <= slow_sub <= max(slow_a, slow_b) * 1.1
    assert r["factor"] == pytest.approx(slow_a / slow_sub, rel=0.1)
    if pays:
        assert r["gain"] > 1.2
        assert s.partition_factor(MFMA, HBM) == pytest.approx(r["factor"]) and s.partition_factor(HBM, MFMA) == pytest.approx(1 / r["factor"])
    else:
        assert r["gain"] < 1.02 and s.partition_factor(MFMA, HBM) < 0 and s.partition_factor(HBM, MFMA) < 0


@pytest.mark.parametrize("mode_name", ["liger", "sequential"])
def test_batched_decode_steps_share_one_launch_vector(fake, mode_name):
    """Requests that are in their decode steps at the same time run one step together (per-sequence cache slots and lengths),
    a request joins at the first step boundary after its prefill and leaves after its last step.  Invariants: every request
    runs exactly its number of decode steps; fewer batched steps are launched than the requests have steps in total; a
    request's row is copied in after its last prefill kernel and copied out after its last step; rows that belong to no
    request point at the spare cache slot."""
    host = fake.host
    pool = 3
    m = host.Model(1, pool + 1, 64, 4, 64, layer_num=2, ffn_inner=512, causal=True, fused=True, max_cache_len=128, factor=4, seed=0)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=pool, ctx_batch=1)
    s.profile(1, 32, 64, 16, 2)
    for bs in (1, 2, 3):
        for past in (32, 48, 64, 80):
            s.profile_decode(bs, past, 2)
    s.set_merge_minor(True)
    s.enable_batch_decode(True, 2)
    reqs = [(1, 48, 5), (1, 64, 3), (1, 32, 6)]
    fake.reset()
    for r in reqs:
        s.serve(*r)
    rep = s.run_queued(host.MODE_LIGER if mode_name == "liger" else host.MODE_SEQUENTIAL)
    t = fake.trace()
    assert rep["records"] == 3 and rep["profile_misses"] == 0
    steps = [e for e in t if e["name"] == "attn_decode_varlen"]
    layers = 2
    assert len(steps) == rep["batched_steps"] * layers
    total_steps = sum(n for _, _, n in reqs)
    assert max(n for _, _, n in reqs) <= rep["batched_steps"] < total_steps          # some steps were shared
    # keys attended per step = sum over the live sequences of (cached + 1); a row of no request attends to 1 key of the spare slot.
    # Summed over all steps of one layer: every request contributes sum_{t < n} (seq + t + 1); the rest are holes (1 key each)
    keys = sum(e["n"] for e in steps[::layers])
    rows = sum(e["m"] // 4 for e in steps[::layers])          # 4 heads
    own = sum(sum(seq + t + 1 for t in range(n)) for _, seq, n in reqs)
    holes = rows - total_steps
    assert rows == rep["batched_rows"] and holes >= 0 and keys == own + holes
    copies = [e for e in t if e["name"] == "memcpy_d2d"]
    assert len(copies) == 2 * len(reqs)                        # one row in, one row out per request
    # a request's row is copied into the batch only after its last prefill kernel: the three prefills end with a LayerNorm over
    # 48, 64 and 32 token rows; the copy-in of the context with the matching output buffer starts after it
    for i, (_, seq, _) in enumerate(reqs):
        pin, pout = s.ctx_ptrs(i)
        last_ln = [e for e in t if e["name"] == "layer_norm" and e["m"] == seq][-1]
        assert last_ln["C"] == pout
        row_bytes = 256 * 2
        join = [e for e in copies if e["A"] == pout + (seq - 1) * row_bytes]
        assert len(join) == 1 and join[0]["start"] >= last_ln["end"] - 1e-12
    # no batched decode without the spare cache slot
    m2 = host.Model(1, pool, 64, 4, 64, layer_num=1, ffn_inner=512, causal=True, fused=True, max_cache_len=128, seed=0)
    s2 = host.Scheduler(m2, pool_count=pool, ctx_batch=1)
    with pytest.raises(host.capi.LigerError):
        s2.enable_batch_decode(True)


@pytest.mark.parametrize("steps_ahead", [1, 3])
def test_every_batched_step_carries_each_live_request_at_its_own_position(fake, steps_ahead):
    """The per-step row tables the batched decode vector is built from, seen through the step hook: row r of step k belongs
    to cache slot r (one-sequence contexts) at the position that request has reached, or to the spare slot at position 0.
    For every request the steps that carry it are consecutive, start at its prompt length, advance by one and number exactly
    its decode steps; no step is empty; a step never has more rows than the highest live slot + 1."""
    host = fake.host
    pool = 4
    m = host.Model(1, pool + 1, 64, 4, 64, layer_num=2, ffn_inner=512, causal=True, fused=True, max_cache_len=128, factor=4, seed=0)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=16, pool_count=pool, ctx_batch=1)
    s.profile(1, 16, 64, 16, 2)
    for bs in (1, 2, 3, 4):
        for past in (16, 32, 48, 64, 80):
            s.profile_decode(bs, past, 2)
    s.set_merge_minor(True)
    s.enable_batch_decode(True, steps_ahead)
    seen = []
    s.set_decode_step_hook(lambda step, slots, pasts, ptr, stream: seen.append((step, slots, pasts)))
    reqs = [(1, 48, 5), (1, 64, 1), (1, 17, 7), (1, 32, 4)]
    fake.reset()
    for r in reqs:
        s.serve(*r)
    rep = s.run_queued(host.MODE_LIGER)
    assert rep["records"] == len(reqs) and rep["batched_steps"] == len(seen)
    assert [k for k, _, _ in seen] == list(range(len(seen)))
    spare = pool
    for i, (_, seq, n) in enumerate(reqs):
        carried = [(k, pasts[i]) for k, slots, pasts in seen if i < len(slots) and slots[i] == i]
        assert [p for _, p in carried] == list(range(seq, seq + n)), "request %d" % i
        assert [k for k, _ in carried] == list(range(carried[0][0], carried[0][0] + n))
    for k, slots, pasts in seen:
        live = [r for r, sl in enumerate(slots) if sl != spare]
        assert live and len(slots) == live[-1] + 1
        assert all(sl == r for r, sl in enumerate(slots) if sl != spare)
        assert all(pasts[r] == 0 for r, sl in enumerate(slots) if sl == spare)
    # launch order around a step: join copies come before the first kernel of the step that first carries the request, the
    # copy-out after the last kernel of its last step
    t = fake.trace()
    steps = [e for e in t if e["name"] == "attn_decode_varlen"][::2]       # first layer's attention of every step
    assert len(steps) == len(seen)
    row_bytes = 256 * 2
    for i, (_, seq, n) in enumerate(reqs):
        pout = s.ctx_ptrs(i)[1]
        first = next(k for k, slots, _ in seen if i < len(slots) and slots[i] == i)
        join = [e for e in t if e["name"] == "memcpy_d2d" and e["A"] == pout + (seq - 1) * row_bytes]
        assert len(join) == 1 and join[0]["end"] <= steps[first]["start"] + 1e-12
        if first > 0:
            assert join[0]["start"] >= steps[first - 1]["end"] - 1e-12       # it joined at a step boundary
    s.set_decode_step_hook(None)
    s.close()


@pytest.mark.parametrize("mode_name", ["sequential", "liger"])
def test_chunked_prefill_lets_the_decode_batch_step_between_chunks(fake, mode_name):
    """Request A (prompt 32, 12 decode tokens) is in its decode steps when request B (prompt 128) has its prefill.  With
    prefill_chunk = 32 B's prefill is four chunks of 32 tokens, each through both layers over B's cache slot: the attention of
    chunk c is the continuing kind with past = 32 c, every other kernel works on 32 token rows, and between two chunks the
    batched decode step gets the primary's turn.  Without chunking B's prefill is one vector of 128-token kernels."""
    host = fake.host
    pool = 3
    m = host.Model(1, pool + 1, 128, 4, 64, layer_num=2, ffn_inner=512, causal=True, fused=True, max_cache_len=192, factor=4, seed=0)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, seq_bucket=32, pool_count=pool, ctx_batch=1)
    s.profile(1, 32, 128, 32, 2)
    for bs in (1, 2):
        for past in (32, 64, 128, 160):
            s.profile_decode(bs, past, 2)
    s.set_merge_minor(True)
    s.enable_batch_decode(True, 1)
    mode = host.MODE_LIGER if mode_name == "liger" else host.MODE_SEQUENTIAL

    def run(chunk):
        s.set_prefill_chunk(chunk)
        fake.reset()
        s.serve(1, 32, 12)      # A: as long as a chunk, so never cut
        s.serve(1, 128, 3)      # B
        r = s.run_queued(mode)
        assert r["records"] == 2 and r["profile_misses"] == 0
        return r, fake.trace(), s.chunk_counters()

    r0, t0, c0 = run(0)
    assert c0 == {"chunked_prefills": 0, "yield_turns": 0}
    assert not [e for e in t0 if e["name"] == "attn_prefill_past"]
    assert sorted(e["n"] for e in t0 if e["name"] == "attn_prefill") == [32, 32, 128, 128]
    r1, t1, c1 = run(32)
    assert c1["chunked_prefills"] == 1 and c1["yield_turns"] >= 2
    # B's chunks: one plain attention (past 0) and three continuing ones per layer, pasts 32, 64, 96, each over 32 queries
    past_attn = [e for e in t1 if e["name"] == "attn_prefill_past"]
    assert [(e["n"], e["k"]) for e in past_attn] == [(32, p) for p in (32, 32, 64, 64, 96, 96)]
    assert sorted(e["n"] for e in t1 if e["name"] == "attn_prefill") == [32, 32, 32, 32]     # A's two layers, B's first chunk
    # nothing of B works on 128 token rows any more (GEMMs: n = token rows; LayerNorm: m)
    assert not [e for e in t1 if (e["name"] in ("gemm", "gemm_fused") and e["n"] == 128) or (e["name"] == "layer_norm" and e["m"] == 128)]
    # every decode step of A and B is still there
    assert len([e for e in t1 if e["name"] == "attn_decode_varlen"]) == len([e for e in t0 if e["name"] == "attn_decode_varlen"])
    # between two consecutive chunks of B at least one batched decode step was launched (A is decoding all the while)
    marks = [i for i, e in enumerate(t1) if e["name"] == "attn_prefill_past"][::2]     # layer 0 of chunks 1, 2, 3
    assert len(marks) == 3
    for a, b in zip(marks, marks[1:]):
        assert any(e["name"] == "attn_decode_varlen" for e in t1[a:b]), "no decode step between two chunks"

    if mode_name == "sequential":
        # A's first decode steps no longer wait for the whole of B's prefill, only for its first chunk
        first = lambda t, k: [e["start"] for e in t if e["name"] == "attn_decode_varlen"][2 * k]
        b_done = lambda t: max(e["end"] for e in t if e["name"] in ("attn_prefill", "attn_prefill_past"))
        assert first(t0, 0) > b_done(t0)                 # unchunked: every decode step comes after B's last attention
        assert first(t1, 0) < 0.5 * first(t0, 0) and first(t1, 2) < b_done(t1)
    s.set_prefill_chunk(0)
    s.close()


@pytest.mark.parametrize("factor", [2, 4, 8])
@pytest.mark.parametrize("axis", [0, 1])
def test_cfg4_shapes_pieces_cover_the_prefill_exactly(fake, factor, axis):
    """BASELINE config 4 at its real shapes on the virtual-time backend, where every launch is visible: prefill batch 4 x seq
    512 on the TP=2 GLM-130B layer shard, decomposed by `factor`, next to a decode batch of 32 sequences at 1024 cached
    positions.  Whatever is split, the pieces of every weight GEMM of the prefill must cover its 2048 token rows (or its
    output features) exactly once, in order, with the operand pointers offset accordingly."""
    host = fake.host
    m = host.Model(1, 64, 512, 96, 128, layer_num=1, world_size=2, ffn_inner=32768, causal=True, fused=True, max_cache_len=1088, factor=factor, seed=0)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, axis=axis, seq_bucket=64, pool_count=2, ctx_batch=32)
    s.set_factor(factor)
    s.profile(4, 512, 512, 1, 2)
    s.profile_decode(32, 1024, 2)
    s.set_merge_minor(True)
    fake.reset()
    s.serve_decode(32, 1000, 3)   # three steps: a window that holds the attention block of the prefill and part of FFN-1
    s.serve(4, 512, 0)
    r = s.run_queued(host.MODE_LIGER)
    t = fake.trace()
    assert r["records"] == 2 and r["splits"] > 0 and r["profile_misses"] == 0 and r["sub_profile_misses"] == 0
    H, Hl, F, M = 12288, 6144, 16384, 2048
    pin, pout = s.ctx_ptrs(1)
    gemms = [e for e in t if e["name"] in ("gemm", "gemm_fused") and e["n"] != 32]      # the prefill's (the decode batch has 32 rows)
    by_weight = {}
    for e in gemms:
        by_weight.setdefault(e["A"] if axis == 1 else None, []).append(e)
    if axis == 1:   # token-row pieces share the weight pointer: group by it
        assert len(by_weight) == 6
        widths = sorted(v[0]["m"] for v in by_weight.values())
        assert widths == sorted([Hl, Hl, Hl, H, F, H])
        n_split = 0
        for v in by_weight.values():
            v.sort(key=lambda e: e["B"])
            assert sum(e["n"] for e in v) == M
            k = v[0]["k"]
            for a, b in zip(v, v[1:]):
                assert b["B"] - a["B"] == a["n"] * k * 2        # the next piece's activations start where this one's end
            n_split += len(v) > 1
        # the three head-transposing projections are always split by output features (token rows would move the batch decode)
        assert n_split >= 1
    else:           # output-feature pieces: every piece shares the activations; weights / outputs advance by whole features
        total = sum(e["m"] * e["n"] for e in gemms)
        assert total == M * (3 * Hl + H + F + H) and all(e["n"] == M for e in gemms)
        assert len(gemms) > 6


@pytest.mark.parametrize("weight_layout", [0, 1, 2])
def test_loading_a_parameter_relays_it_into_the_layers_storage_layout(fake, weight_layout):
    """lgh_model_load_param: one launch per parameter on the model's stream -- a copy when the source layout is the layer's,
    a transpose between the two plain layouts, the tiling kernel for a layer that stores fragment blocks; vectors are
    copied; interleaved (fused GeGLU) parameters, bad layouts and a parameter loaded from itself are refused."""
    host = fake.host
    m = host.Model(1, 2, 32, 4, 64, ffn_inner=512, fused=True, weight_layout=weight_layout, max_cache_len=40)
    info = m.param_info()
    name = [k for k, v in info.items() if v["rows"] > 1][0]
    vec = [k for k, v in info.items() if v["rows"] == 1][0]
    src = info[vec]["ptr"]    # any other device address will do for the fake backend
    for src_layout in (0, 1):
        fake.reset()
        m.load_param(name, src, src_layout)
        tr = fake.trace()
        assert len(tr) == 1 and tr[0]["C"] == info[name]["ptr"] and tr[0]["A"] == src
        want = "weight_tile" if weight_layout == 2 else ("memcpy_d2d" if src_layout == weight_layout else "transpose")
        assert tr[0]["name"] == want, (weight_layout, src_layout, tr[0]["name"])
    fake.reset()
    m.load_param(vec, info[name]["ptr"], 0)
    assert [t["name"] for t in fake.trace()] == ["memcpy_d2d"]
    with pytest.raises(Exception, match="src_layout"):
        m.load_param(name, src, 2)
    with pytest.raises(Exception, match="itself"):
        m.load_param(name, info[name]["ptr"], 0)
    with pytest.raises(KeyError):
        m.load_param("no_such_parameter", src, 0)
    m.close()
    g = host.Model(1, 2, 32, 4, 64, ffn_inner=512, fused=True, ffn_act=host.FFN_GEGLU, weight_layout=weight_layout)
    gi = g.param_info()
    inter = [k for k, v in gi.items() if v["interleave16"] and v["rows"] > 1][0]
    with pytest.raises(Exception, match="interleaved"):
        g.load_param(inter, gi[vec]["ptr"], 0)
    g.close()


def test_closing_a_scheduler_and_a_model_releases_streams_and_memory(fake):
    """Every stream holds a hardware queue on the GPU, so schedulers must give theirs back: the two streams of the
    constructor, the four CU-masked streams of the share in use (asking for another share releases the previous four), the
    request contexts and the decode batch's buffers."""
    host, lib = fake.host, fake.lib
    s0, a0 = lib.fake_live_streams(), lib.fake_live_allocs()
    m = host.Model(1, 9, 64, 4, 64, layer_num=2, ffn_inner=512, fused=True, max_cache_len=96)
    s1, a1 = lib.fake_live_streams(), lib.fake_live_allocs()
    assert s1 == s0 + 1 and a1 > a0
    sch = host.Scheduler(m, pool_count=4, ctx_batch=2)
    assert lib.fake_live_streams() == s1 + 2
    sch.enable_partition(64)
    assert lib.fake_live_streams() == s1 + 6
    sch.enable_partition(0)
    sch.enable_partition(64)                      # off and on again: the same four streams
    assert lib.fake_live_streams() == s1 + 6
    sch.enable_partition(128)                     # another share: the previous four are released first
    assert lib.fake_live_streams() == s1 + 6
    sch.enable_batch_decode(True, 2)
    sch.profile(2, 32, 64, 32, 1)
    sch.profile_decode(2, 32, 1)
    sch.serve(2, 32, 2)
    sch.run_queued(host.MODE_LIGER)
    assert lib.fake_live_allocs() > a1
    sch.close()
    assert (lib.fake_live_streams(), lib.fake_live_allocs()) == (s1, a1)
    sch.close()                                   # closing twice is harmless
    m.close()
    assert (lib.fake_live_streams(), lib.fake_live_allocs()) == (s0, a0)
