"""The scheduler on the real GPU: interleaved and decomposed launches must not change any request's result."""
import ctypes as C
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def host(liger):
    return importlib.import_module("24ppopp-liger_amd.host")


def ctx_output(dev, sched, model, i, rows, H):
    """(scheduler's output for context i, plain sequential run of the same input)"""
    pin, pout = sched.ctx_ptrs(i)
    got = torch.empty(rows, H, device="cuda", dtype=torch.float16)
    dev.capi.call("lg_memcpy_d2d_async", got.data_ptr(), pout, rows * H * 2, None)
    return got, pin


@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("fused", [False, True])
def test_interleaved_decomposed_requests_match_sequential(dev, host, axis, fused):
    """Two prefill requests under the resource-class policy with a hand-made profile that forces the second request's
    GEMMs to be split (and re-split) into the first one's LayerNorm windows.  Each request's output must equal a plain
    in-order run of the same input: pieces tile the GEMM outputs exactly and streams are ordered.  A piece may take a
    kernel that sums K in slices where the whole GEMM does not (or the other way round), so single outputs may differ by
    the rounding of one fp32 summation order (and what that becomes two layers later), never by more."""
    B, S, heads, d, F = 2, 128, 8, 128, 2048
    H = heads * d
    m = host.Model(1, 2 * B, S, heads, d, layer_num=2, ffn_inner=F, causal=True, fused=fused, factor=8, seed=11)
    s = host.Scheduler(m, contention_factor=0.8, policy=host.POLICY_RESOURCE, axis=axis, ignore_num=0, pool_count=2, ctx_batch=B)
    kpl = m.kernels_per_layer()
    desc = m.describe(B, S)[:kpl]
    for e in desc:
        if e["type"] == "GEMM":
            s.set_profile(e["idx"], B, S, 1.0, sub=[0.125 * (i + 1) for i in range(7)])
        elif e["class"] == "HBM_BOUND":
            s.set_profile(e["idx"], B, S, 2.2)     # window 0.8 * 2.2 = 1.76: one whole GEMM + 6/8 of the next
        else:
            s.set_profile(e["idx"], B, S, 0.3)
    s.serve(B, S)
    s.serve(B, S)
    r = s.run_queued(host.MODE_LIGER)
    assert r["records"] == 2 and r["secondary_launches"] > 0 and r["splits"] > 0
    torch.cuda.synchronize()
    for i in range(2):
        got, pin = ctx_output(dev, s, m, i, B * S, H)
        ref = torch.empty_like(got)
        m.run(pin, ref.data_ptr(), B, S, None, dev.stream)
        torch.cuda.synchronize()
        diff = (got.float() - ref.float()).abs()
        assert float(diff.max()) <= 4e-3 * float(ref.float().abs().max()), "request %d differs from its sequential run" % i


def test_prefill_plus_decode_trace_on_gpu(dev, host):
    """Requests with decode steps, profiled on the device, replayed in real time in both modes."""
    heads, d, F = 8, 128, 2048
    m = host.Model(1, 4, 128, heads, d, layer_num=2, ffn_inner=F, causal=True, fused=True, max_cache_len=192, factor=4, weight_layout=1, seed=5)
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS, seq_bucket=32, ignore_num=0, pool_count=4, ctx_batch=1)
    s.profile(1, 64, 128, 32, 3)
    for past in (64, 96, 128, 160):
        s.profile_decode(1, past, 3)
    assert s.lookup(0, 1, 128) > 0 and s.lookup(1004, 1, 128) > 0
    trace = [{"arrival_s": 0.001 * i, "batch": 1, "seq": 64 + 32 * (i % 3), "n_decode": 4} for i in range(10)]
    for mode in (host.MODE_SEQUENTIAL, host.MODE_LIGER):
        r = s.run_trace(trace, mode)
        assert r["records"] == 10 and r["profile_misses"] == 0
        assert r["avg_latency_ms"] > 0 and r["p99_latency_ms"] >= r["avg_latency_ms"] * 0.5


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("partition", [0, 128])
def test_batched_decode_equals_every_request_on_its_own(dev, host, mode, partition):
    """Requests of different prompt lengths and decode lengths, all in flight at once: with batched decode steps (and the
    prefills interleaved into them, optionally on a CU partition) every request must end with the hidden state it gets when it
    runs alone, step by step, on the same model.  A step over several rows may take another weight-streaming kernel than a step
    over one row (which rows share a step depends on the timing of the run), so every step may differ by the rounding of the
    fp32 summation order, and a later step starts from the earlier steps' differences.  This is a free-running comparison of
    two GPU runs: both sides round to fp16 after every kernel, a difference of one fp16 unit in a step's output (2^-11
    relative, about 1e-3 of the largest output after LayerNorm) enters the next step as an input perturbation, and up to 12
    steps x 2 layers compound.  The step-by-step check against the oracle is
    test_batched_decode_steps_teacher_forced_against_the_oracle (1e-2 at every step); here a fixed 2e-2 bounds the drift."""
    if mode == 0 and partition:
        pytest.skip("partitioned rounds belong to the interleaving scheduler")
    heads, d, F, layers, pool = 8, 128, 2048, 2, 6
    H = heads * d
    m = host.Model(1, pool + 1, 128, heads, d, layer_num=layers, ffn_inner=F, causal=True, fused=True, max_cache_len=192, factor=4,
                   weight_layout=1, seed=5)
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS, seq_bucket=32, ignore_num=0, pool_count=pool, ctx_batch=1)
    s.profile(1, 32, 128, 32, 3)
    for bs in (1, 2, 4, 6):
        for past in (32, 64, 96, 128, 160):
            s.profile_decode(bs, past, 3)
    s.set_merge_minor(True)
    s.enable_batch_decode(True, 2)
    if partition:
        s.enable_partition(partition)
        s.set_partition_factor(0, 1, 1.0)     # every co-running round is partitioned, whatever a measurement would say
        s.set_partition_factor(1, 0, 1.0)
    reqs = [(1, 96, 7), (1, 33, 12), (1, 128, 3), (1, 64, 9), (1, 50, 1), (1, 120, 10)]
    for r in reqs:
        s.serve(*r)
    rep = s.run_queued(host.MODE_LIGER if mode else host.MODE_SEQUENTIAL)
    torch.cuda.synchronize()
    assert rep["records"] == len(reqs) and rep["profile_misses"] == 0
    assert rep["batched_steps"] < sum(n for _, _, n in reqs)
    if partition and mode:
        assert rep["partition_rounds"] > 0
    worst = 0.0
    for i, (_, S, n) in enumerate(reqs):
        pin, pout = s.ctx_ptrs(i)
        da, db = s.ctx_decode_ptrs(i)
        got = torch.empty(H, device="cuda", dtype=torch.float16)
        dev.capi.call("lg_memcpy_d2d_async", got.data_ptr(), db if n % 2 else da, H * 2, None)
        # the request alone: prefill into its context's cache slot, then n single steps
        y = torch.empty(S, H, device="cuda", dtype=torch.float16)
        torch.cuda.synchronize()
        m.run(pin, y.data_ptr(), 1, S, None, None, cache_slot=i)     # on the model's own stream
        torch.cuda.synchronize()
        a = y[S - 1:S].clone()
        b = torch.empty_like(a)
        torch.cuda.synchronize()
        for t in range(n):
            m.run_decode(a.data_ptr(), b.data_ptr(), 1, S + t, i, None, None)
            a, b = b, a
        torch.cuda.synchronize()
        ref = a[0].float()
        err = float((got.float() - ref).abs().max() / ref.abs().max())
        worst = max(worst, err)
        assert err < 2e-2, "request %d (prompt %d, %d steps): max rel err %g" % (i, S, n, err)
    print("free-running batched decode vs. per-request steps: worst max-rel %.3g" % worst)


@pytest.mark.parametrize("mode", [0, 1])
def test_chunked_prefills_between_batched_decode_steps_equal_every_request_on_its_own(dev, host, mode):
    """Prompts longer than prefill_chunk are prefilled in chunks over their cache slots, with the batched decode step taking the
    turn between two chunks: every request must still end with the hidden state it gets when it runs alone (whole-prompt
    prefill, then its decode steps one by one).  Chunks change the summation order of the attention (another split of the
    keys into tiles of the online softmax), and batched steps that of the decode GEMMs: a fixed 2e-2 bounds the free-running
    drift over up to 10 steps x 2 layers, as in the unchunked test."""
    heads, d, F, layers, pool = 8, 128, 2048, 2, 6
    H = heads * d
    m = host.Model(1, pool + 1, 128, heads, d, layer_num=layers, ffn_inner=F, causal=True, fused=True, max_cache_len=192, factor=4,
                   weight_layout=2, seed=5)
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS, seq_bucket=16, ignore_num=0, pool_count=pool, ctx_batch=1)
    s.profile(1, 16, 128, 16, 3)
    for bs in (1, 2, 4, 6):
        for past in (32, 64, 96, 128, 160):
            s.profile_decode(bs, past, 3)
    s.set_merge_minor(True)
    s.enable_batch_decode(True, 2)
    s.set_prefill_chunk(48)
    reqs = [(1, 96, 7), (1, 33, 10), (1, 128, 3), (1, 64, 9), (1, 50, 1), (1, 120, 10)]
    for r in reqs:
        s.serve(*r)
    rep = s.run_queued(host.MODE_LIGER if mode else host.MODE_SEQUENTIAL)
    torch.cuda.synchronize()
    cc = s.chunk_counters()
    assert rep["records"] == len(reqs) and cc["chunked_prefills"] == 5 and cc["yield_turns"] > 0
    worst = 0.0
    for i, (_, S, n) in enumerate(reqs):
        pin, pout = s.ctx_ptrs(i)
        da, db = s.ctx_decode_ptrs(i)
        got = torch.empty(H, device="cuda", dtype=torch.float16)
        dev.capi.call("lg_memcpy_d2d_async", got.data_ptr(), db if n % 2 else da, H * 2, None)
        y = torch.empty(S, H, device="cuda", dtype=torch.float16)
        torch.cuda.synchronize()
        # the prompt's hidden states, as the scheduler left them, against the whole-prompt prefill
        mine = _read(dev, pout, S * H).reshape(S, H)
        m.run(pin, y.data_ptr(), 1, S, None, None, cache_slot=i)
        torch.cuda.synchronize()
        e_pre = float((mine - y.float()).abs().max() / y.float().abs().max())
        assert e_pre < 4e-3, "request %d: chunked prefill differs from the whole-prompt prefill (%g)" % (i, e_pre)
        a = y[S - 1:S].clone()
        b = torch.empty_like(a)
        for t in range(n):
            m.run_decode(a.data_ptr(), b.data_ptr(), 1, S + t, i, None, None)
            a, b = b, a
        torch.cuda.synchronize()
        ref = a[0].float()
        err = float((got.float() - ref).abs().max() / ref.abs().max())
        worst = max(worst, err)
        assert err < 2e-2, "request %d (prompt %d, %d steps): max rel err %g" % (i, S, n, err)
    print("chunked prefills + batched decode vs. per-request runs: worst max-rel %.3g" % worst)
    s.close()


@pytest.mark.parametrize("weight_layout", [0, 1, 2])
@pytest.mark.parametrize("mode", [0, 1])
def test_batched_decode_steps_teacher_forced_against_the_oracle(dev, po, host, mode, weight_layout):
    """Batched decode steps through the scheduler (join -> step -> retire vectors built from the requests in flight),
    checked against the CPU oracle at EVERY step: after the kernels of a step the hook compares each live row with the
    oracle's decoder step over that request's own cache (two stacked layers) and writes the oracle's rounded row back, so the
    next step starts from the oracle's state on both sides and no step inherits an earlier step's rounding.  Requests have
    different prompt and decode lengths, so the batch changes composition while it runs; the bound is the stated 1e-2 at
    every step, and the element-wise figure is held to the same 1e-2."""
    from tests.conftest import elementwise_err, max_rel_err
    heads, d, F, layers, pool, Lmax = 8, 128, 2048, 2, 5, 128
    H = heads * d
    m = host.Model(1, pool + 1, 64, heads, d, layer_num=layers, ffn_inner=F, causal=True, fused=True, max_cache_len=Lmax, factor=4,
                   weight_layout=weight_layout, seed=9)
    P = m.download_params()
    W = [{k[len("layer%d." % l):]: v for k, v in P.items() if k.startswith("layer%d." % l)} for l in range(layers)]
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS, seq_bucket=32, ignore_num=0, pool_count=pool, ctx_batch=1)
    s.profile(1, 32, 64, 32, 3)
    for bs in (1, 2, 3, 4, 5):
        for past in (32, 64, 96):
            s.profile_decode(bs, past, 3)
    s.set_merge_minor(True)
    s.enable_batch_decode(True, 2)
    s.set_recycle_contexts(False)
    reqs = [(1, 48, 9), (1, 33, 12), (1, 64, 8), (1, 40, 3), (1, 57, 10)]
    # oracle side: every request's prompt goes through the two layers; K and V of each layer's input fill its caches
    caches, state = [], {}
    for i, (_, S, n) in enumerate(reqs):
        x = _read(dev, s.ctx_ptrs(i)[0], S * H).cpu().numpy().reshape(S, H)
        shape = dict(batch=1, seq=S, hidden=H, head_num=heads, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=1)
        per_layer = []
        for l in range(layers):
            k = po.gemm(x, W[l]["wk"], 1)
            v = po.gemm(x, W[l]["wv"], 1)
            _, kb, vb = po.add_qkv_bias_transpose(k, W[l]["bk"], k, W[l]["bk"], v, W[l]["bv"], 1, S, heads, d, 1)
            kc = np.zeros((1, heads, Lmax, d), dtype=np.float32)
            vc = np.zeros_like(kc)
            kc[:, :, :S] = kb
            vc[:, :, :S] = vb
            per_layer.append((kc, vc))
            x = po.round_f16(po.encoder_forward(shape, W[l], x))
        caches.append(per_layer)
        state[i] = x[S - 1:S].copy()          # the oracle's own last prompt row: the first decode input if the GPU's agrees
    worst = {"rel": 0.0, "elem": 0.0, "steps": 0, "rows": 0, "first": 0.0}
    failures = []
    row_bytes = H * 2

    def hook(step, slots, pasts, rows_ptr, stream):
        dev.capi.call("lg_stream_synchronize", stream)
        got = _read(dev, rows_ptr, len(slots) * H).cpu().numpy().reshape(len(slots), H)
        forced = got.copy()
        for r, (slot, past) in enumerate(zip(slots, pasts)):
            if slot >= pool:
                continue                       # a row of no request
            _, S, n = reqs[slot]
            if past == S:                      # first step: the row was joined from the GPU's own prefill output
                gpu_in = _read(dev, s.ctx_ptrs(slot)[1] + (S - 1) * row_bytes, H).cpu().numpy().reshape(1, H)
                worst["first"] = max(worst["first"], max_rel_err(gpu_in, state[slot]))
                state[slot] = gpu_in
            x = state[slot]
            shape = dict(batch=1, seq=S, hidden=H, head_num=heads, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=1)
            for l in range(layers):
                x = po.round_f16(po.decoder_step(shape, W[l], x, caches[slot][l][0], caches[slot][l][1], past))
            e1, e2 = max_rel_err(got[r:r + 1], x), elementwise_err(got[r:r + 1], x)
            worst["rel"], worst["elem"] = max(worst["rel"], e1), max(worst["elem"], e2)
            worst["rows"] += 1
            if e1 >= 1e-2 or e2 >= 1e-2:
                failures.append((step, slot, past, e1, e2))
            state[slot] = x
            forced[r] = x[0]
        t = torch.from_numpy(forced).cuda().half()
        dev.capi.call("lg_memcpy_d2d_async", rows_ptr, t.data_ptr(), t.numel() * 2, stream)
        dev.capi.call("lg_stream_synchronize", stream)
        worst["steps"] += 1

    s.set_decode_step_hook(hook)
    for r in reqs:
        s.serve(*r)
    rep = s.run_queued(host.MODE_LIGER if mode else host.MODE_SEQUENTIAL)
    s.set_decode_step_hook(None)
    torch.cuda.synchronize()
    print("teacher-forced batched decode: %d steps, %d rows, worst max-rel %.3g, worst element-wise %.3g, prefill rows %.3g"
          % (worst["steps"], worst["rows"], worst["rel"], worst["elem"], worst["first"]))
    assert rep["records"] == len(reqs) and rep["profile_misses"] == 0
    assert worst["steps"] == rep["batched_steps"] >= max(n for _, _, n in reqs) >= 8
    assert worst["rows"] == sum(n for _, _, n in reqs)
    assert not failures, "steps beyond 1e-2 (step, slot, cached, max-rel, element-wise): %s" % failures[:5]
    assert worst["first"] < 1e-2
    # what the requests end with is the forced (oracle) state of their last step: the copy-out comes after the hook
    for i, (_, S, n) in enumerate(reqs):
        da, db = s.ctx_decode_ptrs(i)
        out = _read(dev, db if n % 2 else da, H).cpu().numpy().reshape(1, H)
        assert np.array_equal(out, state[i])
    s.close()


CFG = dict(hidden=12288, heads_global=96, d=128, ffn_global=32768, world_size=2)   # GLM-130B, one TP=2 shard


def _read(dev, ptr, elems):
    t = torch.empty(elems, device="cuda", dtype=torch.float16)
    dev.capi.call("lg_memcpy_d2d_async", t.data_ptr(), ptr, elems * 2, None)
    torch.cuda.synchronize()
    return t.float()


@pytest.mark.parametrize("weight_layout", [0, 1, 2])
def test_cfg4_decomposition_sweep_at_its_real_shapes(dev, host, weight_layout):
    """BASELINE config 4: a prefill request of batch 4 x seq 512 on the TP=2 layer shard, decomposed by 1, 2, 4 and 8 along
    its token rows and interleaved on two streams with a decode batch of 32 sequences at 1024 cached positions (3 steps, so
    that the prefill does not fit the decode window whole and something has to be split).  Durations come from profiling on
    the device.  For every factor both requests must end with the result of their sequential run: the pieces of a split
    GEMM tile its output exactly, and the two streams are ordered.  A piece of at most 256 token rows may sum K in slices
    where the whole GEMM does not, so values may differ by the rounding of one fp32 summation order."""
    c = CFG
    H = c["hidden"]
    m = host.Model(1, 64, 512, c["heads_global"], c["d"], layer_num=1, world_size=c["world_size"], ffn_inner=c["ffn_global"], causal=True,
                   fused=True, max_cache_len=1024 + 64, weight_layout=weight_layout, seed=0)
    s = host.Scheduler(m, schedule_deep=6, contention_factor=0.8, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS, seq_bucket=64,
                       ignore_num=0, pool_count=2, ctx_batch=32)
    s.set_merge_minor(True)
    s.profile_decode(32, 1024, 5)

    tokens = _read(dev, s.ctx_decode_ptrs(0)[0], 32 * H).half()   # the decode request's input rows (its steps overwrite them)

    def run(mode):
        dev.capi.call("lg_memcpy_d2d_async", s.ctx_decode_ptrs(0)[0], tokens.data_ptr(), 32 * H * 2, None)
        torch.cuda.synchronize()
        s.serve_decode(32, 1000, 3)       # context 0
        s.serve(4, 512, 0)                # context 1
        r = s.run_queued(mode)
        torch.cuda.synchronize()
        assert r["records"] == 2 and r["profile_misses"] == 0
        return r, _read(dev, s.ctx_decode_ptrs(0)[1], 32 * H), _read(dev, s.ctx_ptrs(1)[1], 4 * 512 * H)

    s.profile(4, 512, 512, 1, 5)
    _, dec_ref, pre_ref = run(host.MODE_SEQUENTIAL)
    assert bool(torch.isfinite(dec_ref).all()) and bool(torch.isfinite(pre_ref).all())
    for factor in (1, 2, 4, 8):
        s.set_factor(factor)
        s.profile(4, 512, 512, 1, 5)      # durations of the whole GEMMs and of their 1/f .. (f-1)/f pieces
        # The decode request's three steps open one window.  Its budget is set so that the prefill's attention block fits and
        # 0.62 of FFN-1 is left: FFN-1 does not fit whole, half of it does -- whatever this GPU's timings are today.
        step_ms = sum(s.lookup(1000 + j, 32, 1024) for j in range(m.kernels_per_layer(decode=True)))
        d = [s.lookup(j, 4, 512) for j in range(m.kernels_per_layer())]
        assert [e["label"] for e in m.describe(4, 512)][6] == "ffn1+bias+gelu" and step_ms > 0 and min(d) > 0
        s.set_contention(1, 0, (sum(d[:6]) + 0.62 * d[6]) / (3 * step_ms))
        r, dec, pre = run(host.MODE_LIGER)
        assert r["secondary_launches"] > 0
        assert (r["splits"] > 0) == (factor > 1), "factor %d: %d splits" % (factor, r["splits"])
        assert r["sub_profile_misses"] == 0
        for name, got, ref in (("decode", dec, dec_ref), ("prefill", pre, pre_ref)):
            err = float((got - ref).abs().max() / ref.abs().max())
            print("cfg4 factor %d, layout %d: %s request %.3g" % (factor, weight_layout, name, err))
            assert err < 4e-3, "factor %d: the %s request differs from its sequential run (%g)" % (factor, name, err)
    # the same on a CU partition (128 units for the HBM-bound side): results unchanged
    s.enable_partition(128)
    s.set_partition_factor(0, 1, 1.0)
    s.set_partition_factor(1, 0, 1.0)
    r, dec, pre = run(host.MODE_LIGER)
    assert r["partition_rounds"] > 0
    e_dec, e_pre = float((dec - dec_ref).abs().max() / dec_ref.abs().max()), float((pre - pre_ref).abs().max() / pre_ref.abs().max())
    print("cfg4 on a 128-unit partition, layout %d: decode request %.3g, prefill request %.3g of the sequential run's largest output" % (weight_layout, e_dec, e_pre))
    # On a share of the compute units the weight-streaming blocks are dealt other runs of tiles, and a block starts its walk
    # over k at the chunk (block index mod chunks): every output is still one fp32 sum over all of k, but in a rotated order,
    # so fp16 roundings flip here and there and three free-running steps carry them on (3-4.3e-3 observed in all layouts).
    assert e_dec < 8e-3 and e_pre < 4e-3


@pytest.mark.parametrize("packed_qkv", [False, True])
def test_cfg5_mixed_trace_at_its_real_shapes(dev, host, packed_qkv):
    """BASELINE config 5, shortened: 12 Poisson arrivals at 16 requests/s through 4 stacked TP=2 layer shards, prompts uniform
    in [128, 1024] (rounded to 64), 32 decode tokens each, durations profiled on the device.  Every request must end with the
    hidden state of its sequential run -- with interleaving, and with interleaving plus batched decode steps (where a step over
    several rows may take another weight-streaming kernel than a step over one row: rounding of the fp32 summation order)."""
    c = CFG
    H, n = c["hidden"], 12
    m = host.Model(1, n + 1, 1024, c["heads_global"], c["d"], layer_num=4, world_size=c["world_size"], ffn_inner=c["ffn_global"], causal=True,
                   fused=True, max_cache_len=1024 + 64, weight_layout=1, factor=8, seed=0, packed_qkv=packed_qkv)
    s = host.Scheduler(m, schedule_deep=6, contention_factor=0.8, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS, seq_bucket=64,
                       ignore_num=0, pool_count=n, ctx_batch=1)
    s.profile(1, 128, 1024, 64, 3)
    for bs in (1, 2, 3, 4, 6, 8, 12):
        for past in range(128, 1024 + 64 + 1, 64):
            s.profile_decode(bs, min(past, 1024 + 63), 3)
    s.set_merge_minor(True)
    s.set_recycle_contexts(False)         # request i keeps context i: its result stays readable after the run
    trace = host.make_poisson_trace(16.0, n, 1, 128, 1024, 64, 32, 0)
    gaps = np.diff([0.0] + [t["arrival_s"] for t in trace])
    assert all(128 <= t["seq"] <= 1024 and t["seq"] % 64 == 0 for t in trace) and 0.02 < gaps.mean() < 0.2

    def run(mode, batched):
        s.enable_batch_decode(batched, 2)
        r = s.run_trace(trace, mode)
        torch.cuda.synchronize()
        assert r["records"] == n and r["profile_misses"] == 0
        return r, [_read(dev, s.ctx_decode_ptrs(i)[0], H) for i in range(n)]   # 32 steps: the last state is in the first buffer

    _, ref = run(host.MODE_SEQUENTIAL, False)
    assert all(bool(torch.isfinite(x).all()) for x in ref)
    r_on, on = run(host.MODE_LIGER, False)
    r_b, batched = run(host.MODE_LIGER, True)
    assert r_b["batched_steps"] > 0
    for i in range(n):
        e1 = float((on[i] - ref[i]).abs().max() / ref[i].abs().max())
        e2 = float((batched[i] - ref[i]).abs().max() / ref[i].abs().max())
        assert e1 < 4e-3, "request %d (prompt %d) differs from its sequential run with interleaving: %g" % (i, trace[i]["seq"], e1)
        assert e2 < 1e-2, "request %d (prompt %d) differs from its sequential run with batched decode steps: %g" % (i, trace[i]["seq"], e2)
    assert r_b["avg_e2e_ms"] > 0 and r_on["avg_e2e_ms"] > 0


def test_measured_contention_on_gpu(dev, host):
    """The contention measurement runs on the device, yields a fraction in [0.05, 1] consistent with its three times, and
    a trace scheduled with the measured table completes like one scheduled with the constant."""
    heads, d, F = 8, 128, 2048
    m = host.Model(1, 4, 128, heads, d, layer_num=2, ffn_inner=F, causal=True, fused=True, max_cache_len=192, factor=4, weight_layout=1, seed=5)
    s = host.Scheduler(m, policy=host.POLICY_RESOURCE, axis=host.SPLIT_TOKEN_ROWS, seq_bucket=32, ignore_num=0, pool_count=4, ctx_batch=1)
    r = s.profile_contention(1, 128, 1, 128)
    assert r["main_ms"] > 0 and r["sub_ms"] > 0 and r["both_ms"] > 0 and r["sub_repeats"] >= 1
    assert r["both_ms"] <= (r["main_ms"] + r["sub_ms"]) * 1.5
    hidden = (r["main_ms"] + r["sub_ms"] - r["both_ms"]) / r["sub_ms"]
    assert r["hidden"] == pytest.approx(min(1.0, max(0.05, hidden)), rel=1e-4)
    assert s.contention(0, 1) == pytest.approx(r["hidden"])
    s.profile(1, 64, 128, 32, 3)
    for past in (64, 96, 128, 160):
        s.profile_decode(1, past, 3)
    trace = [{"arrival_s": 0.001 * i, "batch": 1, "seq": 64 + 32 * (i % 3), "n_decode": 4} for i in range(10)]
    rr = s.run_trace(trace, host.MODE_LIGER)
    assert rr["records"] == 10 and rr["profile_misses"] == 0


def test_command_line_driver_runs_both_modes(tmp_path):
    """The C++ driver (counterpart of the reference's main.cu): profile, serve the reference's own request generator with
    interleaving and without, print the report.  Run as a child process in a scratch directory (it writes the two
    profile JSON files there under the reference's file-name convention)."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "24ppopp-liger_amd", "lib", "liger_main")
    assert os.path.exists(exe), "liger_main is not built; run __graft_entry__.build()"
    #            max_batch max_seq heads d layers factor rate world requests
    args = [exe, "2", "64", "8", "128", "1", "4", "400", "1", "30"]
    r = subprocess.run(args, cwd=str(tmp_path), capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "---- run_stream_sync ----" in r.stdout and "---- run_sequential ----" in r.stdout
    assert r.stdout.count("Average Latency") == 2 and r.stdout.count("Throughput") == 2
    assert os.path.exists(tmp_path / "Main_1_128_8_2_64.json") and os.path.exists(tmp_path / "Sub_1_128_8_2_64.json")
