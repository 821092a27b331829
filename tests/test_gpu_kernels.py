"""GPU parity: every reference-shaped kernel, called through the C ABI, against the CPU oracle.

Tolerances: fp32 kernels 2e-5 relative to the largest reference magnitude; fp16 kernels must meet the
stated bar (max rel err <= 1e-2) and are additionally held to a few fp16 ulps element-wise where the
operation is a single rounding away from the oracle.
"""
import numpy as np
import pytest

from tests.conftest import max_rel_err

pytestmark = pytest.mark.gpu

F16_TOL = 1e-2   # the stated tolerance
SUF = {0: "f32", 1: "f16"}


def rnd(po, n, tid, dt, std=1.0, mean=0.0):
    return po.fill_normal(n, 0, tid, mean, std, dt)


def tol(dt):
    return 2e-5 if dt == 0 else 2e-3


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("m,n", [(64, 256), (5, 12288), (3, 1000), (7, 37), (2, 16392), (1, 40000), (0, 64)])
def test_layer_norm(dev, po, dt, m, n):
    x = rnd(po, m * n, 1, dt).reshape(m, n) * 3 + 0.5
    x = po.round_f16(x) if dt else x
    g = rnd(po, n, 2, dt, 0.1, 1.0)
    b = rnd(po, n, 3, dt, 0.1)
    ref = po.layer_norm(x, g, b, dt)
    dx, dg, db = dev.up(x, dt), dev.up(g, dt), dev.up(b, dt)
    out = dev.empty((m, n), dt)
    dev.call("lg_layer_norm_" + SUF[dt], dx, dg, db, out, m, n)
    if m:
        assert max_rel_err(dev.down(out), ref) < tol(dt)


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("m,n", [(64, 1024), (4, 16384), (3, 100), (5, 7)])
def test_add_bias_gelu(dev, po, dt, m, n):
    x = rnd(po, m * n, 4, dt, 2.0).reshape(m, n)
    bias = rnd(po, n, 5, dt, 0.5)
    ref = po.add_bias_gelu(x.copy(), bias, dt)
    dx, dbias = dev.up(x, dt), dev.up(bias, dt)
    dev.call("lg_add_bias_act_" + SUF[dt], dx, dbias, m, n)
    assert max_rel_err(dev.down(dx), ref) < (2e-5 if dt == 0 else 4e-3)


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("m,f", [(64, 1024), (4, 16384), (3, 100), (5, 7), (0, 64)])
def test_add_bias_geglu(dev, po, dt, m, f):
    x2 = rnd(po, m * 2 * f, 9, dt, 2.0).reshape(m, 2 * f)
    bias = rnd(po, 2 * f, 10, dt, 0.5)
    out = dev.empty((m, f), dt)
    dev.call("lg_add_bias_geglu_" + SUF[dt], out, dev.up(x2, dt), dev.up(bias, dt), m, f)
    if m:
        assert max_rel_err(dev.down(out), po.add_bias_geglu(x2, bias, dt)) < (2e-5 if dt == 0 else 4e-3)


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("m,n", [(16, 256), (4, 12288), (3, 1001)])
def test_add_bias_input_layernorm_family(dev, po, dt, m, n):
    out0 = rnd(po, m * n, 6, dt).reshape(m, n)
    inp = rnd(po, m * n, 7, dt).reshape(m, n)
    bias = rnd(po, n, 8, dt, 0.2)
    g = rnd(po, n, 9, dt, 0.1, 1.0)
    b = rnd(po, n, 10, dt, 0.1)
    s = SUF[dt]
    # add_bias_input_layernorm (in place)
    ref = po.add_bias_input_layernorm(out0.copy(), inp, bias, g, b, dt)
    d_out = dev.up(out0, dt)
    dev.call("lg_add_bias_input_layernorm_" + s, d_out, dev.up(inp, dt), dev.up(bias, dt), dev.up(g, dt), dev.up(b, dt), m, n)
    assert max_rel_err(dev.down(d_out), ref) < tol(dt)
    # add_bias_input_layernorm_2 (two outputs)
    ref_sum, ref_norm = po.add_bias_input_layernorm_2(inp, g, b, bias, out0.copy(), dt)
    d_out = dev.up(out0, dt)
    d_norm = dev.empty((m, n), dt)
    dev.call("lg_add_bias_input_layernorm_2_" + s, dev.up(inp, dt), dev.up(g, dt), dev.up(b, dt), dev.up(bias, dt), d_out, d_norm, m, n)
    assert max_rel_err(dev.down(d_out), ref_sum) < tol(dt)
    assert max_rel_err(dev.down(d_norm), ref_norm) < tol(dt)
    # add_bias_input
    ref = po.add_bias_input(out0.copy(), bias, inp, dt)
    d_out = dev.up(out0, dt)
    dev.call("lg_add_bias_input_" + s, d_out, dev.up(bias, dt), dev.up(inp, dt), m, n)
    assert max_rel_err(dev.down(d_out), ref) < tol(dt)


@pytest.mark.parametrize("n", [64, 12288, 100, 33])
def test_layernorm_2_f16_row_of_near_ties(dev, po, n):
    """add_bias_input_layernorm_2 in half on a row whose every sum 1 + 2^-11 ties down to 1.0: the stored sums are all 1.0,
    the mean comes from the unrounded sums (cuda_kernels.cu:377-384), variance and output from the stored ones (:392-408),
    so every output is -u / sqrt(u^2 + 1e-6) = -0.43877 with u = 2^-11 (0 if the mean came from the stored values, -0.48828
    if the variance came from the unrounded ones).  n = 64 and 12288 take the register-cached kernel, 100 and 33 the scalar
    one."""
    u = 2.0 ** -11
    m = 5
    inp = np.ones((m, n), dtype=np.float32)
    out0 = np.full((m, n), u, dtype=np.float32)
    g, b, z = np.ones(n, dtype=np.float32), np.zeros(n, dtype=np.float32), np.zeros(n, dtype=np.float32)
    ref_sum, ref_norm = po.add_bias_input_layernorm_2(inp, g, b, z, out0.copy(), 1)
    d_out, d_norm = dev.up(out0, 1), dev.empty((m, n), 1)
    dev.call("lg_add_bias_input_layernorm_2_f16", dev.up(inp, 1), dev.up(g, 1), dev.up(b, 1), dev.up(z, 1), d_out, d_norm, m, n)
    assert np.array_equal(dev.down(d_out), ref_sum) and np.all(ref_sum == 1.0)
    got = dev.down(d_norm)
    assert np.abs(got - ref_norm).max() <= 2.0 ** -11 and np.abs(got + 0.43877).max() < 5e-4


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("B,S,h,d", [(2, 32, 4, 64), (2, 8, 12, 128), (1, 5, 3, 20), (3, 7, 2, 9)])
def test_qkv_bias_transpose_and_back(dev, po, dt, B, S, h, d):
    n = h * d
    M = B * S
    Q, K, V = (rnd(po, M * n, 11 + i, dt).reshape(M, n) for i in range(3))
    bq, bk, bv = (rnd(po, n, 14 + i, dt, 0.3) for i in range(3))
    rq, rk, rv = po.add_qkv_bias_transpose(Q, bq, K, bk, V, bv, B, S, h, d, dt)
    s = SUF[dt]
    dq, dk, dv = (dev.empty((B, h, S, d), dt) for _ in range(3))
    dev.call("lg_add_qkv_bias_transpose_" + s, dq, dk, dv, dev.up(Q, dt), dev.up(bq, dt), dev.up(K, dt), dev.up(bk, dt),
             dev.up(V, dt), dev.up(bv, dt), B, S, h, d)
    for got, ref in ((dq, rq), (dk, rk), (dv, rv)):
        assert max_rel_err(dev.down(got), ref) < tol(dt)
    # packed variant must give the same three buffers
    QKV = np.ascontiguousarray(np.stack([Q, K, V], axis=1))  # [M, 3, n]
    bias = np.concatenate([bq, bk, bv])
    fq, fk, fv = (dev.empty((B, h, S, d), dt) for _ in range(3))
    dev.call("lg_add_fused_qkv_bias_transpose_" + s, fq, fk, fv, dev.up(QKV, dt), dev.up(bias, dt), B, S, h, d)
    for got, ref in ((fq, dq), (fk, dk), (fv, dv)):
        assert np.array_equal(dev.down(got), dev.down(ref))
    # transpose back: exact permutation
    back = dev.empty((B, S, h, d), dt)
    dev.call("lg_transpose_" + s, back, dq, B, S, h, d)
    assert np.array_equal(dev.down(back), po.transpose(dev.down(dq)))


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("B,h,S,causal", [(2, 4, 32, False), (2, 3, 512, True), (1, 2, 77, True), (1, 1, 2048, False),
                                           (1, 2, 4100, True)])
def test_attn_softmax(dev, po, dt, B, h, S, causal):
    qk = rnd(po, B * h * S * S, 20, dt, 4.0).reshape(B, h, S, S)
    if causal:
        mask = np.broadcast_to(np.tril(np.ones((S, S), dtype=np.float32)), (B, S, S)).copy()
    else:
        mask = (rnd(po, B * S * S, 21, 0).reshape(B, S, S) > -1.0).astype(np.float32)
        mask[:, :, 0] = 1.0
    scalar = 1.0 / np.sqrt(64.0)
    ref = po.attn_softmax(qk.copy(), mask, scalar, dt)
    d = dev.up(qk, dt)
    dev.call("lg_attn_softmax_" + SUF[dt], d, dev.up(mask, dt), B, S, h, float(scalar))
    got = dev.down(d)
    # probabilities are <= 1; absolute error is the meaningful measure
    assert np.abs(got - ref).max() < (2e-6 if dt == 0 else 2e-3)
    assert np.abs(got.sum(-1) - 1.0).max() < (1e-4 if dt == 0 else 2e-2)


def test_error_paths(dev):
    x = dev.empty((4, 8), 0)
    assert dev.call_rc("lg_layer_norm_f32", x, x, x, x, 4, 0) == dev.capi.ERR_INVALID
    assert "bad shape" in dev.capi.last_error()
    assert dev.call_rc("lg_add_bias_act_f32", x, x, -1, 8) == dev.capi.ERR_INVALID
    assert dev.call_rc("lg_gemm_f32", 0, 1, 4, 4, 4, x, 4, x, 4, x, 4) == dev.capi.ERR_INVALID
    assert dev.call_rc("lg_gemm_f32", 0, 0, 8, 4, 8, x, 4, x, 8, x, 8) == dev.capi.ERR_INVALID  # lda < m


def test_fill_normal_matches_oracle_bitwise(dev, po):
    for dt in (0, 1):
        n = 100003
        t = dev.empty((n,), dt)
        dev.call("lg_fill_normal_" + SUF[dt], t, n, 7, 42, 0.25, 0.02)
        ref = po.fill_normal(n, 7, 42, 0.25, 0.02, dt)
        assert np.array_equal(dev.down(t), ref)


def test_cu_masked_stream_runs_kernels(dev, po):
    """A stream restricted to 32 compute units computes the same LayerNorm as any other stream; an empty mask is refused."""
    import ctypes as C
    lib = dev.lib
    m, n = 96, 1024
    x = rnd(po, m * n, 1, 0).reshape(m, n) * 3 + 0.5
    g = rnd(po, n, 2, 0, 0.1, 1.0)
    b = rnd(po, n, 3, 0, 0.1)
    ref = po.layer_norm(x, g, b, 0)
    words = (C.c_uint * 8)(0xFFFFFFFF, 0, 0, 0, 0, 0, 0, 0)
    s = C.c_void_p()
    assert lib.lg_stream_create_cu_mask(C.byref(s), words, 8) == 0, dev.capi.last_error()
    try:
        dx, dg, db = dev.up(x, 0), dev.up(g, 0), dev.up(b, 0)
        out = dev.empty((m, n), 0)
        dev.down(out)  # the uploads on the default stream are complete before the masked stream reads them
        ptr = lambda t: C.c_void_p(t.data_ptr())
        assert lib.lg_layer_norm_f32(ptr(dx), ptr(dg), ptr(db), ptr(out), m, n, s) == 0, dev.capi.last_error()
        assert lib.lg_stream_synchronize(s) == 0
        assert max_rel_err(dev.down(out), ref) < tol(0)
    finally:
        assert lib.lg_stream_destroy(s) == 0
    empty = (C.c_uint * 8)(*([0] * 8))
    s2 = C.c_void_p()
    assert lib.lg_stream_create_cu_mask(C.byref(s2), empty, 8) == 1  # LG_ERR_INVALID


def test_cu_masked_streams_that_never_ran_a_kernel_can_be_destroyed(dev):
    """The four streams of a partitioned scheduler are created together, and a run may never use some of them: creating and
    destroying CU-masked streams without submitting anything must return (the library gives each stream one empty kernel at
    creation, because destroying one that never ran anything has blocked in the runtime)."""
    import ctypes as C
    lib = dev.lib
    hbm = (C.c_uint * 8)(*([0xFFFFFFFF] * 2 + [0] * 6))     # compute units 0..63: 8 on every die
    mfma = (C.c_uint * 8)(*([0] * 2 + [0xFFFFFFFF] * 6))
    streams = []
    for words in (mfma, hbm, mfma, hbm):
        s = C.c_void_p()
        assert lib.lg_stream_create_cu_mask(C.byref(s), words, 8) == 0, dev.capi.last_error()
        streams.append(s)
    assert lib.lg_stream_cu_count(streams[0]) == 192 and lib.lg_stream_cu_count(streams[1]) == 64
    for s in streams:
        assert lib.lg_stream_destroy(s) == 0, dev.capi.last_error()


def test_second_stream_is_verified_to_run_next_to_the_first(dev, po):
    """lg_stream_create_concurrent hands out a stream whose kernels overlap with the given stream's (measured by the
    library) even when the process already holds more streams than there are hardware queues; the stream computes like any
    other; null arguments are refused."""
    import ctypes as C
    lib = dev.lib
    crowd = []
    for _ in range(6):  # more streams than the default four hardware queues of a process
        s = C.c_void_p()
        assert lib.lg_stream_create(C.byref(s)) == 0
        crowd.append(s)
    first, second, verified = crowd[2], C.c_void_p(), C.c_int(-1)
    assert lib.lg_stream_create_concurrent(C.byref(second), first, C.byref(verified)) == 0, dev.capi.last_error()
    try:
        assert verified.value in (0, 1)
        m, n = 64, 512
        x = rnd(po, m * n, 4, 0).reshape(m, n)
        g = rnd(po, n, 5, 0, 0.1, 1.0)
        b = rnd(po, n, 6, 0, 0.1)
        dx, dg, db = dev.up(x, 0), dev.up(g, 0), dev.up(b, 0)
        out = dev.empty((m, n), 0)
        dev.down(out)
        ptr = lambda t: C.c_void_p(t.data_ptr())
        assert lib.lg_layer_norm_f32(ptr(dx), ptr(dg), ptr(db), ptr(out), m, n, second) == 0, dev.capi.last_error()
        assert lib.lg_stream_synchronize(second) == 0
        assert max_rel_err(dev.down(out), po.layer_norm(x, g, b, 0)) < tol(0)
        # the probe on its own agrees with what the creation reported; one stream with itself, and a null stream, are refused
        conc = C.c_int(-1)
        assert lib.lg_streams_run_concurrently(first, second, C.byref(conc)) == 0, dev.capi.last_error()
        assert conc.value == verified.value
        assert lib.lg_streams_run_concurrently(first, first, C.byref(conc)) == 1
        assert lib.lg_streams_run_concurrently(first, None, C.byref(conc)) == 1
    finally:
        assert lib.lg_stream_destroy(second) == 0
        for s in crowd:
            assert lib.lg_stream_destroy(s) == 0
    ok = verified.value
    assert lib.lg_stream_create_concurrent(C.byref(second), None, C.byref(verified)) == 1  # LG_ERR_INVALID
    if ok != 1:
        pytest.skip("no candidate stream overlapped with the first one on this box (a single hardware queue?)")


def test_ceiling_probes_report_plausible_figures_and_refuse_bad_arguments(dev):
    """lg_probe_mfma_f16 / lg_probe_mfma_stream_f16 / lg_probe_read (measurement entries of the bench): short runs return
    figures inside what the device can do at all (no more than the published peaks, a sensible fraction of them), the matrix
    loop with operand traffic does not beat the one without, zero operands are not slower than random ones; arguments the
    kernels' indexing does not allow are refused before any launch."""
    import ctypes as C
    import torch
    lib = dev.lib
    n = 1 << 20
    ops = torch.empty(n, device="cuda", dtype=torch.float16)
    dev.call("lg_fill_normal_f16", ops, n, 0, 77, 0.0, 1.0)
    scratch = torch.zeros(64, device="cuda", dtype=torch.float32)
    dev.sync()
    ms, tf, ghz = C.c_float(), C.c_float(), C.c_float()
    ptr = lambda t: C.c_void_p(t.data_ptr())

    def mfma(stream_traffic, t, iters=400, loads=8, reads=12, elems=n):
        if stream_traffic:
            rc = lib.lg_probe_mfma_stream_f16(ptr(t), elems, ptr(scratch), 256, iters, loads, reads, C.byref(ms), C.byref(tf), C.byref(ghz), None)
        else:
            rc = lib.lg_probe_mfma_f16(ptr(t), elems, ptr(scratch), 256, iters, C.byref(ms), C.byref(tf), C.byref(ghz), None)
        return rc, tf.value, ghz.value

    rc, plain, clock = mfma(False, ops)
    assert rc == 0, dev.capi.last_error()
    assert 800.0 < plain < 2600.0 and 1.0 < clock < 2.6, (plain, clock)
    rc, zeros, _ = mfma(False, torch.zeros_like(ops))
    assert rc == 0 and zeros > 0.98 * plain and zeros < 2600.0, (zeros, plain)
    rc, streamed, clock = mfma(True, ops)
    assert rc == 0, dev.capi.last_error()
    assert 600.0 < streamed < 1.03 * plain and 1.0 < clock < 2.6, (streamed, plain, clock)
    rc, bare, _ = mfma(True, ops, loads=0, reads=0)
    assert rc == 0 and bare > streamed, (bare, streamed)
    print("matrix loop: %.0f TFLOP/s on N(0,1) operands, %.0f on zeros; with the GEMM's operand traffic %.0f, same kernel without it %.0f"
          % (plain, zeros, streamed, bare))
    assert mfma(True, ops, loads=3)[0] == 1 and mfma(True, ops, reads=5)[0] == 1          # LG_ERR_INVALID
    assert mfma(False, ops, elems=1000)[0] == 1 and mfma(True, ops, elems=1000)[0] == 1
    assert mfma(False, ops, iters=0)[0] == 1
    assert lib.lg_probe_mfma_f16(None, n, ptr(scratch), 256, 10, C.byref(ms), None, None, None) == 1
    buf = torch.empty(64 << 20, device="cuda", dtype=torch.uint8)
    gb = C.c_float()
    for nt in (0, 1):
        assert lib.lg_probe_read(ptr(buf), buf.numel(), ptr(scratch), 3, nt, C.byref(ms), C.byref(gb), None) == 0, dev.capi.last_error()
        assert 1000.0 < gb.value < 40000.0, gb.value       # 64 MiB stays in the memory-side cache: above the HBM peak is possible
    assert lib.lg_probe_read(ptr(buf), 1000, ptr(scratch), 3, 0, C.byref(ms), C.byref(gb), None) == 1
    assert lib.lg_probe_read(ptr(buf), buf.numel(), ptr(scratch), 0, 0, C.byref(ms), C.byref(gb), None) == 1
