"""GPU parity for weights in the tiled layout (transa = LG_OP_TILED: 16-feature x 32-k fragment blocks, lg_weight_tile_f16).

Every kernel that can take such weights is checked against the CPU oracle on the plain operands, and against the same call on
the plain [out, in] weights where both must sum k in the same order (bit for bit)."""
import ctypes as C

import numpy as np
import pytest

from tests.conftest import max_rel_err

pytestmark = pytest.mark.gpu
TILED = 2


def rnd(po, n, tid, std=1.0):
    return po.fill_normal(n, 0, tid, 0.0, std, 1)


def tile_host(a):
    """[features, k] -> tiled storage order (numpy restatement of the layout: block (t, c) = 512 elements at
    (t * k / 32 + c) * 512, element (f, j) of a block at ((j // 8) * 16 + f) * 8 + j % 8)."""
    n, k = a.shape
    out = np.empty(n * k, dtype=a.dtype)
    for t in range(n // 16):
        for c in range(k // 32):
            blk = a[16 * t:16 * t + 16, 32 * c:32 * c + 32]          # [f, j]
            out[(t * (k // 32) + c) * 512:(t * (k // 32) + c + 1) * 512] = blk.reshape(16, 4, 8).transpose(1, 0, 2).reshape(-1)
    return out


@pytest.mark.parametrize("plain_transa", [0, 1])
@pytest.mark.parametrize("N,K", [(16, 32), (48, 96), (256, 4096), (6144, 1024)])
def test_tile_and_untile_are_the_documented_permutation(dev, po, N, K, plain_transa):
    w = rnd(po, N * K, 70).reshape(N, K)                               # logical [features, k]
    plain = w if plain_transa else np.ascontiguousarray(w.T)
    ld = K if plain_transa else N
    dp = dev.up(plain, 1)
    dt = dev.empty((N * K,), 1)
    dev.call("lg_weight_tile_f16", dt, dp, N, K, plain_transa, ld)
    assert np.array_equal(dev.down(dt), tile_host(po.round_f16(w)))
    back = dev.empty(plain.shape, 1)
    back.zero_()
    dev.call("lg_weight_untile_f16", back, dt, N, K, plain_transa, ld)
    assert np.array_equal(dev.down(back), po.round_f16(plain))


def test_tile_rejects_what_the_layout_cannot_hold(dev):
    a, b = dev.empty((64 * 64,), 1), dev.empty((64 * 64,), 1)
    for (n, k) in ((24, 64), (32, 48)):
        assert dev.call_rc("lg_weight_tile_f16", a, b, n, k, 1, k) == dev.capi.ERR_INVALID
    assert dev.call_rc("lg_weight_tile_f16", a, a, 32, 64, 1, 64) == dev.capi.ERR_INVALID       # in place
    assert dev.call_rc("lg_gemm_f16", TILED, 0, 24, 8, 64, a, 64, b, 64, a, 24) == dev.capi.ERR_INVALID
    assert dev.call_rc("lg_gemm_f16", TILED, 0, 32, 8, 64, a, 72, b, 64, a, 32) == dev.capi.ERR_INVALID   # lda != k
    f = dev.empty((64 * 64,), 0)
    assert dev.call_rc("lg_gemm_f32", TILED, 0, 32, 8, 64, f, 64, f, 64, f, 32) == dev.capi.ERR_INVALID   # an fp16 layout


# (tokens, features, k): generic kernel (small, ragged token counts), pipelined kernel at its three tile widths and with a
# partial last row of tiles, one row of tiles with K-slices, unsliced weight-streaming blocks of 3..8 waves at 1..64 rows
# (a whole chip has 256 compute units: 12288 features = 768 tiles = 3 waves a block), too few features for those (generic)
SHAPES = [(64, 256, 256), (1, 16, 32), (33, 80, 96), (130, 144, 160), (257, 96, 1024),
          (256, 256, 64), (512, 768, 256), (1024, 2048, 192), (256, 384, 128), (512, 576, 192), (256, 640, 128), (768, 1152, 320),
          (2048, 8192, 64), (4096, 12288, 64), (320, 256, 128), (1000, 512, 256), (161, 768, 128), (65, 256, 192),
          (128, 1024, 2048), (200, 512, 4096),
          (32, 12288, 1024), (48, 12304, 1536), (64, 16384, 512), (5, 12288, 512), (16, 6144, 1024), (1, 6144, 2048), (3, 8192, 1024),
          (32, 20480, 512), (8, 32768, 512), (32, 1024, 2048), (17, 640, 4096)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_gemm_on_tiled_weights(dev, po, M, N, K):
    X = rnd(po, M * K, 71).reshape(M, K)
    W = rnd(po, K * N, 72, 0.05).reshape(K, N)
    ref = po.gemm(X, W, 1)
    dWt = dev.up(np.ascontiguousarray(W.T), 1)                         # [features, k]
    dT = dev.empty((N * K,), 1)
    dev.call("lg_weight_tile_f16", dT, dWt, N, K, 1, K)
    dX = dev.up(X, 1)
    dY = dev.empty((M, N), 1)
    dev.call("lg_gemm_f16", TILED, 0, N, M, K, dT, K, dX, K, dY, N)
    got = dev.down(dY)
    assert max_rel_err(got, ref) < 2e-3
    # Above 256 token rows every output is one sequential fp32 sum over k in both layouts; at 5..64 rows the unsliced
    # weight-streaming blocks are the same code in both.  There the two layouts must agree bit for bit.
    if M > 256 or (5 <= M <= 64 and N >= 6144):
        dY2 = dev.empty((M, N), 1)
        dev.call("lg_gemm_f16", 1, 0, N, M, K, dWt, K, dX, K, dY2, N)
        assert np.array_equal(dev.down(dY2), got)


@pytest.mark.parametrize("M,S", [(512, 256), (32, 1), (2, 1), (96, 48)])
def test_fused_epilogues_and_subranges_on_tiled_weights(dev, po, M, S):
    """Bias, bias + GELU and the head-transposed store, and the two halves of the features computed separately (the piece
    starts at a whole 16-feature tile, (first feature) * k elements into the tiled matrix) into one destination."""
    h, d, K = 48, 128, 512
    N, B = h * d, M // S
    X = rnd(po, M * K, 73).reshape(M, K)
    W = rnd(po, K * N, 74, 0.05).reshape(K, N)
    bias = rnd(po, N, 75, 0.3)
    dT = dev.empty((N * K,), 1)
    dev.call("lg_weight_tile_f16", dT, dev.up(np.ascontiguousarray(W.T), 1), N, K, 1, K)
    dX, dB = dev.up(X, 1), dev.up(bias, 1)
    y = po.gemm(X, W, 1)
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", TILED, N, M, K, dT, K, dX, K, out, N, dev.capi.EPI_BIAS_GELU, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), po.add_bias_gelu(y.copy(), bias, 1)) < 4e-3
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", TILED, N, M, K, dT, K, dX, K, out, N, dev.capi.EPI_BIAS, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), po.round_f16(y + bias)) < 2e-3
    ref_heads, _, _ = po.add_qkv_bias_transpose(y, bias, y, bias, y, bias, B, S, h, d, 1)
    rows = S + 3
    whole = dev.empty((B, h, rows, d), 1)
    whole.zero_()
    dev.call("lg_gemm_fused_f16", TILED, N, M, K, dT, K, dX, K, whole, rows, dev.capi.EPI_BIAS_HEADS, dB, S, d, h)
    got = dev.down(whole)
    assert max_rel_err(got[:, :, :S], ref_heads) < 2e-3 and np.all(got[:, :, S:] == 0)
    half = N // 2
    parts = dev.empty((B, h, rows, d), 1)
    parts.zero_()
    dev.call("lg_gemm_fused_f16", TILED, half, M, K, dT, K, dX, K, parts, rows, dev.capi.EPI_BIAS_HEADS, dB, S, d, h)
    dev.call("lg_gemm_fused_f16", TILED, N - half, M, K, dT.data_ptr() + half * K * 2, K, dX, K,
             parts.data_ptr() + (half // d) * rows * d * 2, rows, dev.capi.EPI_BIAS_HEADS, dB.data_ptr() + half * 2, S, d, h)
    assert max_rel_err(dev.down(parts)[:, :, :S], ref_heads) < 2e-3


def _interleave16(n):
    p = np.arange(n)
    return (p // 32) * 16 + p % 16 + np.where(p % 32 >= 16, n // 2, 0)


@pytest.mark.parametrize("M,F,K", [(512, 512, 256), (300, 1024, 192), (70, 48, 96), (32, 2048, 1024), (8, 8192, 512), (1, 512, 2048)])
def test_geglu_epilogue_on_tiled_weights(dev, po, M, F, K):
    X = rnd(po, M * K, 76).reshape(M, K)
    W = rnd(po, K * 2 * F, 77, 0.05).reshape(K, 2 * F)
    bias = rnd(po, 2 * F, 78, 0.3)
    ref = po.add_bias_geglu(po.gemm(X, W, 1), bias, 1)
    idx = _interleave16(2 * F)
    Ws, bs = np.ascontiguousarray(W[:, idx]), np.ascontiguousarray(bias[idx])
    dT = dev.empty((2 * F * K,), 1)
    dev.call("lg_weight_tile_f16", dT, dev.up(Ws, 1), 2 * F, K, 0, 2 * F)        # from the [k, features] matrix
    dY = dev.empty((M, F), 1)
    dev.call("lg_gemm_fused_f16", TILED, 2 * F, M, K, dT, K, dev.up(X, 1), K, dY, F, 5, dev.up(bs, 1), 0, 0, 0)
    assert max_rel_err(dev.down(dY), ref) < 4e-3


@pytest.mark.parametrize("M", [1, 8, 32, 64, 300, 4096])
def test_grouped_qkv_on_tiled_weights_equals_three_plain_calls(dev, po, M):
    """Q, K and V as one grouped call on three tiled weights -- and on the three row blocks of ONE packed tiled weight -- against
    three plain calls on the same weights; per-row destinations (rows entry) at decode sizes.  4096 rows x 6144 features is the
    shape the library runs as Q and K in one launch + V in two pieces (whole rounds of 256-wide tiles and one round of 128-wide
    ones): the pieces must land exactly where the plain calls put them."""
    h, d, K, rows, past = 48, 128, 2048, 6, 3
    N = h * d
    S = 1 if M <= 64 else M
    B = M // S
    X = rnd(po, M * K, 80).reshape(M, K)
    dX = dev.up(X, 1)
    Wp = rnd(po, K * 3 * N, 81, 0.05).reshape(K, 3 * N)                # packed [k, 3 features]
    bs = [rnd(po, N, 84 + t, 0.3) for t in range(3)]
    dP = dev.empty((3 * N * K,), 1)
    dev.call("lg_weight_tile_f16", dP, dev.up(Wp, 1), 3 * N, K, 0, 3 * N)
    dA = [dP.data_ptr() + t * N * K * 2 for t in range(3)]            # row blocks of the packed tiled weight
    dB = [dev.up(b, 1) for b in bs]
    ldc = [S, rows + S, rows + S]

    def outputs():
        o = [dev.empty((B, h, S, d), 1), dev.empty((B, h, rows + S, d), 1), dev.empty((B, h, rows + S, d), 1)]
        for t in o:
            t.zero_()
        return o

    def dst(o, t):
        return o[t].data_ptr() + (past * d * 2 if t else 0)

    arr = lambda ptrs: (C.c_void_p * 3)(*ptrs)
    plain = outputs()
    for t in range(3):
        dev.call("lg_gemm_fused_f16", TILED, N, M, K, dA[t], K, dX, K, dst(plain, t), ldc[t], dev.capi.EPI_BIAS_HEADS, dB[t], S, d, h)
    grouped = outputs()
    dev.call("lg_gemm_fused_grouped_f16", TILED, N, M, K, 3, arr(dA), K, dX, K, arr([dst(grouped, t) for t in range(3)]),
             (C.c_int * 3)(*ldc), dev.capi.EPI_BIAS_HEADS, arr([b.data_ptr() for b in dB]), S, d, h)
    for t in range(3):
        y = po.gemm(X, np.ascontiguousarray(Wp[:, t * N:(t + 1) * N]), 1)
        ref, _, _ = po.add_qkv_bias_transpose(y, bs[t], y, bs[t], y, bs[t], B, S, h, d, 1)
        got = dev.down(grouped[t])[:, :, (past if t else 0):(past if t else 0) + S]
        assert max_rel_err(got, ref) < 2e-3
        assert max_rel_err(dev.down(grouped[t]), dev.down(plain[t])) < 1e-3
        if M > 256:
            assert np.array_equal(dev.down(grouped[t]), dev.down(plain[t]))     # the pipelined kernel: same bits whatever the plan
    if M <= 64:
        # every token row to its own (slot, position) of the K / V destinations
        slots = [(5 * r + 2) % M for r in range(M)]
        pos = [(r * 3) % rows for r in range(M)]
        o = outputs()
        dev.call("lg_gemm_fused_grouped_rows_f16", TILED, N, M, K, 3, arr(dA), K, dX, K, arr([t.data_ptr() for t in o]), (C.c_int * 3)(1, rows + S, rows + S),
                 arr([b.data_ptr() for b in dB]), d, h, (C.c_int * 3)(0, 1, 1), (C.c_int * M)(*slots), (C.c_int * M)(*pos))
        for t in (1, 2):
            y = po.round_f16(po.gemm(X, np.ascontiguousarray(Wp[:, t * N:(t + 1) * N]), 1) + bs[t]).reshape(M, h, d)
            got = dev.down(o[t])
            for r in range(M):
                assert max_rel_err(got[slots[r], :, pos[r]], y[r]) < 2e-3
