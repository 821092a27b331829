"""GPU parity for the GEMM entry points (cuBLAS-convention C ABI) against the CPU oracle."""
import numpy as np
import pytest

from tests.conftest import max_rel_err

pytestmark = pytest.mark.gpu
SUF = {0: "f32", 1: "f16"}


def rnd(po, n, tid, dt, std=1.0):
    return po.fill_normal(n, 0, tid, 0.0, std, dt)


# (tokens, out_features, k): aligned, ragged, tiny, skinny (decode-like)
SHAPES = [(64, 256, 256), (128, 128, 32), (130, 136, 72), (1, 8, 8), (33, 70, 19), (32, 1024, 512), (257, 96, 1000),
          (512, 384, 160),
          # multiples of the 256 x 256 x 64 tile: the pipelined kernel
          (256, 256, 64), (512, 768, 256), (256, 512, 1024), (1024, 2048, 192), (2048, 256, 128),
          # 256 x 192 tiles (weights stored [out, in] only) and 256 x 128 tiles (both layouts)
          (256, 384, 128), (512, 576, 192), (256, 1344, 64), (256, 640, 128), (512, 128, 192), (768, 1152, 320),
          # tile counts that take the region mappings of the workgroups: 8 x 32 tiles and 16 x 48 tiles
          (2048, 8192, 64), (4096, 12288, 64),
          # token counts that are not a multiple of the tile: the pipelined kernel pads the last row of tiles
          (320, 256, 128), (448, 384, 192), (1000, 512, 256), (200, 256, 64), (161, 768, 128), (65, 256, 192), (100, 384, 64),
          # few tokens, many features: the weight-streaming split-K kernel (weights stored [out, in])
          (32, 1024, 2048), (1, 512, 1024), (17, 640, 4104), (64, 2048, 1536), (33, 516, 1032),
          # ... and enough features for unsliced blocks: 64 features per block (any M <= 64, K % 512 == 0), 32 per block
          # (M <= 16, K % 1024 == 0); N not a multiple of the block width
          (32, 12288, 1024), (48, 12292, 1536), (64, 12352, 512), (5, 12288, 512), (9, 6148, 2048), (16, 6144, 1024),
          # one to four token rows and K a multiple of 2048: the matrix-vector kernel (weights stored [out, in])
          (1, 512, 2048), (2, 1024, 4096), (3, 256, 2048), (4, 644, 6144), (1, 6144, 12288)]


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("transa", [0, 1])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_gemm(dev, po, dt, transa, M, N, K):
    """Row-major Y[M,N] = X[M,K] W, called as cublasGemmEx(transa, N, m=N, n=M, k=K, A=W, B=X, C=Y)."""
    X = rnd(po, M * K, 30, dt).reshape(M, K)
    W = rnd(po, K * N, 31, dt, 0.05).reshape(K, N)
    ref = po.gemm(X, W, dt)
    if transa:
        A = np.ascontiguousarray(W.T)  # [N, K] row-major == column-major k x m with lda = K
        lda = K
    else:
        A = W                          # [K, N] row-major == column-major m x k with lda = N
        lda = N
    dA, dX = dev.up(A, dt), dev.up(X, dt)
    dY = dev.empty((M, N), dt)
    dev.call("lg_gemm_" + SUF[dt], transa, 0, N, M, K, dA, lda, dX, K, dY, N)
    assert max_rel_err(dev.down(dY), ref) < (2e-5 if dt == 0 else 2e-3)
    # the oracle's own cuBLAS-convention entry must agree with its row-major one
    C2 = np.zeros((M, N), dtype=np.float32)
    po.gemm_ex(transa, 0, N, M, K, A, lda, X, K, C2, N, dt)
    assert max_rel_err(C2, ref) < 1e-5


def _interleave16(n):
    """stored order of n = 2 f features [gate | up] interleaved in groups of 16: stored[p] = logical[idx[p]]"""
    p = np.arange(n)
    return (p // 32) * 16 + p % 16 + np.where(p % 32 >= 16, n // 2, 0)


# (tokens, f, k): the pipelined kernel with 256- and 128-wide tiles, the generic kernel (ragged k / tokens / f % 64 != 0),
# the weight-streaming kernels (few tokens; one slice and several), a single token row
GEGLU_SHAPES = [(512, 512, 256), (256, 192, 128), (300, 1024, 192), (70, 48, 72), (130, 16, 40), (32, 2048, 1024),
                (32, 256, 2048), (8, 8192, 512), (1, 512, 2048), (64, 1024, 1536), (4096, 256, 64)]


@pytest.mark.parametrize("transa", [0, 1])
@pytest.mark.parametrize("M,F,K", GEGLU_SHAPES)
def test_gemm_geglu_epilogue(dev, po, transa, M, F, K):
    """FFN-1 of a GeGLU MLP with the product formed in the GEMM's epilogue: the weight [K, 2F] = [gate | up] and its bias are
    handed over with gate and up interleaved in groups of 16 features, the result [M, F] must equal the oracle's
    GEMM -> bias + GeGLU on the plain operands."""
    X = rnd(po, M * K, 40, 1).reshape(M, K)
    W = rnd(po, K * 2 * F, 41, 1, 0.05).reshape(K, 2 * F)
    bias = rnd(po, 2 * F, 42, 1, 0.3)
    ref = po.add_bias_geglu(po.gemm(X, W, 1), bias, 1)
    idx = _interleave16(2 * F)
    Ws, bs = np.ascontiguousarray(W[:, idx]), np.ascontiguousarray(bias[idx])
    A, lda = (np.ascontiguousarray(Ws.T), K) if transa else (Ws, 2 * F)
    dY = dev.empty((M, F), 1)
    dev.call("lg_gemm_fused_f16", transa, 2 * F, M, K, dev.up(A, 1), lda, dev.up(X, 1), K, dY, F, 5, dev.up(bs, 1), 0, 0, 0)
    assert max_rel_err(dev.down(dY), ref) < 4e-3
    # a wider destination (ldc > f) leaves the columns beyond f alone
    wide = dev.up(np.full((M, F + 8), 7.0, dtype=np.float32), 1)
    dev.call("lg_gemm_fused_f16", transa, 2 * F, M, K, dev.up(A, 1), lda, dev.up(X, 1), K, wide, F + 8, 5, dev.up(bs, 1), 0, 0, 0)
    got = dev.down(wide)
    assert np.all(got[:, F:] == 7.0) and max_rel_err(got[:, :F], ref) < 4e-3


@pytest.mark.parametrize("transa", [0, 1])
def test_gemm_geglu_subrange_concatenation_is_exact(dev, po, transa):
    """Decomposition of a GeGLU FFN-1 (decompose_callback: whole groups of 32 stored features = 16 output columns; weight
    and bias move by c0 features, the output by c0 / 2 columns; token rows as for any GEMM): the pieces reproduce the full
    call bit for bit."""
    M, F, K = 512, 768, 256
    X = rnd(po, M * K, 43, 1).reshape(M, K)
    Ws = rnd(po, K * 2 * F, 44, 1, 0.05).reshape(K, 2 * F)      # already in the stored (interleaved) order
    bs = rnd(po, 2 * F, 45, 1, 0.3)
    dX, dB = dev.up(X, 1), dev.up(bs, 1)
    dW = dev.up(np.ascontiguousarray(Ws.T) if transa else Ws, 1)
    lda = K if transa else 2 * F
    full = dev.empty((M, F), 1)
    dev.call("lg_gemm_fused_f16", transa, 2 * F, M, K, dW, lda, dX, K, full, F, 5, dB, 0, 0, 0)
    # stored features split at 3/8 (a multiple of 32)
    c0 = (2 * F * 3 // 8) // 32 * 32
    cols = dev.empty((M, F), 1)
    wstep = c0 * K * 2 if transa else c0 * 2
    dev.call("lg_gemm_fused_f16", transa, c0, M, K, dW, lda, dX, K, cols, F, 5, dB, 0, 0, 0)
    dev.call("lg_gemm_fused_f16", transa, 2 * F - c0, M, K, dW.data_ptr() + wstep, lda, dX, K, cols.data_ptr() + (c0 // 2) * 2, F, 5,
             dB.data_ptr() + c0 * 2, 0, 0, 0)
    assert np.array_equal(dev.down(cols), dev.down(full))
    # token rows split at 5/8 (both pieces above 256 rows: every output stays one sequential sum over k)
    rows = dev.empty((M, F), 1)
    m1 = 320
    dev.call("lg_gemm_fused_f16", transa, 2 * F, m1, K, dW, lda, dX, K, rows, F, 5, dB, 0, 0, 0)
    dev.call("lg_gemm_fused_f16", transa, 2 * F, M - m1, K, dW, lda, dX.data_ptr() + m1 * K * 2, K, rows.data_ptr() + m1 * F * 2, F, 5, dB, 0, 0, 0)
    got, ref = dev.down(rows), dev.down(full)
    assert np.array_equal(got[:m1], ref[:m1]) and max_rel_err(got[m1:], ref[m1:]) < 1e-3   # 192 rows may slice K


def test_gemm_geglu_epilogue_rejects_bad_shapes(dev):
    x = dev.empty((4, 64), 1)
    w = dev.empty((48, 64), 1)
    y = dev.empty((4, 24), 1)
    b = dev.empty((48,), 1)
    with pytest.raises(dev.capi.LigerError):   # features not a multiple of 32
        dev.call("lg_gemm_fused_f16", 1, 48, 4, 64, w, 64, x, 64, y, 24, 5, b, 0, 0, 0)
    w2, b2 = dev.empty((64, 64), 1), dev.empty((64,), 1)
    with pytest.raises(dev.capi.LigerError):   # ldc below features / 2
        dev.call("lg_gemm_fused_f16", 1, 64, 4, 64, w2, 64, x, 64, y, 24, 5, b2, 0, 0, 0)
    with pytest.raises(dev.capi.LigerError):   # no bias
        dev.call("lg_gemm_fused_f16", 1, 64, 4, 64, w2, 64, x, 64, y, 32, 5, None, 0, 0, 0)


@pytest.mark.parametrize("dt", [0, 1])
def test_gemm_subrange_concatenation_is_exact(dev, po, dt):
    """Decomposition invariant: computing column slices / row slices of Y separately (pointer offsets, same
    leading dimensions) reproduces the full product bit for bit (the K order is unchanged)."""
    M, N, K = 256, 512, 320
    X = rnd(po, M * K, 32, dt).reshape(M, K)
    W = rnd(po, K * N, 33, dt, 0.05).reshape(K, N)
    dW, dX = dev.up(W, dt), dev.up(X, dt)
    full = dev.empty((M, N), dt)
    s = SUF[dt]
    es = 4 if dt == 0 else 2
    dev.call("lg_gemm_" + s, 0, 0, N, M, K, dW, N, dX, K, full, N)
    # split output features (the reference's axis, utils.h:218-260) at 3/8
    cols = dev.empty((M, N), dt)
    n1 = N * 3 // 8
    dev.call("lg_gemm_" + s, 0, 0, n1, M, K, dW, N, dX, K, cols, N)
    dev.call("lg_gemm_" + s, 0, 0, N - n1, M, K, dW.data_ptr() + n1 * es, N, dX, K, cols.data_ptr() + n1 * es, N)
    assert np.array_equal(dev.down(cols), dev.down(full))
    # split token rows at 5/8
    rows = dev.empty((M, N), dt)
    m1 = M * 5 // 8
    dev.call("lg_gemm_" + s, 0, 0, N, m1, K, dW, N, dX, K, rows, N)
    dev.call("lg_gemm_" + s, 0, 0, N, M - m1, K, dW, N, dX.data_ptr() + m1 * K * es, K, rows.data_ptr() + m1 * N * es, N)
    assert np.array_equal(dev.down(rows), dev.down(full))


@pytest.mark.parametrize("dt", [0, 1])
@pytest.mark.parametrize("B,h,S,d", [(2, 4, 32, 64), (1, 3, 80, 128), (1, 2, 33, 24)])
def test_attention_batched_gemms(dev, po, dt, B, h, S, d):
    """qk_gemm and qkv_gemm exactly as bert_layer.h:145-163 issues them."""
    nb = B * h
    q = rnd(po, nb * S * d, 34, dt).reshape(nb, S, d)
    k = rnd(po, nb * S * d, 35, dt).reshape(nb, S, d)
    v = rnd(po, nb * S * d, 36, dt).reshape(nb, S, d)
    s = SUF[dt]
    ref_qk = np.zeros((nb, S, S), dtype=np.float32)
    po.gemm_strided_batched(1, 0, S, S, d, k, d, S * d, q, d, S * d, ref_qk, S, S * S, nb, dt)
    assert max_rel_err(ref_qk, np.einsum("bqd,bkd->bqk", q.astype(np.float64), k.astype(np.float64))) < 2e-3
    dq, dk, dv = dev.up(q, dt), dev.up(k, dt), dev.up(v, dt)
    dqk = dev.empty((nb, S, S), dt)
    dev.call("lg_gemm_strided_batched_" + s, 1, 0, S, S, d, dk, d, S * d, dq, d, S * d, dqk, S, S * S, nb)
    assert max_rel_err(dev.down(dqk), ref_qk) < (2e-5 if dt == 0 else 2e-3)
    p = np.abs(ref_qk) / np.abs(ref_qk).sum(-1, keepdims=True)
    p = po.round_f16(p) if dt else p
    ref_o = np.zeros((nb, S, d), dtype=np.float32)
    po.gemm_strided_batched(0, 0, d, S, S, v, d, S * d, p, S, S * S, ref_o, d, S * d, nb, dt)
    do = dev.empty((nb, S, d), dt)
    dev.call("lg_gemm_strided_batched_" + s, 0, 0, d, S, S, dv, d, S * d, dev.up(p, dt), S, S * S, do, d, S * d, nb)
    assert max_rel_err(dev.down(do), ref_o) < (2e-5 if dt == 0 else 2e-3)


@pytest.mark.parametrize("transa", [0, 1])
def test_gemm_fused_epilogues(dev, po, transa):
    B, S, h, d, K = 2, 48, 4, 64, 192
    M, N = B * S, h * d
    X = rnd(po, M * K, 37, 1).reshape(M, K)
    W = rnd(po, K * N, 38, 1, 0.05).reshape(K, N)
    bias = rnd(po, N, 39, 1, 0.3)
    A, lda = (np.ascontiguousarray(W.T), K) if transa else (W, N)
    dA, dX, dB = dev.up(A, 1), dev.up(X, 1), dev.up(bias, 1)
    # two-kernel references on the GPU itself and from the oracle
    y = po.gemm(X, W, 1)
    ref_gelu = po.add_bias_gelu(y.copy(), bias, 1)
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", transa, N, M, K, dA, lda, dX, K, out, N, dev.capi.EPI_BIAS_GELU, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), ref_gelu) < 4e-3
    ref_heads, _, _ = po.add_qkv_bias_transpose(y, bias, y, bias, y, bias, B, S, h, d, 1)
    out = dev.empty((B, h, S, d), 1)
    dev.call("lg_gemm_fused_f16", transa, N, M, K, dA, lda, dX, K, out, S, dev.capi.EPI_BIAS_HEADS, dB, S, d, 0)
    assert max_rel_err(dev.down(out), ref_heads) < 2e-3
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", transa, N, M, K, dA, lda, dX, K, out, N, dev.capi.EPI_BIAS, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), po.round_f16(y + bias)) < 2e-3


@pytest.mark.parametrize("transa", [0, 1])
def test_gemm_fused_epilogues_on_the_pipelined_kernel(dev, po, transa):
    """Same epilogues on a tile-aligned problem (256-multiples), which takes the pipelined kernel, incl. a column slice
    written into a wider head-transposed destination (the decomposition case)."""
    B, S, h, d, K = 2, 256, 4, 128, 320
    M, N = B * S, h * d
    X = rnd(po, M * K, 40, 1).reshape(M, K)
    W = rnd(po, K * N, 41, 1, 0.05).reshape(K, N)
    bias = rnd(po, N, 42, 1, 0.3)
    A, lda = (np.ascontiguousarray(W.T), K) if transa else (W, N)
    dA, dX, dB = dev.up(A, 1), dev.up(X, 1), dev.up(bias, 1)
    y = po.gemm(X, W, 1)
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", transa, N, M, K, dA, lda, dX, K, out, N, dev.capi.EPI_BIAS_GELU, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), po.add_bias_gelu(y.copy(), bias, 1)) < 4e-3
    ref_heads, _, _ = po.add_qkv_bias_transpose(y, bias, y, bias, y, bias, B, S, h, d, 1)
    rows = S + 32  # destination reserves more rows per (batch, head) than the sequence has (a KV cache)
    out = dev.empty((B, h, rows, d), 1)
    out.zero_()
    half = N // 2
    es = 2
    a_off = (half * K if transa else half) * es
    dev.call("lg_gemm_fused_f16", transa, half, M, K, dA, lda, dX, K, out, rows, dev.capi.EPI_BIAS_HEADS, dB, S, d, h)
    dev.call("lg_gemm_fused_f16", transa, N - half, M, K, dA.data_ptr() + a_off, lda, dX, K,
             out.data_ptr() + (half // d) * rows * d * es, rows, dev.capi.EPI_BIAS_HEADS, dB.data_ptr() + half * es, S, d, h)
    got = dev.down(out)
    assert max_rel_err(got[:, :, :S], ref_heads) < 2e-3
    assert np.all(got[:, :, S:] == 0)


@pytest.mark.parametrize("M", [1, 2, 4])
def test_gemm_fused_epilogues_on_the_matrix_vector_kernel(dev, po, M):
    """Decode-shaped calls (a few token rows, weights [out, in]): bias + GELU and the head-transposed store into a
    KV-cache-shaped destination with more rows per head than tokens."""
    h, d, K = 6, 128, 4096
    N = h * d
    X = rnd(po, M * K, 43, 1).reshape(M, K)
    W = rnd(po, K * N, 44, 1, 0.05).reshape(K, N)
    bias = rnd(po, N, 45, 1, 0.3)
    dA, dX, dB = dev.up(np.ascontiguousarray(W.T), 1), dev.up(X, 1), dev.up(bias, 1)
    y = po.gemm(X, W, 1)
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", 1, N, M, K, dA, K, dX, K, out, N, dev.capi.EPI_BIAS_GELU, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), po.add_bias_gelu(y.copy(), bias, 1)) < 4e-3
    # one token per sequence (batch = M, seq = 1) written to row 0 of a [M, h, rows, d] destination
    ref_heads, _, _ = po.add_qkv_bias_transpose(y, bias, y, bias, y, bias, M, 1, h, d, 1)
    rows = 5
    out = dev.empty((M, h, rows, d), 1)
    out.zero_()
    dev.call("lg_gemm_fused_f16", 1, N, M, K, dA, K, dX, K, out, rows, dev.capi.EPI_BIAS_HEADS, dB, 1, d, h)
    got = dev.down(out)
    assert max_rel_err(got[:, :, :1], ref_heads) < 2e-3
    assert np.all(got[:, :, 1:] == 0)


@pytest.mark.parametrize("M,h", [(8, 96), (32, 96), (40, 16), (12, 48)])
def test_gemm_fused_epilogues_on_the_weight_streaming_kernels(dev, po, M, h):
    """5..64 token rows, weights [out, in]: h = 96 takes the blocks that walk the whole of K and apply the epilogue
    themselves (64 features per block), h = 48 with <= 16 rows the 32-feature blocks, h = 16 the K-sliced kernel whose
    second kernel applies it."""
    d, K = 128, 1024
    N = h * d
    X = rnd(po, M * K, 46, 1).reshape(M, K)
    W = rnd(po, K * N, 47, 1, 0.05).reshape(K, N)
    bias = rnd(po, N, 48, 1, 0.3)
    dA, dX, dB = dev.up(np.ascontiguousarray(W.T), 1), dev.up(X, 1), dev.up(bias, 1)
    y = po.gemm(X, W, 1)
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", 1, N, M, K, dA, K, dX, K, out, N, dev.capi.EPI_BIAS_GELU, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), po.add_bias_gelu(y.copy(), bias, 1)) < 4e-3
    out = dev.empty((M, N), 1)
    dev.call("lg_gemm_fused_f16", 1, N, M, K, dA, K, dX, K, out, N, dev.capi.EPI_BIAS, dB, 0, 0, 0)
    assert max_rel_err(dev.down(out), po.round_f16(y + bias)) < 2e-3
    # one token per sequence (batch = M, seq = 1) written to row 2 of a [M, h, rows, d] destination (a KV cache)
    ref_heads, _, _ = po.add_qkv_bias_transpose(y, bias, y, bias, y, bias, M, 1, h, d, 1)
    rows = 4
    out = dev.empty((M, h, rows, d), 1)
    out.zero_()
    dev.call("lg_gemm_fused_f16", 1, N, M, K, dA, K, dX, K, out.data_ptr() + 2 * d * 2, rows, dev.capi.EPI_BIAS_HEADS, dB, 1, d, h)
    got = dev.down(out)
    assert max_rel_err(got[:, :, 2:3], ref_heads) < 2e-3
    assert np.all(got[:, :, :2] == 0) and np.all(got[:, :, 3:] == 0)


@pytest.mark.parametrize("M,transa", [(1, 1), (3, 1), (8, 1), (32, 1), (64, 1), (100, 1), (8, 0)])
def test_grouped_qkv_gemm_equals_three_plain_calls(dev, po, M, transa):
    """The grouped entry (Q, K and V projections of a decode step as one call) must return what three plain fused calls
    return: one launch of the matrix-vector / weight-streaming kernels for few token rows and weights [out, in] (bit for
    bit on the matrix-vector kernel; the weight-streaming kernel may choose another block width for the group and then
    sums k in another order), three plain calls otherwise (bit for bit).  Q goes to [M, h, 1, d], K and V to row `past`
    of cache-shaped buffers."""
    import ctypes as C
    h, d, K, rows, past = 48, 128, 2048, 6, 3
    N = h * d
    X = rnd(po, M * K, 50, 1).reshape(M, K)
    dX = dev.up(X, 1)
    Ws = [rnd(po, K * N, 51 + t, 1, 0.05).reshape(K, N) for t in range(3)]
    bs = [rnd(po, N, 54 + t, 1, 0.3) for t in range(3)]
    dA = [dev.up(np.ascontiguousarray(W.T) if transa else W, 1) for W in Ws]
    dB = [dev.up(b, 1) for b in bs]
    lda = K if transa else N
    ldc = [1, rows, rows]

    def outputs():
        o = [dev.empty((M, h, 1, d), 1), dev.empty((M, h, rows, d), 1), dev.empty((M, h, rows, d), 1)]
        for t in o:
            t.zero_()
        return o

    def dst(o, t):
        return o[t].data_ptr() + (past * d * 2 if t else 0)

    plain = outputs()
    for t in range(3):
        dev.call("lg_gemm_fused_f16", transa, N, M, K, dA[t], lda, dX, K, dst(plain, t), ldc[t], dev.capi.EPI_BIAS_HEADS, dB[t], 1, d, h)
    grouped = outputs()
    arr = lambda ptrs: (C.c_void_p * 3)(*ptrs)
    dev.call("lg_gemm_fused_grouped_f16", transa, N, M, K, 3, arr([a.data_ptr() for a in dA]), lda, dX, K,
             arr([dst(grouped, t) for t in range(3)]), (C.c_int * 3)(*ldc), dev.capi.EPI_BIAS_HEADS,
             arr([b.data_ptr() for b in dB]), 1, d, h)
    for t in range(3):
        if transa == 0 or M <= 4 or M > 64:
            assert np.array_equal(dev.down(grouped[t]), dev.down(plain[t]))
        else:
            assert max_rel_err(dev.down(grouped[t]), dev.down(plain[t])) < 1e-3
    y = po.gemm(X, Ws[1], 1)
    ref, _, _ = po.add_qkv_bias_transpose(y, bs[1], y, bs[1], y, bs[1], M, 1, h, d, 1)
    got = dev.down(grouped[1])
    assert max_rel_err(got[:, :, past:past + 1], ref) < 2e-3
    assert np.all(got[:, :, :past] == 0) and np.all(got[:, :, past + 1:] == 0)
    # a null member is reported, nothing is launched
    bad = arr([dA[0].data_ptr(), 0, dA[2].data_ptr()])
    assert dev.call_rc("lg_gemm_fused_grouped_f16", transa, N, M, K, 3, bad, lda, dX, K, arr([dst(grouped, t) for t in range(3)]),
                       (C.c_int * 3)(*ldc), dev.capi.EPI_BIAS_HEADS, arr([b.data_ptr() for b in dB]), 1, d, h) != 0


@pytest.mark.parametrize("transa", [0, 1])
@pytest.mark.parametrize("B,S,h,d", [(4, 128, 6, 128), (2, 384, 4, 64), (3, 100, 8, 96), (8, 512, 16, 128), (8, 512, 48, 128)])
def test_grouped_qkv_gemm_on_a_packed_weight_prefill(dev, po, transa, B, S, h, d):
    """Q, K and V of a prefill as one grouped call on the column blocks of ONE packed [K, 3 N] weight (the pointers of the
    members are offsets into it, lda is the packed matrix's): with more than 256 token rows the pipelined kernel runs the
    group as one launch where the members' tiles side by side need fewer rounds of workgroups than each member's own, else
    member by member (the last shape: 4096 rows x 2048 features fill one round per member with 128-wide tiles, three
    members together would need three; the one after it, 4096 rows x 6144 features, runs as Q and K in one launch and V in two
    pieces, whole rounds of 256-wide tiles and a last round of 128-wide ones); either way the result must equal three plain
    fused calls bit for bit (same tiles, same k order) and the oracle.  q goes to [B, h, S, d], k and v into cache-shaped buffers with more rows than S."""
    import ctypes as C
    K, rows = 512, S + 24
    N, M = h * d, B * S
    X = rnd(po, M * K, 70, 1).reshape(M, K)
    W = rnd(po, K * 3 * N, 71, 1, 0.05).reshape(K, 3 * N)
    bias = rnd(po, 3 * N, 72, 1, 0.3)
    dX, dB = dev.up(X, 1), dev.up(bias, 1)
    dW = dev.up(np.ascontiguousarray(W.T) if transa else W, 1)
    lda = K if transa else 3 * N
    step = N * K * 2 if transa else N * 2       # bytes between the members inside the packed weight
    A = [dW.data_ptr() + t * step for t in range(3)]
    bp = [dB.data_ptr() + t * N * 2 for t in range(3)]
    ldc = [S, rows, rows]

    def outputs():
        o = [dev.empty((B, h, S, d), 1), dev.empty((B, h, rows, d), 1), dev.empty((B, h, rows, d), 1)]
        for t in o:
            t.zero_()
        return o

    plain, grouped = outputs(), outputs()
    for t in range(3):
        dev.call("lg_gemm_fused_f16", transa, N, M, K, A[t], lda, dX, K, plain[t], ldc[t], dev.capi.EPI_BIAS_HEADS, bp[t], S, d, h)
    arr = lambda ptrs: (C.c_void_p * 3)(*ptrs)
    dev.call("lg_gemm_fused_grouped_f16", transa, N, M, K, 3, arr(A), lda, dX, K, arr([g.data_ptr() for g in grouped]),
             (C.c_int * 3)(*ldc), dev.capi.EPI_BIAS_HEADS, arr(bp), S, d, h)
    for t in range(3):
        got = dev.down(grouped[t])
        assert np.array_equal(got, dev.down(plain[t]))
        y = po.round_f16(po.gemm(X, np.ascontiguousarray(W[:, t * N:(t + 1) * N]), 1) + bias[t * N:(t + 1) * N])
        ref = y.reshape(B, S, h, d).transpose(0, 2, 1, 3)
        assert max_rel_err(got[:, :, :S], ref) < 4e-3
        assert np.all(got[:, :, S:] == 0)


@pytest.mark.parametrize("M,count,epi", [(1, 2, "bias"), (4, 1, "gelu"), (16, 2, "bias"), (40, 3, "none"), (16, 3, "gelu")])
def test_grouped_gemm_other_epilogues_and_counts(dev, po, M, count, epi):
    """Groups of one, two and three problems with the plain, bias and bias + GELU epilogues and different leading
    dimensions of the outputs: equal to the plain fused calls (up to the fp32 summation order on the weight-streaming
    kernel) and to the oracle."""
    import ctypes as C
    N, K = 6144, 2048
    kind = {"none": dev.capi.EPI_NONE, "bias": dev.capi.EPI_BIAS, "gelu": dev.capi.EPI_BIAS_GELU}[epi]
    X = rnd(po, M * K, 60, 1).reshape(M, K)
    dX = dev.up(X, 1)
    Ws = [rnd(po, K * N, 61 + t, 1, 0.05).reshape(K, N) for t in range(count)]
    bs = [rnd(po, N, 64 + t, 1, 0.3) for t in range(count)]
    dA = [dev.up(np.ascontiguousarray(W.T), 1) for W in Ws]
    dB = [dev.up(b, 1) for b in bs]
    ldc = [N + 8 * t for t in range(count)]          # outputs with padded rows
    plain = [dev.empty((M, ldc[t]), 1) for t in range(count)]
    grouped = [dev.empty((M, ldc[t]), 1) for t in range(count)]
    for t in plain + grouped:
        t.zero_()
    for t in range(count):
        dev.call("lg_gemm_fused_f16", 1, N, M, K, dA[t], K, dX, K, plain[t], ldc[t], kind, dB[t] if epi != "none" else None, 0, 0, 0)
    arr = lambda ptrs: (C.c_void_p * count)(*ptrs)
    dev.call("lg_gemm_fused_grouped_f16", 1, N, M, K, count, arr([a.data_ptr() for a in dA]), K, dX, K,
             arr([g.data_ptr() for g in grouped]), (C.c_int * count)(*ldc), kind,
             arr([b.data_ptr() for b in dB]) if epi != "none" else None, 0, 0, 0)
    for t in range(count):
        got, ref_gpu = dev.down(grouped[t]), dev.down(plain[t])
        assert np.all(got[:, N:] == 0)                                   # the padding is not written
        if M <= 4:
            assert np.array_equal(got, ref_gpu)
        else:
            assert max_rel_err(got, ref_gpu) < 1e-3
        y = po.gemm(X, Ws[t], 1)
        ref = y if epi == "none" else (po.round_f16(y + bs[t]) if epi == "bias" else po.add_bias_gelu(y.copy(), bs[t], 1))
        assert max_rel_err(got[:, :N], ref) < 4e-3


@pytest.mark.parametrize("M,N,K,transa", [(3, 1024, 2048, 1), (12, 6144, 2048, 1), (40, 6144, 4096, 1), (5, 512, 512, 1), (6, 1024, 2048, 0)])
def test_grouped_gemm_with_a_destination_per_token_row(dev, po, M, N, K, transa):
    """Q, K and V of a decode step whose sequences sit in arbitrary cache slots at different positions: q goes to row r, the
    K and V rows of token r to (slot[r], head, pos[r]) of a cache [slots, heads, rows, d].  Shapes for the matrix-vector
    kernel (M <= 4), the weight-streaming kernel, and the plain-call fallback (small N, or weights stored [in, out]).  Checked
    against the oracle's GEMM + bias scattered by numpy, bit-for-bit untouched elsewhere."""
    import ctypes as C
    d = 128
    h = N // d
    slots, rows = 7, 24
    X = rnd(po, M * K, 80, 1).reshape(M, K)
    Ws = [rnd(po, K * N, 81 + t, 1, 0.05).reshape(K, N) for t in range(3)]
    bs = [rnd(po, N, 84 + t, 1, 0.3) for t in range(3)]
    dA = [dev.up(np.ascontiguousarray(W.T) if transa else W, 1) for W in Ws]
    dB = [dev.up(b, 1) for b in bs]
    dX = dev.up(X, 1)
    cells = [(11 * r + 5) % (slots * rows) for r in range(M)]      # distinct (slot, position) cells, scattered
    slot, pos = [c % slots for c in cells], [c // slots for c in cells]
    q = dev.empty((M, h, d), 1); q.zero_()
    kc0 = rnd(po, slots * h * rows * d, 90, 1).reshape(slots, h, rows, d)
    vc0 = rnd(po, slots * h * rows * d, 91, 1).reshape(slots, h, rows, d)
    dkc, dvc = dev.up(kc0, 1), dev.up(vc0, 1)
    arr = lambda ptrs: (C.c_void_p * 3)(*ptrs)
    lda = K if transa else N
    dev.call("lg_gemm_fused_grouped_rows_f16", transa, N, M, K, 3, arr([a.data_ptr() for a in dA]), lda, dX, K,
             arr([q.data_ptr(), dkc.data_ptr(), dvc.data_ptr()]), (C.c_int * 3)(1, rows, rows), arr([b.data_ptr() for b in dB]),
             d, h, (C.c_int * 3)(0, 1, 1), (C.c_int * M)(*slot), (C.c_int * M)(*pos))
    ref = [po.round_f16(po.gemm(X, Ws[t], 1) + bs[t]).reshape(M, h, d) for t in range(3)]
    assert max_rel_err(dev.down(q), ref[0]) < 4e-3
    for got, base, want in ((dev.down(dkc), kc0, ref[1]), (dev.down(dvc), vc0, ref[2])):
        exp = base.copy()
        touched = np.zeros(base.shape[:3], dtype=bool)
        for r in range(M):
            exp[slot[r], :, pos[r], :] = want[r]
            touched[slot[r], :, pos[r]] = True
        assert np.array_equal(got[~touched], base[~touched]), "rows other than the addressed ones were written"
        assert max_rel_err(got[touched], exp[touched]) < 4e-3
    # rows outside the destination are refused on the host
    bad = (C.c_int * M)(*([rows] + pos[1:]))
    assert dev.call_rc("lg_gemm_fused_grouped_rows_f16", transa, N, M, K, 3, arr([a.data_ptr() for a in dA]), lda, dX, K,
                       arr([q.data_ptr(), dkc.data_ptr(), dvc.data_ptr()]), (C.c_int * 3)(1, rows, rows), arr([b.data_ptr() for b in dB]),
                       d, h, (C.c_int * 3)(0, 1, 1), (C.c_int * M)(*slot), bad) == dev.capi.ERR_INVALID
