"""ctypes binding of oracle/libliger_oracle.so (see liger_oracle.h).

TEST INFRASTRUCTURE ONLY.  All arrays are C-contiguous numpy float32; fp16 mode (dtype=1) keeps
values in float32 storage but rounds them to binary16 wherever the reference's half kernels do.
"""
import ctypes as C
import os
import subprocess

import numpy as np

F32, F16 = 0, 1
POST_NORESID, PRE_LN_RESID = 0, 1

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libliger_oracle.so")
_lib = None

_fp = C.POINTER(C.c_float)
_dp = C.POINTER(C.c_double)


class LayerWeightsC(C.Structure):
    _fields_ = [(n, _fp) for n in (
        "wq", "wk", "wv", "bq", "bk", "bv", "wo", "bo", "ln1_g", "ln1_b", "w1", "b1", "w2", "b2",
        "ln2_g", "ln2_b")]


class LayerShapeC(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "batch", "seq", "hidden", "head_num", "size_per_head", "ffn_inner", "causal", "norm_mode",
        "dtype", "ffn_act")]


def build(force=False):
    """Compile the oracle with the Makefile next to it (gcc + OpenMP)."""
    if force or not os.path.exists(_LIB_PATH) or any(
            os.path.getmtime(os.path.join(_HERE, f)) > os.path.getmtime(_LIB_PATH)
            for f in ("liger_oracle.c", "liger_oracle.h")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    i, i64, u64, f = C.c_int, C.c_int64, C.c_uint64, C.c_float
    sig = {
        "lo_round_f16": (f, [f]),
        "lo_f32_to_f16_bits": (C.c_uint16, [f]),
        "lo_f16_bits_to_f32": (f, [C.c_uint16]),
        "lo_round_f16_array": (None, [_fp, i64]),
        "lo_num_threads": (i, []),
        "lo_fill_normal": (None, [_fp, i64, u64, u64, f, f, i]),
        "lo_gemm": (None, [i, i, i, _fp, _fp, _fp, i]),
        "lo_gemm_naive_f64": (None, [i, i, i, _fp, i, _fp, i, _dp, i]),
        "lo_gemm_ex": (None, [i, i, i, i, i, _fp, i, _fp, i, _fp, i, i]),
        "lo_gemm_strided_batched": (None, [i, i, i, i, i, _fp, i, i64, _fp, i, i64, _fp, i, i64, i, i]),
        "lo_add_bias_gelu": (None, [_fp, _fp, i, i, i]),
        "lo_add_bias_geglu": (None, [_fp, _fp, _fp, i, i, i]),
        "lo_layer_norm": (None, [_fp, _fp, _fp, _fp, i, i, i]),
        "lo_add_bias_input_layernorm": (None, [_fp, _fp, _fp, _fp, _fp, i, i, i]),
        "lo_add_bias_input_layernorm_2": (None, [_fp, _fp, _fp, _fp, _fp, _fp, i, i, i]),
        "lo_add_bias_input": (None, [_fp, _fp, _fp, i, i, i]),
        "lo_add_qkv_bias_transpose": (None, [_fp] * 9 + [i, i, i, i, i]),
        "lo_add_fused_qkv_bias_transpose": (None, [_fp] * 5 + [i, i, i, i, i]),
        "lo_attn_softmax": (None, [_fp, _fp, i, i, i, f, i]),
        "lo_transpose": (None, [_fp, _fp, i, i, i, i]),
        "lo_attn_decode": (None, [_fp, _fp, _fp, _fp, i, i, i, i, i, f, i]),
        "lo_attn_prefill": (None, [_fp, _fp, _fp, _fp, i, i, i, i, f, i, i]),
        "lo_encoder_forward": (i, [C.POINTER(LayerShapeC), C.POINTER(LayerWeightsC), _fp, _fp, _fp]),
        "lo_mha_forward": (i, [C.POINTER(LayerShapeC), C.POINTER(LayerWeightsC), _fp, _fp, _fp]),
        "lo_mlp_forward": (i, [C.POINTER(LayerShapeC), C.POINTER(LayerWeightsC), _fp, _fp]),
        "lo_decoder_step": (i, [C.POINTER(LayerShapeC), C.POINTER(LayerWeightsC), _fp, _fp, _fp, i, i, _fp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _p(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], \
        "oracle arrays must be C-contiguous float32"
    return a.ctypes.data_as(_fp)


def f32(a):
    """Any array-like (incl. float16) -> fresh C-contiguous float32 array."""
    return np.array(a, dtype=np.float32, order="C", copy=True)


def round_f16(a):
    a = f32(a)
    lib().lo_round_f16_array(_p(a), a.size)
    return a


def fill_normal(n, seed, tensor_id, mean=0.0, stddev=1.0, dtype=F32):
    out = np.empty(int(n), dtype=np.float32)
    lib().lo_fill_normal(_p(out), out.size, seed, tensor_id, mean, stddev, dtype)
    return out


def gemm(X, W, dtype=F32):
    M, K = X.shape
    K2, N = W.shape
    assert K == K2
    Y = np.empty((M, N), dtype=np.float32)
    lib().lo_gemm(M, N, K, _p(X), _p(W), _p(Y), dtype)
    return Y


def gemm_naive_f64(X, W):
    M, K = X.shape
    _, N = W.shape
    Y = np.empty((M, N), dtype=np.float64)
    lib().lo_gemm_naive_f64(M, N, K, _p(X), K, _p(W), N, Y.ctypes.data_as(_dp), N)
    return Y


def gemm_ex(transa, transb, m, n, k, A, lda, B, ldb, C_, ldc, dtype=F32):
    lib().lo_gemm_ex(transa, transb, m, n, k, _p(A), lda, _p(B), ldb, _p(C_), ldc, dtype)
    return C_


def gemm_strided_batched(transa, transb, m, n, k, A, lda, sA, B, ldb, sB, C_, ldc, sC, batch, dtype=F32):
    lib().lo_gemm_strided_batched(transa, transb, m, n, k, _p(A), lda, sA, _p(B), ldb, sB, _p(C_), ldc, sC,
                                  batch, dtype)
    return C_


def add_bias_gelu(out, bias, dtype=F32):
    m, n = out.shape
    lib().lo_add_bias_gelu(_p(out), _p(bias), m, n, dtype)
    return out


def add_bias_geglu(x2, bias, dtype=F32):
    """x2: [m, 2f] = [gate | up]; returns gelu(gate + b) * (up + b) as [m, f]."""
    m, f2 = x2.shape
    out = np.empty((m, f2 // 2), dtype=np.float32)
    lib().lo_add_bias_geglu(_p(out), _p(x2), _p(bias), m, f2 // 2, dtype)
    return out


def layer_norm(x, gamma, beta, dtype=F32):
    m, n = x.shape
    out = np.empty_like(x)
    lib().lo_layer_norm(_p(x), _p(gamma), _p(beta), _p(out), m, n, dtype)
    return out


def add_bias_input_layernorm(out, inp, bias, gamma, beta, dtype=F32):
    m, n = out.shape
    lib().lo_add_bias_input_layernorm(_p(out), _p(inp), _p(bias), _p(gamma), _p(beta), m, n, dtype)
    return out


def add_bias_input_layernorm_2(inp, gamma, beta, bias, output, dtype=F32):
    m, n = output.shape
    norm = np.empty_like(output)
    lib().lo_add_bias_input_layernorm_2(_p(inp), _p(gamma), _p(beta), _p(bias), _p(output), _p(norm), m, n,
                                        dtype)
    return output, norm


def add_bias_input(output, bias, inp, dtype=F32):
    m, n = output.shape
    lib().lo_add_bias_input(_p(output), _p(bias), _p(inp), m, n, dtype)
    return output


def add_qkv_bias_transpose(Q, bq, K, bk, V, bv, batch, seq, head_num, d, dtype=F32):
    qb, kb, vb = (np.empty((batch, head_num, seq, d), dtype=np.float32) for _ in range(3))
    lib().lo_add_qkv_bias_transpose(_p(qb), _p(kb), _p(vb), _p(Q), _p(bq), _p(K), _p(bk), _p(V), _p(bv),
                                    batch, seq, head_num, d, dtype)
    return qb, kb, vb


def add_fused_qkv_bias_transpose(QKV, bias, batch, seq, head_num, d, dtype=F32):
    qb, kb, vb = (np.empty((batch, head_num, seq, d), dtype=np.float32) for _ in range(3))
    lib().lo_add_fused_qkv_bias_transpose(_p(qb), _p(kb), _p(vb), _p(QKV), _p(bias), batch, seq, head_num, d,
                                          dtype)
    return qb, kb, vb


def attn_softmax(buf, mask, scalar, dtype=F32):
    batch, head_num, seq, seq2 = buf.shape
    assert seq == seq2 and mask.shape == (batch, seq, seq)
    lib().lo_attn_softmax(_p(buf), _p(mask), batch, seq, head_num, scalar, dtype)
    return buf


def transpose(src):
    batch, head_num, seq, d = src.shape
    dst = np.empty((batch, seq, head_num, d), dtype=np.float32)
    lib().lo_transpose(_p(dst), _p(src), batch, seq, head_num, d)
    return dst


def attn_decode(q, k_cache, v_cache, length, scalar, dtype=F32):
    batch, head_num, d = q.shape
    max_len = k_cache.shape[2]
    out = np.empty_like(q)
    lib().lo_attn_decode(_p(q), _p(k_cache), _p(v_cache), _p(out), batch, head_num, d, length, max_len,
                         scalar, dtype)
    return out


def attn_prefill(qb, kb, vb, scalar, causal, dtype=F32):
    batch, head_num, seq, d = qb.shape
    out = np.empty_like(qb)
    lib().lo_attn_prefill(_p(qb), _p(kb), _p(vb), _p(out), batch, seq, head_num, d, scalar, int(causal), dtype)
    return out


_WNAMES = [n for n, _ in LayerWeightsC._fields_]


def _mk(shape, weights):
    sh = LayerShapeC(**shape)
    wc = LayerWeightsC()
    keep = []
    for n in _WNAMES:
        a = weights.get(n)
        if a is not None:
            keep.append(a)
            setattr(wc, n, _p(a))
    return sh, wc, keep


def encoder_forward(shape, weights, x, mask=None):
    """shape: dict of LayerShapeC fields; weights: dict name -> float32 array; x: [B*S, H]."""
    sh, wc, _keep = _mk(shape, weights)
    out = np.empty_like(x)
    rc = lib().lo_encoder_forward(C.byref(sh), C.byref(wc), _p(mask), _p(x), _p(out))
    if rc != 0:
        raise ValueError("lo_encoder_forward: bad shape")
    return out


def mha_forward(shape, weights, x, mask=None):
    sh, wc, _keep = _mk(shape, weights)
    out = np.empty_like(x)
    rc = lib().lo_mha_forward(C.byref(sh), C.byref(wc), _p(mask), _p(x), _p(out))
    if rc != 0:
        raise ValueError("lo_mha_forward: bad shape")
    return out


def mlp_forward(shape, weights, x):
    sh, wc, _keep = _mk(shape, weights)
    out = np.empty_like(x)
    rc = lib().lo_mlp_forward(C.byref(sh), C.byref(wc), _p(x), _p(out))
    if rc != 0:
        raise ValueError("lo_mlp_forward: bad shape")
    return out


def decoder_step(shape, weights, x, k_cache, v_cache, past):
    sh, wc, _keep = _mk(shape, weights)
    out = np.empty_like(x)
    max_len = k_cache.shape[2]
    rc = lib().lo_decoder_step(C.byref(sh), C.byref(wc), _p(x), _p(k_cache), _p(v_cache), past, max_len,
                               _p(out))
    if rc != 0:
        raise ValueError("lo_decoder_step: bad shape")
    return out
