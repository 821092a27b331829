"""ctypes binding of lib/libliger_hip.so -- one Python callable per entry point of include/liger_hip.h.

No compute happens here and there is no fallback: a missing library is an ImportError-grade failure.
Pointers are passed as integers (e.g. `tensor.data_ptr()`); streams as integers (`stream.cuda_stream`).
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libliger_hip.so")

OK, ERR_INVALID, ERR_LAUNCH = 0, 1, 2
F32, F16 = 0, 1
OP_N, OP_T, OP_TILED = 0, 1, 2
EPI_NONE, EPI_BIAS, EPI_BIAS_GELU, EPI_BIAS_HEADS = 0, 1, 2, 3

_i, _i64, _u64, _f, _p, _sz = C.c_int, C.c_int64, C.c_uint64, C.c_float, C.c_void_p, C.c_size_t

# name -> (restype, argtypes); kept in the order of include/liger_hip.h
SIGNATURES = {
    "lg_last_error": (C.c_char_p, []),
    "lg_version": (C.c_char_p, []),
    "lg_device_info": (_i, [C.c_char_p, _i, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.POINTER(_sz)]),
    "lg_malloc": (_i, [C.POINTER(_p), _sz]),
    "lg_free": (_i, [_p]),
    "lg_memcpy_h2d": (_i, [_p, _p, _sz]),
    "lg_memcpy_d2h": (_i, [_p, _p, _sz]),
    "lg_memcpy_d2d_async": (_i, [_p, _p, _sz, _p]),
    "lg_memset_async": (_i, [_p, _i, _sz, _p]),
    "lg_device_synchronize": (_i, []),
    "lg_stream_create": (_i, [C.POINTER(_p)]),
    "lg_stream_attach": (_i, [_p, _i]),
    "lg_stream_detach": (_i, [_p]),
    "lg_stream_cu_count": (_i, [_p]),
    "lg_stream_create_cu_mask": (_i, [C.POINTER(_p), C.POINTER(C.c_uint), _i]),
    "lg_stream_create_concurrent": (_i, [_p, _p, _p]),
    "lg_streams_run_concurrently": (_i, [_p, _p, _p]),
    "lg_stream_destroy": (_i, [_p]),
    "lg_stream_synchronize": (_i, [_p]),
    "lg_stream_wait_event": (_i, [_p, _p]),
    "lg_event_create": (_i, [C.POINTER(_p)]),
    "lg_event_destroy": (_i, [_p]),
    "lg_event_record": (_i, [_p, _p]),
    "lg_event_synchronize": (_i, [_p]),
    "lg_event_query": (_i, [_p]),
    "lg_event_elapsed_ms": (_i, [C.POINTER(_f), _p, _p]),
    "lg_fill_normal_f32": (_i, [_p, _i64, _u64, _u64, _f, _f, _p]),
    "lg_fill_normal_f16": (_i, [_p, _i64, _u64, _u64, _f, _f, _p]),
    "lg_fill_const_f32": (_i, [_p, _i64, _f, _p]),
    "lg_fill_const_f16": (_i, [_p, _i64, _f, _p]),
    "lg_fill_causal_mask_f32": (_i, [_p, _i, _i, _p]),
    "lg_fill_causal_mask_f16": (_i, [_p, _i, _i, _p]),
    "lg_layer_norm_f32": (_i, [_p, _p, _p, _p, _i, _i, _p]),
    "lg_layer_norm_f16": (_i, [_p, _p, _p, _p, _i, _i, _p]),
    "lg_add_bias_act_f32": (_i, [_p, _p, _i, _i, _p]),
    "lg_add_bias_act_f16": (_i, [_p, _p, _i, _i, _p]),
    "lg_add_bias_geglu_f32": (_i, [_p, _p, _p, _i, _i, _p]),
    "lg_add_bias_geglu_f16": (_i, [_p, _p, _p, _i, _i, _p]),
    "lg_add_bias_input_layernorm_f32": (_i, [_p, _p, _p, _p, _p, _i, _i, _p]),
    "lg_add_bias_input_layernorm_f16": (_i, [_p, _p, _p, _p, _p, _i, _i, _p]),
    "lg_add_bias_input_layernorm_2_f32": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _p]),
    "lg_add_bias_input_layernorm_2_f16": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _p]),
    "lg_add_bias_input_f32": (_i, [_p, _p, _p, _i, _i, _p]),
    "lg_add_bias_input_f16": (_i, [_p, _p, _p, _i, _i, _p]),
    "lg_add_qkv_bias_transpose_f32": (_i, [_p] * 9 + [_i, _i, _i, _i, _p]),
    "lg_add_qkv_bias_transpose_f16": (_i, [_p] * 9 + [_i, _i, _i, _i, _p]),
    "lg_add_fused_qkv_bias_transpose_f32": (_i, [_p] * 5 + [_i, _i, _i, _i, _p]),
    "lg_add_fused_qkv_bias_transpose_f16": (_i, [_p] * 5 + [_i, _i, _i, _i, _p]),
    "lg_attn_softmax_f32": (_i, [_p, _p, _i, _i, _i, _f, _p]),
    "lg_attn_softmax_f16": (_i, [_p, _p, _i, _i, _i, _f, _p]),
    "lg_transpose_f32": (_i, [_p, _p, _i, _i, _i, _i, _p]),
    "lg_transpose_f16": (_i, [_p, _p, _i, _i, _i, _i, _p]),
    "lg_gemm_f32": (_i, [_i, _i, _i, _i, _i, _p, _i, _p, _i, _p, _i, _p]),
    "lg_gemm_f16": (_i, [_i, _i, _i, _i, _i, _p, _i, _p, _i, _p, _i, _p]),
    "lg_gemm_strided_batched_f32": (_i, [_i, _i, _i, _i, _i, _p, _i, _i64, _p, _i, _i64, _p, _i, _i64, _i, _p]),
    "lg_gemm_strided_batched_f16": (_i, [_i, _i, _i, _i, _i, _p, _i, _i64, _p, _i, _i64, _p, _i, _i64, _i, _p]),
    "lg_gemm_fused_f16": (_i, [_i, _i, _i, _i, _p, _i, _p, _i, _p, _i, _i, _p, _i, _i, _i, _p]),
    "lg_gemm_fused_grouped_f16": (_i, [_i, _i, _i, _i, _i, _p, _i, _p, _i, _p, _p, _i, _p, _i, _i, _i, _p]),
    "lg_gemm_fused_grouped_rows_f16": (_i, [_i, _i, _i, _i, _i, _p, _i, _p, _i, _p, _p, _p, _i, _i, _p, _p, _p, _p]),
    "lg_attn_prefill_f16": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p]),
    "lg_attn_prefill_past_f16": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _i, _i, _p]),
    "lg_attn_decode_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "lg_attn_decode_f16": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _f, _p]),
    "lg_attn_decode_varlen_f16": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, C.POINTER(_i), C.POINTER(_i), _i, _f, _p]),
    "lg_attn_decode_static_f16": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _f, _p]),
    "lg_kv_append_f16": (_i, [_p] * 9 + [_i, _i, _i, _i, _i, _p]),
    "lg_kv_append_varlen_f16": (_i, [_p] * 9 + [_i, _i, _i, C.POINTER(_i), C.POINTER(_i), _i, _p]),
    "lg_weight_tile_f16": (_i, [_p, _p, _i, _i, _i, _i, _p]),
    "lg_weight_untile_f16": (_i, [_p, _p, _i, _i, _i, _i, _p]),
    "lg_probe_mfma_f16": (_i, [_p, _i64, _p, _sz, _i, C.POINTER(_f), C.POINTER(_f), C.POINTER(_f), _p]),
    "lg_probe_mfma_stream_f16": (_i, [_p, _i64, _p, _sz, _i, _i, _i, C.POINTER(_f), C.POINTER(_f), C.POINTER(_f), _p]),
    "lg_probe_read": (_i, [_p, _sz, _p, _i, _i, C.POINTER(_f), C.POINTER(_f), _p]),
}


class LigerError(RuntimeError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libliger_hip.so is not built (expected at %s); run __graft_entry__.build() -- there is no "
            "fallback path" % LIB_PATH)
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def last_error():
    return lib.lg_last_error().decode()


def check(rc, what=""):
    """Raise LigerError on a non-zero status."""
    if rc != OK:
        raise LigerError("%s failed with status %d: %s" % (what or "liger call", rc, last_error()))


def call(name, *args):
    """Call entry point `name` and raise on error."""
    check(getattr(lib, name)(*args), name)


def device_info():
    name = C.create_string_buffer(128)
    cu, clk, mclk, bus = _i(), _i(), _i(), _i()
    mem = _sz()
    check(lib.lg_device_info(name, 128, C.byref(cu), C.byref(clk), C.byref(mclk), C.byref(bus), C.byref(mem)),
          "lg_device_info")
    return {"name": name.value.decode(), "cu_count": cu.value, "clock_khz": clk.value, "mem_clock_khz": mclk.value,
            "bus_width_bits": bus.value, "total_mem": mem.value}
