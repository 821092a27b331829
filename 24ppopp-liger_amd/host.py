"""ctypes binding of lib/libliger_host.so: the C++ launch-vector runtime (layer assembly, Sample, Scheduler).

No compute and no fallback here; importing raises if the native libraries are missing.
"""
import ctypes as C
import os

import numpy as np

from . import capi

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libliger_host.so")

POST_NORESID, PRE_LN_RESID = 0, 1
POLICY_CLASSIC, POLICY_RESOURCE = 0, 1
FFN_GELU, FFN_GEGLU = 0, 1
SPLIT_OUT_COLS, SPLIT_TOKEN_ROWS = 0, 1
MODE_SEQUENTIAL, MODE_LIGER = 0, 1

_i, _i64, _u64, _f, _d, _p = C.c_int, C.c_int64, C.c_uint64, C.c_float, C.c_double, C.c_void_p


class Report(C.Structure):
    _fields_ = [("records", _i), ("avg_latency_ms", _d), ("p99_latency_ms", _d), ("avg_gpu_ms", _d),
                ("avg_queue_ms", _d), ("total_duration_ms", _d), ("throughput", _d), ("rounds", _i),
                ("secondary_launches", _i), ("splits", _i), ("profile_misses", _i), ("avg_e2e_ms", _d), ("p99_e2e_ms", _d),
                ("partition_rounds", _i), ("sub_profile_misses", _i), ("batched_steps", _i), ("batched_rows", _i)]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


SIGNATURES = {
    "lgh_first_error": (_i, [C.c_char_p, _i]),
    "lgh_clear_error": (None, []),
    "lgh_model_create": (_p, [_i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _u64]),
    "lgh_model_create_ex": (_p, [_i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _u64]),
    "lgh_model_kernels_per_layer": (_i, [_p, _i]),
    "lgh_model_workspace_elems": (_i64, [_p, _i, _i]),
    "lgh_model_stream": (_p, [_p]),
    "lgh_model_param_count": (_i, [_p]),
    "lgh_model_load_param": (_i, [_p, _i, _p, _i, _p]),
    "lgh_model_param_info": (_i, [_p, _i, C.c_char_p, _i, C.POINTER(_p), C.POINTER(_i64), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)]),
    "lgh_model_kv_cache": (_i, [_p, _i, C.POINTER(_p), C.POINTER(_p)]),
    "lgh_model_describe": (_i, [_p, _i, _i, _i, C.c_char_p, _i]),
    "lgh_model_run": (_i, [_p, _p, _p, _i, _i, _p, _p, _i]),
    "lgh_model_run_chunked": (_i, [_p, _p, _p, _i, _i, _p, _p, _i]),
    "lgh_model_run_decode": (_i, [_p, _p, _p, _i, _i, _i, _p, _p]),
    "lgh_model_run_decode_seqs": (_i, [_p, _p, _p, _i, C.POINTER(_i), C.POINTER(_i), _p, _p]),
    "lgh_model_time_kernels": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _i, C.POINTER(_f), _i]),
    "lgh_model_time_step": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, C.POINTER(_f), _i]),
    "lgh_model_time_one": (_f, [_p, _p, _p, _i, _i, _i, _i, _i, _i]),
    "lgh_sched_create": (_p, [_p, _i, _f, _i, _i, _i, _i, _i, _i]),
    "lgh_sched_destroy": (_i, [_p]),
    "lgh_model_destroy": (_i, [_p]),
    "lgh_sched_profile": (_i, [_p, _i, _i, _i, _i, _i]),
    "lgh_sched_profile_decode": (_i, [_p, _i, _i, _i]),
    "lgh_sched_profile_contention": (_i, [_p, _i, _i, _i, _i, C.POINTER(_f)]),
    "lgh_sched_set_contention": (_i, [_p, _i, _i, _f]),
    "lgh_sched_enable_partition": (_i, [_p, _i]),
    "lgh_sched_set_decode_step_hook": (_i, [_p, _p, _p]),
    "lgh_sched_set_prefill_chunk": (_i, [_p, _i]),
    "lgh_sched_chunk_counters": (_i, [_p, C.POINTER(_i)]),
    "lgh_sched_set_partition_feedback": (_i, [_p, _i, _i, _i, _f]),
    "lgh_sched_partition_feedback_state": (_i, [_p, C.POINTER(C.c_double)]),
    "lgh_sched_enable_batch_decode": (_i, [_p, _i, _i]),
    "lgh_sched_set_recycle_contexts": (_i, [_p, _i]),
    "lgh_sched_ctx_decode_ptrs": (_i, [_p, _i, C.POINTER(_p), C.POINTER(_p)]),
    "lgh_sched_profile_partition": (_i, [_p, _i, _i, _i, _i, C.POINTER(_f)]),
    "lgh_sched_set_partition_factor": (_i, [_p, _i, _i, _f]),
    "lgh_sched_get_partition_factor": (_f, [_p, _i, _i]),
    "lgh_sched_get_contention": (_f, [_p, _i, _i]),
    "lgh_sched_streams_concurrent": (_i, [_p]),
    "lgh_sched_partition_streams_concurrent": (_i, [_p]),
    "lgh_sched_set_verify_partition_streams": (_i, [_p, _i]),
    "lgh_sched_set_merge_minor": (_i, [_p, _i]),
    "lgh_sched_save": (_i, [_p, C.c_char_p, C.c_char_p]),
    "lgh_sched_load": (_i, [_p, C.c_char_p, C.c_char_p]),
    "lgh_sched_lookup": (_f, [_p, _i, _i, _i]),
    "lgh_sched_sub_lookup": (_i, [_p, _i, _i, _i, C.POINTER(_f), _i]),
    "lgh_sched_run_trace": (_i, [_p, _i, C.POINTER(_d), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), _i, C.POINTER(Report)]),
    "lgh_sched_set_profile": (_i, [_p, _i, _i, _i, _f, C.POINTER(_f), _i]),
    "lgh_sched_serve": (_i, [_p, _i, _i, _i]),
    "lgh_sched_serve_decode": (_i, [_p, _i, _i, _i]),
    "lgh_sched_set_factor": (_i, [_p, _i]),
    "lgh_sched_ctx_ptrs": (_i, [_p, _i, C.POINTER(_p), C.POINTER(_p)]),
    "lgh_sched_run_queued": (_i, [_p, _i, C.POINTER(Report)]),
    "lgh_summarize": (_i, [C.POINTER(_d), C.POINTER(_d), _i, _d, C.POINTER(Report)]),
    "lgh_make_poisson_trace": (_i, [_d, _i, _i, _i, _i, _i, _i, _u64, C.POINTER(_d), C.POINTER(_i)]),
}


def _load(path=LIB_PATH, mode=C.RTLD_GLOBAL):
    if not os.path.exists(path):
        raise ImportError("%s is not built; run __graft_entry__.build()" % path)
    lib = C.CDLL(path, mode=mode)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def use_library(path):
    """Rebinds this module to another build of the host runtime.  Exists for the CPU unit tests, which link the same
    runtime sources against a virtual-time stand-in for the device library; returns the previous binding."""
    global lib
    prev = lib
    lib = _load(path, C.RTLD_LOCAL)
    return prev


def first_error():
    buf = C.create_string_buffer(1024)
    code = lib.lgh_first_error(buf, 1024)
    return code, buf.value.decode()


def check(rc, what):
    if rc != 0:
        code, text = first_error()
        lib.lgh_clear_error()
        raise capi.LigerError("%s failed (%d): %s" % (what, code or rc, text))


def summarize(cpu_ms, gpu_ms, total_duration_ms):
    cpu = (C.c_double * len(cpu_ms))(*cpu_ms)
    gpu = (C.c_double * len(gpu_ms))(*gpu_ms)
    r = Report()
    check(lib.lgh_summarize(cpu, gpu, len(cpu_ms), total_duration_ms, C.byref(r)), "lgh_summarize")
    return r.as_dict()


def make_poisson_trace(lam, n, batch, seq_lo, seq_hi, seq_round, n_decode, seed):
    arr = (C.c_double * n)()
    seq = (C.c_int * n)()
    check(lib.lgh_make_poisson_trace(lam, n, batch, seq_lo, seq_hi, seq_round, n_decode, seed, arr, seq), "lgh_make_poisson_trace")
    return [{"arrival_s": arr[i], "batch": batch, "seq": seq[i], "n_decode": n_decode} for i in range(n)]


def _tile(a):
    """[features, k] -> the tiled storage order of lg_weight_tile_f16 (flat): blocks of 16 features x 32 k, inside a block
    element (f, j) at ((j // 8) * 16 + f) * 8 + j % 8."""
    n, k = a.shape
    return a.reshape(n // 16, 16, k // 32, 4, 8).transpose(0, 2, 3, 1, 4).reshape(-1)


def _untile(flat, n, k):
    return flat.reshape(n // 16, k // 32, 4, 16, 8).transpose(0, 3, 1, 2, 4).reshape(n * k)


def _interleave16(n, inverse=False):
    """Index vector of the stored order of n = 2 f features [first half | second half] interleaved in groups of 16:
    stored[p] = logical[idx[p]] (inverse: logical[c] = stored[idx[c]])."""
    f = n // 2
    p = np.arange(n)
    idx = (p // 32) * 16 + p % 16 + np.where(p % 32 >= 16, f, 0)
    if not inverse:
        return idx
    inv = np.empty(n, dtype=np.int64)
    inv[idx] = p
    return inv


class Model:
    """One tensor-parallel shard of a stack of encoder layers, assembled as launch vectors by the C++ runtime."""

    def __init__(self, dtype, max_batch, max_seq, head_num, size_per_head, layer_num=1, world_size=1, ffn_inner=0,
                 norm_mode=POST_NORESID, causal=False, fused=False, max_cache_len=0, factor=8, weight_layout=0, seed=0,
                 ffn_act=FFN_GELU, packed_qkv=False):
        lib.lgh_clear_error()
        self.h = lib.lgh_model_create_ex(dtype, max_batch, max_seq, head_num, size_per_head, layer_num, world_size, ffn_inner,
                                         norm_mode, int(causal), int(fused), max_cache_len, factor, weight_layout, int(ffn_act),
                                         int(packed_qkv), seed)
        if not self.h:
            check(1, "lgh_model_create")
        self._lib = lib          # the library the model was created in (tests switch libraries)
        self.dtype = dtype
        self.hidden = head_num * size_per_head
        self.layer_num = layer_num
        self.es = 2 if dtype == capi.F16 else 4

    def kernels_per_layer(self, decode=False):
        return lib.lgh_model_kernels_per_layer(self.h, int(decode))

    def workspace_elems(self, batch, seq):
        return lib.lgh_model_workspace_elems(self.h, batch, seq)

    @property
    def stream(self):
        return lib.lgh_model_stream(self.h)

    def close(self):
        """Frees the model's device memory and stream.  Schedulers built on it must be closed first (they hold a reference
        to the model, so garbage collection keeps that order)."""
        if getattr(self, "h", None) and self._lib is not None:
            self._lib.lgh_model_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def param_info(self):
        """name -> dict(ptr, elems, rows, cols, transposed, interleave16); rows x cols is the logical [in, out] shape;
        interleave16: the out dimension (or the vector) is stored with its two halves interleaved in groups of 16"""
        out = {}
        for i in range(lib.lgh_model_param_count(self.h)):
            name = C.create_string_buffer(128)
            ptr, n = _p(), _i64()
            r, c, t = _i(), _i(), _i()
            check(lib.lgh_model_param_info(self.h, i, name, 128, C.byref(ptr), C.byref(n), C.byref(r), C.byref(c), C.byref(t)),
                  "lgh_model_param_info")
            out[name.value.decode()] = dict(ptr=ptr.value, elems=n.value, rows=r.value, cols=c.value, transposed=t.value & 1,
                                            interleave16=(t.value >> 1) & 1, tiled=(t.value >> 2) & 1)
        return out

    def params(self):
        """name -> (device pointer, element count)"""
        return {k: (v["ptr"], v["elems"]) for k, v in self.param_info().items()}

    def download_params(self):
        """name -> float32 numpy array with the exact device values; weight matrices come back in the logical [in, out]
        orientation whatever their storage layout, vectors flat"""
        res = {}
        for name, info in self.param_info().items():
            n = info["elems"]
            raw = np.empty(n, dtype=np.float16 if self.dtype == capi.F16 else np.float32)
            capi.check(capi.lib.lg_memcpy_d2h(raw.ctypes.data_as(_p), _p(info["ptr"]), n * self.es), "lg_memcpy_d2h")
            a = raw.astype(np.float32)
            if info["rows"] > 1:
                if info["tiled"]:
                    a = _untile(a, info["cols"], info["rows"])      # -> [out, in]
                a = a.reshape(info["cols"], info["rows"]).T if info["transposed"] else a.reshape(info["rows"], info["cols"])
            if info["interleave16"]:
                a = a[..., _interleave16(a.shape[-1], inverse=True)]
            res[name] = np.ascontiguousarray(a)
        return res

    def load_param(self, name, device_ptr, src_layout, stream=None):
        """Takes parameter `name` over from device memory: a plain row-major array, weight matrices [in, out] (src_layout 0)
        or [out, in] (1), vectors flat.  The layer re-lays it into its own storage layout on the device (asynchronous on
        `stream`, default the model's)."""
        names = list(self.param_info().keys())
        if name not in names:
            raise KeyError("no parameter named %r" % name)
        check(lib.lgh_model_load_param(self.h, names.index(name), _p(device_ptr), int(src_layout), _p(stream) if stream else None),
              "lgh_model_load_param")

    def upload_params(self, values):
        """Overwrites parameters with host values: name -> array in the logical orientation download_params returns
        (weight matrices [in, out] whatever their storage layout, vectors flat)."""
        info = self.param_info()
        dt = np.float16 if self.dtype == capi.F16 else np.float32
        for name, a in values.items():
            if name not in info:
                raise KeyError("no parameter named %r" % name)
            i = info[name]
            a = np.asarray(a, dtype=np.float32)
            if i["rows"] > 1:
                if a.shape != (i["rows"], i["cols"]):
                    raise ValueError("%s: expected shape %s, got %s" % (name, (i["rows"], i["cols"]), a.shape))
            if i["interleave16"]:
                a = a[..., _interleave16(a.shape[-1])]
            if i["rows"] > 1:
                a = a.T if i["transposed"] else a
                if i["tiled"]:
                    a = _tile(np.ascontiguousarray(a))
            raw = np.ascontiguousarray(a, dtype=dt).ravel()
            if raw.size != i["elems"]:
                raise ValueError("%s: expected %d elements, got %d" % (name, i["elems"], raw.size))
            capi.check(capi.lib.lg_memcpy_h2d(_p(i["ptr"]), raw.ctypes.data_as(_p), raw.size * self.es), "lg_memcpy_h2d")

    def kv_cache(self, layer=0):
        """(k_cache, v_cache) device pointers of one layer: [max_batch, local heads, max_cache_len, size_per_head]."""
        k, v = _p(), _p()
        check(lib.lgh_model_kv_cache(self.h, layer, C.byref(k), C.byref(v)), "lgh_model_kv_cache")
        return k.value, v.value

    def describe(self, batch, seq, decode_past=-1):
        buf = C.create_string_buffer(1 << 16)
        n = lib.lgh_model_describe(self.h, batch, seq, decode_past, buf, 1 << 16)
        if n < 0:
            check(1, "lgh_model_describe")
        rows = [ln.split("|") for ln in buf.value.decode().strip().split("\n") if ln]
        return [{"idx": int(r[0]), "label": r[1], "type": r[2], "class": r[3]} for r in rows]

    def run(self, input_ptr, output_ptr, batch, seq, workspace_ptr=None, stream=None, cache_slot=-1):
        check(lib.lgh_model_run(self.h, input_ptr, output_ptr, batch, seq, workspace_ptr, stream, cache_slot), "lgh_model_run")

    def run_chunked(self, input_ptr, output_ptr, seq, chunk, cache_slot, workspace_ptr=None, stream=None):
        """The prefill of one sequence in chunks of `chunk` tokens over the KV cache of `cache_slot` (fused assembly)."""
        check(lib.lgh_model_run_chunked(self.h, input_ptr, output_ptr, seq, chunk, workspace_ptr, stream, cache_slot), "lgh_model_run_chunked")

    def run_decode(self, input_ptr, output_ptr, batch, past, cache_slot=0, workspace_ptr=None, stream=None):
        check(lib.lgh_model_run_decode(self.h, input_ptr, output_ptr, batch, past, cache_slot, workspace_ptr, stream),
              "lgh_model_run_decode")

    def run_decode_seqs(self, input_ptr, output_ptr, slots, pasts, workspace_ptr=None, stream=None):
        """One decode step for sequences in cache slots `slots` that hold `pasts` positions each."""
        n = len(slots)
        check(lib.lgh_model_run_decode_seqs(self.h, input_ptr, output_ptr, n, (C.c_int * n)(*slots), (C.c_int * n)(*pasts),
                                            workspace_ptr, stream), "lgh_model_run_decode_seqs")

    def time_step(self, input_ptr, output_ptr, batch, seq, decode_past=-1, cache_slot=-1, reps=20):
        """Mean time of every launch-vector entry inside whole steps (an event between every two entries, `reps` steps)."""
        out = (C.c_float * 4096)()
        n = lib.lgh_model_time_step(self.h, input_ptr, output_ptr, batch, seq, decode_past, cache_slot, reps, out, 4096)
        if n < 0:
            check(1, "lgh_model_time_step")
        return [out[i] for i in range(n)]

    def time_kernels(self, input_ptr, output_ptr, batch, seq, decode_past=-1, cache_slot=-1, iters=20, trials=3):
        out = (C.c_float * 4096)()
        n = lib.lgh_model_time_kernels(self.h, input_ptr, output_ptr, batch, seq, decode_past, cache_slot, iters, trials, out, 4096)
        if n < 0:
            check(1, "lgh_model_time_kernels")
        return [out[i] for i in range(n)]


class Scheduler:
    def __init__(self, model, schedule_deep=6, contention_factor=0.8, policy=POLICY_RESOURCE, axis=SPLIT_OUT_COLS,
                 seq_bucket=1, ignore_num=0, pool_count=0, ctx_batch=1):
        lib.lgh_clear_error()
        self.model = model
        self.h = lib.lgh_sched_create(model.h, schedule_deep, contention_factor, policy, axis, seq_bucket, ignore_num,
                                      pool_count, ctx_batch)
        if not self.h:
            check(1, "lgh_sched_create")
        self._lib = lib

    def close(self):
        """Frees the scheduler's streams, events, request contexts and decode-batch buffers (every stream holds a hardware
        queue: a process that keeps creating schedulers without closing them ends up with streams that share queues)."""
        if getattr(self, "h", None) and self._lib is not None:
            self._lib.lgh_sched_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def profile(self, bs, seq_lo, seq_hi, seq_step=1, itr=20):
        check(lib.lgh_sched_profile(self.h, bs, seq_lo, seq_hi, seq_step, itr), "lgh_sched_profile")

    def profile_decode(self, bs, past, itr=20):
        check(lib.lgh_sched_profile_decode(self.h, bs, past, itr), "lgh_sched_profile_decode")

    def profile_contention(self, bs, seq, dec_bs, past):
        """Measures prefill MFMA-bound kernels || decode-step kernels on the two streams and installs the result in the
        contention table.  Returns primary / secondary / concurrent ms, the hidden fraction and the secondary's repeats."""
        out = (_f * 5)()
        check(lib.lgh_sched_profile_contention(self.h, bs, seq, dec_bs, past, out), "lgh_sched_profile_contention")
        return {"main_ms": out[0], "sub_ms": out[1], "both_ms": out[2], "hidden": out[3], "sub_repeats": int(out[4])}

    def enable_batch_decode(self, on=True, steps_ahead=0):
        """Requests that are in their decode steps at the same time share one launch vector per step."""
        check(lib.lgh_sched_enable_batch_decode(self.h, int(bool(on)), steps_ahead), "lgh_sched_enable_batch_decode")

    def set_decode_step_hook(self, fn):
        """fn(step, slots, pasts, rows_ptr, stream) runs on the scheduler's thread after the kernels of every batched decode step
        have been launched (slots / pasts: per batch row, before the step); None removes it."""
        if fn is None:
            self._hook = None
            check(lib.lgh_sched_set_decode_step_hook(self.h, None, None), "lgh_sched_set_decode_step_hook")
            return
        proto = C.CFUNCTYPE(None, _p, _i, _i, C.POINTER(_i), C.POINTER(_i), _p, _p)

        def tramp(_user, step, rows, slots, pasts, ptr, stream):
            fn(step, [slots[i] for i in range(rows)], [pasts[i] for i in range(rows)], ptr, stream)
        self._hook = proto(tramp)      # kept alive with the scheduler
        check(lib.lgh_sched_set_decode_step_hook(self.h, C.cast(self._hook, _p), None), "lgh_sched_set_decode_step_hook")

    def set_recycle_contexts(self, on):
        """False: finished requests keep their context (and results) until the next run starts."""
        check(lib.lgh_sched_set_recycle_contexts(self.h, int(bool(on))), "lgh_sched_set_recycle_contexts")

    def ctx_decode_ptrs(self, i):
        a, b = _p(), _p()
        check(lib.lgh_sched_ctx_decode_ptrs(self.h, i, C.byref(a), C.byref(b)), "lgh_sched_ctx_decode_ptrs")
        return a.value, b.value

    def enable_partition(self, hbm_cus):
        """Co-running rounds give the HBM-bound side `hbm_cus` compute units and the MFMA-bound side the rest (0 = off)."""
        check(lib.lgh_sched_enable_partition(self.h, hbm_cus), "lgh_sched_enable_partition")

    def set_prefill_chunk(self, rows):
        """With batched decode steps: single-sequence prompts longer than `rows` tokens are prefilled in chunks of `rows` over their
        KV-cache slot and the batched decode step runs between two chunks (0 = off)."""
        check(lib.lgh_sched_set_prefill_chunk(self.h, rows), "lgh_sched_set_prefill_chunk")

    def chunk_counters(self):
        out = (_i * 2)()
        check(lib.lgh_sched_chunk_counters(self.h, out), "lgh_sched_chunk_counters")
        return {"chunked_prefills": out[0], "yield_turns": out[1]}

    def set_partition_feedback(self, on, min_samples=0, probe=-1, margin=0.0):
        """While a run goes on, rounds that could be partitioned are run both ways and partitioned only while that delivers more
        (on by default).  min_samples / probe / margin: samples of each kind before deciding, every n-th such round takes the other
        side, required ratio of the two progress rates; non-positive (probe: negative) values keep what is set."""
        check(lib.lgh_sched_set_partition_feedback(self.h, int(bool(on)), min_samples, probe, margin), "lgh_sched_set_partition_feedback")

    def partition_feedback_state(self):
        out = (C.c_double * 5)()
        check(lib.lgh_sched_partition_feedback_state(self.h, out), "lgh_sched_partition_feedback_state")
        return {"rate_whole_chip": out[0], "rate_partitioned": out[1], "samples_whole_chip": int(out[2]), "samples_partitioned": int(out[3]),
                "declined": int(out[4])}

    def profile_partition(self, bs, seq, dec_bs, past):
        """Measures a partitioned co-run (prefill MFMA-bound kernels || decode steps) and installs the budget factors when
        it beats back-to-back execution on the whole chip."""
        out = (_f * 7)()
        check(lib.lgh_sched_profile_partition(self.h, bs, seq, dec_bs, past, out), "lgh_sched_profile_partition")
        return {"main_ms": out[0], "sub_ms": out[1], "main_part_ms": out[2], "sub_part_ms": out[3], "factor": out[4],
                "gain": out[5], "sub_repeats": int(out[6])}

    def set_partition_factor(self, main_class, sub_class, value):
        check(lib.lgh_sched_set_partition_factor(self.h, main_class, sub_class, value), "lgh_sched_set_partition_factor")

    def partition_factor(self, main_class, sub_class):
        return lib.lgh_sched_get_partition_factor(self.h, main_class, sub_class)

    def set_contention(self, main_class, sub_class, value):
        check(lib.lgh_sched_set_contention(self.h, main_class, sub_class, value), "lgh_sched_set_contention")

    def contention(self, main_class, sub_class):
        return lib.lgh_sched_get_contention(self.h, main_class, sub_class)

    def set_merge_minor(self, on):
        """Minor entries (LayerNorm, residual, cache append, row gather) take the scheduling class of the entry before them."""
        check(lib.lgh_sched_set_merge_minor(self.h, int(bool(on))), "lgh_sched_set_merge_minor")

    @property
    def streams_concurrent(self):
        """True when the second stream was verified (by measurement) to execute at the same time as the first."""
        return bool(lib.lgh_sched_streams_concurrent(self.h))

    @property
    def partition_streams_concurrent(self):
        """True when the CU-masked streams of the share in use were measured to overlap pair by pair (primary, secondary),
        False when a pair could not be made to, None when they were not probed."""
        v = lib.lgh_sched_partition_streams_concurrent(self.h)
        return None if v < 0 else bool(v)

    def set_verify_partition_streams(self, on):
        """enable_partition probes the stream pairs of a share it creates and replaces secondaries that take turns (off by default)."""
        check(lib.lgh_sched_set_verify_partition_streams(self.h, int(bool(on))), "lgh_sched_set_verify_partition_streams")

    def save(self, main_file, sub_file):
        check(lib.lgh_sched_save(self.h, main_file.encode(), sub_file.encode()), "lgh_sched_save")

    def load(self, main_file, sub_file):
        check(lib.lgh_sched_load(self.h, main_file.encode(), sub_file.encode()), "lgh_sched_load")

    def lookup(self, name, bs, seq):
        return lib.lgh_sched_lookup(self.h, name, bs, seq)

    def sub_lookup(self, name, bs, seq):
        out = (C.c_float * 64)()
        n = lib.lgh_sched_sub_lookup(self.h, name, bs, seq, out, 64)
        return None if n < 0 else [out[i] for i in range(n)]

    def set_profile(self, name, bs, seq, ms, sub=None):
        arr = (C.c_float * len(sub))(*sub) if sub else None
        check(lib.lgh_sched_set_profile(self.h, name, bs, seq, ms, arr, len(sub) if sub else 0), "lgh_sched_set_profile")

    def serve(self, bs, seq, n_decode=0):
        check(lib.lgh_sched_serve(self.h, bs, seq, n_decode), "lgh_sched_serve")

    def serve_decode(self, bs, past, n_steps):
        check(lib.lgh_sched_serve_decode(self.h, bs, past, n_steps), "lgh_sched_serve_decode")

    def set_factor(self, factor):
        check(lib.lgh_sched_set_factor(self.h, factor), "lgh_sched_set_factor")

    def ctx_ptrs(self, i):
        a, b = _p(), _p()
        check(lib.lgh_sched_ctx_ptrs(self.h, i, C.byref(a), C.byref(b)), "lgh_sched_ctx_ptrs")
        return a.value, b.value

    def run_queued(self, mode):
        r = Report()
        check(lib.lgh_sched_run_queued(self.h, mode, C.byref(r)), "lgh_sched_run_queued")
        return r.as_dict()

    def run_trace(self, trace, mode):
        n = len(trace)
        arr = (C.c_double * n)(*[t["arrival_s"] for t in trace])
        bs = (C.c_int * n)(*[t["batch"] for t in trace])
        sq = (C.c_int * n)(*[t["seq"] for t in trace])
        nd = (C.c_int * n)(*[t.get("n_decode", 0) for t in trace])
        r = Report()
        check(lib.lgh_sched_run_trace(self.h, mode, arr, bs, sq, nd, n, C.byref(r)), "lgh_sched_run_trace")
        return r.as_dict()
