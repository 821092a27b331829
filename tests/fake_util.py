"""Access to the virtual-time backend (tests/fake_backend) from the CPU unit tests."""
import ctypes as C
import importlib
import os

# LIGER_FAKE_LIB selects another build of the same library (the sanitizer runs load an instrumented one)
FAKE_LIB = os.environ.get("LIGER_FAKE_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "fake_backend", "libliger_host_fake.so")


class Fake:
    """The host runtime bound to the fake backend, plus the backend's trace."""

    def __init__(self):
        self.host = importlib.import_module("24ppopp-liger_amd.host")
        self._prev = self.host.use_library(FAKE_LIB)
        self.lib = self.host.lib
        self.lib.fake_trace_get.argtypes = [C.c_int, C.POINTER(C.c_int), C.c_char_p, C.c_int, C.POINTER(C.c_longlong),
                                            C.POINTER(C.c_ulonglong), C.POINTER(C.c_double)]
        self.lib.fake_set_rates.argtypes = [C.c_double, C.c_double, C.c_double]
        self.lib.fake_host_now.restype = C.c_double
        self.lib.fake_set_corun_speed.argtypes = [C.c_double]
        self.lib.fake_set_share_model.argtypes = [C.c_double, C.c_double]

    def close(self):
        self.host.lib = self._prev

    def reset(self):
        self.lib.fake_reset()

    def set_rates(self, mfma_flop_per_ms, hbm_bytes_per_ms, launch_cost_ms):
        self.lib.fake_set_rates(mfma_flop_per_ms, hbm_bytes_per_ms, launch_cost_ms)

    def set_corun_speed(self, speed):
        """A kernel launched while another stream is busy runs at `speed` (0..1] of its stand-alone speed."""
        self.lib.fake_set_corun_speed(speed)

    def set_share_model(self, matrix_exp, memory_exp):
        """A kernel on a stream with `cus` of 256 compute units costs (256 / cus) ** exp times its whole-chip cost."""
        self.lib.fake_set_share_model(matrix_exp, memory_exp)

    def trace(self):
        out = []
        for i in range(self.lib.fake_trace_count()):
            st = C.c_int()
            name = C.create_string_buffer(64)
            abc = (C.c_longlong * 3)()
            ptrs = (C.c_ulonglong * 3)()
            se = (C.c_double * 2)()
            self.lib.fake_trace_get(i, C.byref(st), name, 64, abc, ptrs, se)
            out.append({"stream": st.value, "name": name.value.decode(), "m": abc[0], "n": abc[1], "k": abc[2],
                        "A": ptrs[0], "B": ptrs[1], "C": ptrs[2], "start": se[0], "end": se[1]})
        return out
