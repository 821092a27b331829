"""Helpers for the GPU parity tests: torch provides device memory and the stream, nothing else."""
import ctypes as C

import numpy as np
import torch


class Dev:
    def __init__(self, liger):
        self.liger = liger
        self.capi = liger.capi
        self.lib = liger.capi.lib
        self.device = torch.device("cuda:0")
        torch.cuda.set_device(0)
        # the device library is told about the stream the tests launch on (it allocates that stream's split-K workspace)
        rc = self.lib.lg_stream_attach(C.c_void_p(self.stream), 0)
        assert rc == 0, self.capi.last_error()

    @property
    def stream(self):
        return torch.cuda.current_stream().cuda_stream

    def up(self, a, dtype):
        """numpy float32 array -> device tensor of dtype ('f32' | 'f16')."""
        t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
        t = t.to(self.device)
        t = t.half() if dtype in ("f16", 1) else t
        torch.cuda.synchronize()   # callers may launch on another stream than torch's
        return t

    def empty(self, shape, dtype):
        return torch.empty(shape, device=self.device, dtype=torch.float16 if dtype in ("f16", 1) else torch.float32)

    def down(self, t):
        torch.cuda.synchronize()
        return t.float().cpu().numpy()

    def call(self, name, *args):
        """Call a C-ABI entry point; tensors are passed as raw device pointers; appends the current stream."""
        conv = [C.c_void_p(a.data_ptr()) if isinstance(a, torch.Tensor) else a for a in args]
        rc = getattr(self.lib, name)(*conv, C.c_void_p(self.stream))
        if rc != 0:
            raise self.capi.LigerError("%s -> %d: %s" % (name, rc, self.capi.last_error()))

    def call_rc(self, name, *args):
        conv = [C.c_void_p(a.data_ptr()) if isinstance(a, torch.Tensor) else a for a in args]
        return getattr(self.lib, name)(*conv, C.c_void_p(self.stream))

    def sync(self):
        torch.cuda.synchronize()
