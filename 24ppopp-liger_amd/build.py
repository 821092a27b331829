"""Build recipe for the native libraries (hipcc for the gfx950 device library, g++ for the host runtime).

Everything is built in-tree so that the shared objects travel with the source tree:
    24ppopp-liger_amd/lib/libliger_hip.so     device kernels + C ABI   (include/liger_hip.h)
    24ppopp-liger_amd/lib/libliger_host.so    launch-vector host runtime (host/*.h, host/host_capi.cpp)
    24ppopp-liger_amd/lib/liger_main          driver mirroring the reference's main.cu
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(PKG, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-value",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-option-ignored",
]
HIP_SOURCES = ["runtime.hip", "elementwise.hip", "attention_aux.hip", "gemm.hip", "gemm_fast.hip", "gemm_skinny.hip", "gemm_skinny_kn.hip", "gemv.hip", "attention.hip",
               "attention_prefill.hip", "ceilings.hip", "weight_layout.hip"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build_device(force=True, verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))]
    headers.append(os.path.join(ROOT, "include", "liger_hip.h"))
    objs, jobs = [], []
    for src in HIP_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJDIR, src.replace(".hip", ".o"))
        objs.append(o)
        if force or _stale(o, [s] + headers):
            jobs.append([HIPCC] + HIP_FLAGS + ["-c", s, "-o", o])
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for out in ex.map(_run, jobs):
            if verbose and out.strip():
                print(out)
    lib = os.path.join(LIBDIR, "libliger_hip.so")
    if jobs or not os.path.exists(lib):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    return lib


def build_host(force=True, verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = [os.path.join(HOST, f) for f in sorted(os.listdir(HOST)) if f.endswith(".cpp") and f != "liger_main.cpp"]
    if not srcs:
        return None
    hdrs = [os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".h")]
    hdrs.append(os.path.join(ROOT, "include", "liger_hip.h"))
    lib = os.path.join(LIBDIR, "libliger_host.so")
    cxx = ["g++", "-O2", "-g", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-pthread", "-I", os.path.join(ROOT, "include"),
           "-I", HOST]
    if force or _stale(lib, srcs + hdrs):
        out = _run(cxx + ["-shared", "-o", lib] + srcs + ["-L", LIBDIR, "-lliger_hip", "-Wl,-rpath,$ORIGIN"])
        if verbose and out.strip():
            print(out)
    main_src = os.path.join(HOST, "liger_main.cpp")
    exe = os.path.join(LIBDIR, "liger_main")
    if os.path.exists(main_src) and (force or _stale(exe, [main_src] + srcs + hdrs)):
        _run(cxx + ["-o", exe, main_src, "-L", LIBDIR, "-lliger_host", "-lliger_hip", "-Wl,-rpath,$ORIGIN"])
    return lib


def build_fake_host(force=True, sanitize=None):
    """The same host runtime linked against tests/fake_backend (virtual-time stand-in for the device library):
    lets the scheduler logic be unit-tested without a GPU.  Test infrastructure; never loaded by the product.
    sanitize = "thread" | "address": an instrumented build (libliger_host_fake_tsan.so / _asan.so) for the two-thread
    scheduler tests; the process that loads it must have the sanitizer's runtime preloaded."""
    fake_dir = os.path.join(ROOT, "tests", "fake_backend")
    src = os.path.join(fake_dir, "fake_hip.cpp")
    if not os.path.exists(src):
        return None
    if sanitize not in (None, "thread", "address"):
        raise ValueError("sanitize must be None, 'thread' or 'address'")
    suffix = {None: "", "thread": "_tsan", "address": "_asan"}[sanitize]
    lib = os.path.join(fake_dir, "libliger_host_fake%s.so" % suffix)
    srcs = [os.path.join(HOST, f) for f in sorted(os.listdir(HOST)) if f.endswith(".cpp") and f != "liger_main.cpp"] + [src]
    hdrs = [os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".h")] + [os.path.join(ROOT, "include", "liger_hip.h")]
    san = ["-fsanitize=" + sanitize, "-fno-omit-frame-pointer"] if sanitize else []
    if force or _stale(lib, srcs + hdrs):
        _run(["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter", "-pthread", "-I",
              os.path.join(ROOT, "include"), "-I", HOST, "-shared", "-Wl,-Bsymbolic"] + san + ["-o", lib] + srcs)
    return lib


def sanitizer_runtime(sanitize):
    """Path of the sanitizer's shared runtime (to preload into a process that loads an instrumented library)."""
    name = {"thread": "libtsan.so", "address": "libasan.so"}[sanitize]
    return subprocess.run(["g++", "-print-file-name=" + name], stdout=subprocess.PIPE, text=True).stdout.strip()


def build_all(force=True, verbose=False):
    dev = build_device(force=force, verbose=verbose)
    host = build_host(force=force, verbose=verbose)
    build_fake_host(force=force)
    return dev, host


if __name__ == "__main__":
    force = "--incremental" not in sys.argv
    print(build_all(force=force, verbose=True))
