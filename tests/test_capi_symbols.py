"""The C-ABI library loads and exports every symbol include/liger_hip.h declares (no compute calls without a GPU)."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "liger_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lg_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(liger):
    names = declared_symbols()
    assert len(names) >= 50
    lib = C.CDLL(liger.capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), "libliger_hip.so does not export %s" % n
        assert n in liger.capi.SIGNATURES, "capi.py has no signature for %s" % n
    assert sorted(liger.capi.SIGNATURES) == names


def test_fake_backend_covers_the_same_abi():
    fake = os.path.join(ROOT, "tests", "fake_backend", "libliger_host_fake.so")
    lib = C.CDLL(fake, mode=C.RTLD_LOCAL)
    for n in declared_symbols():
        assert hasattr(lib, n), "fake backend lacks %s" % n


def test_version_and_error_text_without_a_gpu(liger):
    assert b"gfx950" in liger.capi.lib.lg_version()
    # argument validation happens on the host, before any launch
    assert liger.capi.lib.lg_layer_norm_f32(None, None, None, None, 4, 0, None) == liger.capi.ERR_INVALID
    assert "bad shape" in liger.capi.last_error()
    assert liger.capi.lib.lg_gemm_f16(0, 1, 4, 4, 4, None, 4, None, 4, None, 4, None) == liger.capi.ERR_INVALID
    assert liger.capi.lib.lg_attn_decode_f16(None, None, None, None, None, 1, 1, 80, 8, 8, 1.0, None) == liger.capi.ERR_INVALID


def test_bench_refuses_more_than_one_gpu_with_a_message():
    """bench.py measures one GPU's shard on one GPU: --gpus 2 exits with status 2 and says so, before anything touches a GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                       text=True, timeout=120)
    assert r.returncode == 2
    assert "--gpus 2 is not supported" in r.stderr and r.stdout == ""
