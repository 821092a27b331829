"""The two-thread host runtime (request thread + scheduler thread, tests/test_scheduler_cpu.py) under ThreadSanitizer and
AddressSanitizer.  The runtime is compiled with -fsanitize against the virtual-time backend (no GPU involved), loaded by a child
Python process that has the sanitizer's runtime preloaded, and the whole CPU scheduler suite runs in it: a data race between
serve() / update_vec() / the error state, a use after free of a Sample, a stream context or a request context, or a heap
overflow fails this test with the sanitizer's report."""
import importlib.util
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _build_module():
    spec = importlib.util.spec_from_file_location("liger_build", os.path.join(ROOT, "24ppopp-liger_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("sanitize", ["thread", "address"])
def test_scheduler_suite_is_clean_under_the_sanitizer(sanitize):
    b = _build_module()
    runtime = b.sanitizer_runtime(sanitize)
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        pytest.skip("no %s sanitizer runtime in this toolchain" % sanitize)
    lib = b.build_fake_host(force=False, sanitize=sanitize)
    env = dict(os.environ)
    # the sanitizer's runtime has to come first; whatever is preloaded already stays
    env["LD_PRELOAD"] = runtime + ((":" + env["LD_PRELOAD"]) if env.get("LD_PRELOAD") else "")
    env["LIGER_FAKE_LIB"] = lib
    env["TSAN_OPTIONS"] = "exitcode=66 halt_on_error=0 report_signal_unsafe=0"
    env["ASAN_OPTIONS"] = "exitcode=66 detect_leaks=0"      # the interpreter itself leaks at exit; leaks of the runtime are
    #                                                          counted by the fake backend (streams / allocations alive)
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_scheduler_cpu.py"), "-x", "-q", "-p", "no:cacheprovider"],
                       cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=900)
    report = r.stdout[-3000:] + "\n" + r.stderr[-6000:]
    assert "ThreadSanitizer" not in report and "AddressSanitizer" not in report, report
    assert r.returncode == 0, report
    assert " passed" in r.stdout and "failed" not in r.stdout, report
