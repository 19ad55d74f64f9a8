"""CPU test: the posix store's host runtime (queues, task table, per-block commit bookkeeping)
under ThreadSanitizer.  hipcc builds the two host-only sources of the library plus a stress
driver with -fsanitize=thread on the host pass; the driver exits non-zero on a wrong byte and
TSan turns a data race into a non-zero exit as well."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "unified-cache-management_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not found")
def test_posix_store_is_race_free_under_tsan(tmp_path):
    exe = tmp_path / "stress_tsan"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-Xarch_host", "-fsanitize=thread",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
           "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
           os.path.join(CSRC, "common.hip"), os.path.join(CSRC, "posix_store.hip"),
           os.path.join(ROOT, "tests", "native", "posix_store_stress.cpp"), "-o", str(exe)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    data = tmp_path / "store"
    data.mkdir()
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66")
    r = subprocess.run([str(exe), str(data)], capture_output=True, text=True, timeout=300, env=env)
    if "unexpected memory mapping" in r.stderr or "FATAL: ThreadSanitizer" in r.stderr:
        pytest.skip("ThreadSanitizer cannot run in this environment: " + r.stderr.strip()[:200])
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert "bad=0" in r.stdout
    shutil.rmtree(data, ignore_errors=True)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not found")
def test_cache_store_host_threads_are_race_free_under_tsan(tmp_path):
    """The cache store's worker threads with host-memory stand-ins for the copy streams and an
    asynchronous backend: a failed load task must not give its staging nodes back while the
    backend still writes into them, and destroy waits for backend dumps in flight."""
    exe = tmp_path / "cache_stress_tsan"
    cmd = [HIPCC, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-Xarch_host", "-fsanitize=thread",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
           "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
           os.path.join(CSRC, "common.hip"), os.path.join(CSRC, "cache_store.hip"),
           os.path.join(ROOT, "tests", "native", "cache_store_stress.cpp"), "-o", str(exe)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66")
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, env=env)
    if "unexpected memory mapping" in r.stderr or "FATAL: ThreadSanitizer" in r.stderr:
        pytest.skip("ThreadSanitizer cannot run in this environment: " + r.stderr.strip()[:200])
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert "bad=0" in r.stdout
