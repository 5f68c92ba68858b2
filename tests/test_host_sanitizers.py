"""The library's pure host logic (bi-kv_amd/csrc/host_logic/*.h: chunk planner, duplicate finder, chunk
interleaving order, ring bookkeeping with back-pressure and its producer lock) built with gcc's sanitizers
and run on the CPU. The reference has no sanitizer or race-detection runs of any kind, and its
process-global ring state is raced by its own thread pools (Bi-KV/SharedMemory/CUDA_Shared/
ipc_service.cpp:9-17)."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host_san")


@pytest.fixture(scope="module")
def built():
    r = subprocess.run(["make", "-C", HERE, "-j2"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    return HERE


def _run(path, env_extra):
    env = dict(os.environ, **env_extra)
    r = subprocess.run([path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300, env=env)
    return r.returncode, r.stdout


def test_host_logic_under_address_and_undefined_behaviour_sanitizers(built):
    rc, out = _run(os.path.join(built, "host_logic_asan"),
                   {"ASAN_OPTIONS": "detect_leaks=1:abort_on_error=0", "UBSAN_OPTIONS": "print_stacktrace=1:halt_on_error=1"})
    assert rc == 0 and "host_logic ok" in out, out


def test_ring_bookkeeping_from_three_producer_threads_under_the_thread_sanitizer(built):
    rc, out = _run(os.path.join(built, "ring_threads_tsan"), {"TSAN_OPTIONS": "halt_on_error=1:exitcode=66"})
    assert rc == 0 and "ring_threads ok" in out and "ThreadSanitizer" not in out, out
