"""Host-only sanitizer runs of the two pieces of host logic where memory or threading mistakes would hide: the static
GEMM planner (ASan + UBSan over random problems) and the copy-thread pool of the pageable-operand path (TSan).  The
harnesses live in tests/sanitize/ and are compiled here with g++ straight from the library's host sources; nothing
touches a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "paralia-framework_amd", "csrc")
INC = ["-I", os.path.join(ROOT, "include"), "-I", CSRC]


def _build(tmp_path, name, sources, flags):
    if shutil.which("g++") is None:
        pytest.skip("g++ not available")
    exe = str(tmp_path / name)
    cmd = ["g++", "-O1", "-g", "-std=c++17", "-pthread"] + flags + INC + sources + ["-o", exe]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    if run.returncode != 0 and ("cannot find -l" in run.stderr or "unrecognized" in run.stderr):
        pytest.skip("sanitizer runtime not installed: " + run.stderr[-200:])
    assert run.returncode == 0, run.stderr[-3000:]
    return exe


def test_planner_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    exe = _build(tmp_path, "plan_fuzz", [os.path.join(ROOT, "tests", "sanitize", "plan_fuzz.cpp"), os.path.join(CSRC, "runtime", "gemm_plan.cpp")],
                 ["-fsanitize=address,undefined", "-fno-sanitize-recover=all"])
    run = subprocess.run([exe, "600"], capture_output=True, text=True, timeout=900,
                         env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1:verify_asan_link_order=0"))
    assert run.returncode == 0, (run.stdout[-500:], run.stderr[-3000:])
    assert "built" in run.stdout and "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr


def test_order_search_threads_under_thread_sanitizer(tmp_path):
    """The order search deals its candidate plans to a few worker threads; the same fuzzer under TSan, with the pool
    forced to four threads whatever the machine has, and the small-work shortcut left to chance by the problem sizes."""
    exe = _build(tmp_path, "plan_fuzz_tsan", [os.path.join(ROOT, "tests", "sanitize", "plan_fuzz.cpp"), os.path.join(CSRC, "runtime", "gemm_plan.cpp")],
                 ["-fsanitize=thread"])
    run = subprocess.run([exe, "400"], capture_output=True, text=True, timeout=900, env=dict(os.environ, PARALIA_PLAN_THREADS="4"))
    if "FATAL: ThreadSanitizer: unexpected memory mapping" in run.stderr:
        pytest.skip("ThreadSanitizer cannot map its shadow memory in this container")
    assert run.returncode == 0, (run.stdout[-500:], run.stderr[-3000:])
    assert "built" in run.stdout and "ThreadSanitizer" not in run.stderr


def test_copy_thread_pool_under_thread_sanitizer(tmp_path):
    exe = _build(tmp_path, "copy_threads", [os.path.join(ROOT, "tests", "sanitize", "copy_threads.cpp"), os.path.join(CSRC, "runtime", "host_staging.cpp")],
                 ["-fsanitize=thread"])
    run = subprocess.run([exe], capture_output=True, text=True, timeout=900)
    if "FATAL: ThreadSanitizer: unexpected memory mapping" in run.stderr:
        pytest.skip("ThreadSanitizer cannot map its shadow memory in this container")
    assert run.returncode == 0, (run.stdout[-500:], run.stderr[-3000:])
    assert "ok" in run.stdout and "ThreadSanitizer: data race" not in run.stderr
