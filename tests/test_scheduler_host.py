"""Builds and runs the host-only tests of the scheduler (tests/cpp/test_scheduler.cpp) and
of the search driver above it (tests/cpp/test_search.cpp) with stand-in executors, once
plainly and once under the thread sanitizer."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = [os.path.join(ROOT, "tests", "cpp", "test_scheduler.cpp"),
       os.path.join(ROOT, "leela-zero_amd", "csrc", "hip_scheduler.cpp")]
INC = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "leela-zero_amd", "csrc")]


CSRC = os.path.join(ROOT, "leela-zero_amd", "csrc")
SEARCH_SRC = [os.path.join(ROOT, "tests", "cpp", "test_search.cpp")] + \
    [os.path.join(CSRC, f) for f in ("hip_scheduler.cpp", "search.cpp", "goboard.cpp")]


def build_and_run(tmp_path, extra, env_extra=None, src=None):
    exe = str(tmp_path / "host_test")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-pthread"] + extra + INC + (src or SRC) + ["-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    env = dict(os.environ)
    env.pop("LD_PRELOAD", None)
    env.update(env_extra or {})
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    return r


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_scheduler_plain(tmp_path):
    r = build_and_run(tmp_path, [])
    assert r.returncode == 0, r.stdout + r.stderr
    assert "scheduler tests passed" in r.stdout


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_scheduler_under_thread_sanitizer(tmp_path):
    r = build_and_run(tmp_path, ["-fsanitize=thread"], {"TSAN_OPTIONS": "halt_on_error=1"})
    if "unexpected memory mapping" in r.stderr or "FATAL: ThreadSanitizer" in r.stderr:
        pytest.skip("thread sanitizer cannot start in this sandbox: " + r.stderr[:200])
    assert r.returncode == 0, r.stdout + r.stderr
    assert "WARNING: ThreadSanitizer" not in r.stderr
    assert "scheduler tests passed" in r.stdout


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_search_plain(tmp_path):
    r = build_and_run(tmp_path, [], src=SEARCH_SRC)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "search tests passed" in r.stdout


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_search_under_thread_sanitizer(tmp_path):
    r = build_and_run(tmp_path, ["-fsanitize=thread"], {"TSAN_OPTIONS": "halt_on_error=1"},
                      src=SEARCH_SRC)
    if "unexpected memory mapping" in r.stderr or "FATAL: ThreadSanitizer" in r.stderr:
        pytest.skip("thread sanitizer cannot start in this sandbox: " + r.stderr[:200])
    assert r.returncode == 0, r.stdout + r.stderr
    assert "WARNING: ThreadSanitizer" not in r.stderr
    assert "search tests passed" in r.stdout
