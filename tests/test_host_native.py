"""The host library's C++ under AddressSanitizer and UBSan, driven by a native random workload (CPU only)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "leone_amd", "csrc", "host")


def test_random_workload_is_clean_under_sanitizers(tmp_path):
    compiler = shutil.which("g++") or shutil.which("clang++")
    if compiler is None:
        pytest.skip("no C++ compiler")
    sources = [os.path.join(HOST, f) for f in sorted(os.listdir(HOST)) if f.endswith(".cpp")]
    binary = str(tmp_path / "host_fuzz")
    build = subprocess.run([compiler, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-omit-frame-pointer",
                            "-I", HOST, os.path.join(ROOT, "tests", "native", "host_fuzz.cpp"), *sources, "-o", binary],
                           capture_output=True, text=True)
    if build.returncode != 0 and "sanitize" in build.stderr:
        pytest.skip("the sanitizer runtimes are not installed")
    assert build.returncode == 0, build.stderr
    # Another library may be preloaded in this environment; the sanitizer need not be the first one loaded.
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0",
               UBSAN_OPTIONS="halt_on_error=1")
    run = subprocess.run([binary], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout + run.stderr


def test_prompt_attention_workgroup_numbering_covers_every_pair_once(tmp_path):
    """Every (head, tile group) pair belongs to exactly one workgroup, for 1..64 heads and 1..32 groups
    (head counts that are no multiple of the eight dies once left heads out)."""
    compiler = shutil.which("g++") or shutil.which("clang++")
    if compiler is None:
        pytest.skip("no C++ compiler")
    binary = str(tmp_path / "prefill_order_check")
    build = subprocess.run([compiler, "-std=c++17", "-O1", "-I", os.path.join(ROOT, "leone_amd", "csrc"),
                            os.path.join(ROOT, "tests", "native", "prefill_order_check.cpp"), "-o", binary],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([binary], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout + run.stderr
