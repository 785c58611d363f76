"""The C++ cache manager and scheduler under AddressSanitizer and UndefinedBehaviorSanitizer: a host-only
build of csrc/runtime with a driver (tests/native/runtime_fuzz.cc) that pushes random workloads through
them, small pools included, and checks the manager's invariants after every step."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_runtime_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    cxx = shutil.which("g++")
    if cxx is None:
        pytest.skip("no g++ on this machine")
    rt = os.path.join(ROOT, "mini_llm_amd", "csrc", "runtime")
    exe = str(tmp_path / "runtime_fuzz")
    # (the sanitizers' runtimes are linked statically: they then need not be the first library of the process)
    build = subprocess.run([cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                            "-static-libasan", "-static-libubsan", "-I" + rt, os.path.join(ROOT, "tests", "native", "runtime_fuzz.cc"),
                            os.path.join(rt, "cache_manager.cc"), os.path.join(rt, "scheduler.cc"), "-o", exe],
                           capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe, "300"], capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0, run.stdout + run.stderr
    assert run.stdout.startswith("ok 300 runs") and "ERROR" not in run.stderr, run.stdout + run.stderr


def test_native_readers_survive_damaged_files_under_sanitizers(tmp_path):
    """The C++ safetensors reader and JSON parser (csrc/engine/weights.cc, json.cc) under the same
    sanitizers: thousands of damaged copies of a valid file (header bytes flipped, lengths and offsets
    changed, the file cut) are each either read or refused with an error, and random texts go through the
    JSON parser; no crash, no overflow, no read outside the mapped file."""
    cxx = shutil.which("g++")
    if cxx is None or not os.path.isdir("/opt/rocm/include"):
        pytest.skip("needs g++ and the HIP headers")
    import sys
    sys.path.insert(0, ROOT)
    from conftest import TINY_A
    from mini_llm_amd import write_random_model
    model = write_random_model(dict(TINY_A), str(tmp_path / "m"), seed=0)
    eng = os.path.join(ROOT, "mini_llm_amd", "csrc", "engine")
    exe = str(tmp_path / "loader_fuzz")
    build = subprocess.run([cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                            "-static-libasan", "-static-libubsan", "-x", "c++", "-D__HIP_PLATFORM_AMD__",
                            "-I/opt/rocm/include", "-I" + eng, "-I" + os.path.join(ROOT, "mini_llm_amd", "csrc", "runtime"),
                            os.path.join(ROOT, "tests", "native", "loader_fuzz.cc"), os.path.join(eng, "json.cc"),
                            os.path.join(eng, "weights.cc"), "-o", exe, "-L/opt/rocm/lib", "-lamdhip64",
                            "-Wl,-rpath,/opt/rocm/lib", "-lpthread"], capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe, os.path.join(model, "model.safetensors"), str(tmp_path / "scratch.safetensors"), "2000"],
                         capture_output=True, text=True, timeout=600,
                         env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0", UBSAN_OPTIONS="print_stacktrace=1"))
    assert run.returncode == 0 and run.stdout.startswith("ok:") and "ERROR" not in run.stderr, run.stdout + run.stderr
