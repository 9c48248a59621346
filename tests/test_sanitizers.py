"""AddressSanitizer + UndefinedBehaviorSanitizer over the code that runs on the CPU (no GPU needed):

* oracle/ckks_oracle.c: a sanitizer build of the checker is loaded by a child interpreter (sanitizer runtime
  preloaded) that runs the oracle's own pinning tests against it;
* the host layer's number theory, table construction and record parsing (hostmath.cpp, context.cpp, serialize.cpp):
  tests/sanitize/host_driver.cpp over the host-memory mock of the device ABI, ending with a bounded seeded loop of
  damaged and random records into every load() entry (it stops at the first report: the sanitizers abort).
"""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "lancelot_amd", "csrc", "host")
SAN = ["-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"]


def _runtime(name):
    path = subprocess.check_output(["gcc", "-print-file-name=" + name], text=True).strip()
    if not os.path.isabs(path) or not os.path.exists(path):
        pytest.skip("%s is not installed with this gcc" % name)
    return path


def test_oracle_under_asan_ubsan(tmp_path):
    asan = _runtime("libasan.so")
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-B", "libckks_oracle_san.so"],
                          stdout=subprocess.DEVNULL)
    env = dict(os.environ)
    env["CKKS_ORACLE_LIB"] = os.path.join(ROOT, "oracle", "libckks_oracle_san.so")
    # the runtime has to come first among the preloaded libraries; whatever is preloaded already stays
    env["LD_PRELOAD"] = ":".join([asan] + [p for p in env.get("LD_PRELOAD", "").split(":") if p])
    # the interpreter itself is not instrumented: its allocations at exit are not leaks of the checker
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    env["OMP_NUM_THREADS"] = "2"
    cmd = [sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
           os.path.join(ROOT, "tests", "test_oracle_scalar.py"), os.path.join(ROOT, "tests", "test_oracle_stages.py"),
           os.path.join(ROOT, "tests", "test_oracle_scheme.py")]
    proc = subprocess.run(cmd, env=env, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "passed" in proc.stdout and "ERROR: AddressSanitizer" not in proc.stdout and "runtime error" not in proc.stdout


def test_host_layer_under_asan_ubsan(tmp_path):
    _runtime("libasan.so")
    if not shutil.which("g++"):
        pytest.skip("no g++")
    exe = str(tmp_path / "host_driver")
    sources = [os.path.join(ROOT, "tests", "sanitize", "host_driver.cpp"), os.path.join(ROOT, "tests", "sanitize", "mock_device.cpp"),
               os.path.join(HOST, "hostmath.cpp"), os.path.join(HOST, "context.cpp"), os.path.join(HOST, "serialize.cpp")]
    subprocess.check_call(["g++", "-std=c++17", *SAN, "-I", os.path.join(ROOT, "include"), "-I", HOST, *sources, "-o", exe])
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "abort_on_error=1:detect_leaks=1"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    proc = subprocess.run([exe, "20000"], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "host sanitize driver ok" in proc.stdout
