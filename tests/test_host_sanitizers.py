"""The C++ host runtime under AddressSanitizer and UndefinedBehaviorSanitizer: a driver program
(host_sanitizer_driver.cc) is compiled together with the library's sources and run over random workloads
that reach admission, portions, decoding, preemption, refusal, capping, abort, failed steps and the error
paths. Host code only: nothing here touches a GPU."""
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_DIR = os.path.join(ROOT, "lmsf_amd", "csrc", "host")


def _compiler():
    for cand in (os.environ.get("CXX"), "g++", "clang++"):
        if cand and shutil.which(cand):
            return shutil.which(cand)
    return None


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    cxx = _compiler()
    if cxx is None:
        pytest.skip("no C++ compiler")
    out = str(tmp_path_factory.mktemp("san") / "host_san")
    cmd = [cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-I", HOST_DIR, os.path.join(ROOT, "tests", "host_sanitizer_driver.cc")] + sorted(
               glob.glob(os.path.join(HOST_DIR, "*.cc"))) + ["-o", out]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    if proc.returncode != 0 and "sanitize" in proc.stdout and ("cannot find" in proc.stdout or "unsupported" in proc.stdout):
        pytest.skip("the sanitizer runtimes are not installed: %s" % proc.stdout[-300:])
    assert proc.returncode == 0, proc.stdout[-3000:]
    return out


@pytest.mark.parametrize("seed", [1, 2, 3, 20260101])
def test_host_runtime_is_clean_under_the_sanitizers(driver, seed):
    if os.environ.get("LD_PRELOAD"):
        pytest.skip("a preloaded library is in the environment: the sanitizer's runtime has to come first")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([driver, str(seed)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300,
                          env=env)
    if proc.returncode != 0 and "does not come first in initial library list" in proc.stderr:
        pytest.skip("a library is preloaded into every process here: the sanitizer's runtime cannot come first")
    assert proc.returncode == 0, (proc.stdout[-1000:], proc.stderr[-3000:])
    assert proc.stdout.startswith("OK steps="), proc.stdout
    assert "runtime error" not in proc.stderr and "AddressSanitizer" not in proc.stderr, proc.stderr[-3000:]
    fields = dict(kv.split("=") for kv in proc.stdout.split()[1:])
    assert int(fields["preemptions"]) > 0 and int(fields["finished"]) > 50 and int(fields["aborted"]) > 0
