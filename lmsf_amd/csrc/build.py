"""Compiles the HIP sources of this folder for gfx950 into one shared library, and the C++ host
sources under ``host/`` (cache manager, scheduler, step metadata; no GPU code) into another.

``build()`` always compiles. ``ensure_built()`` compiles only if no library matching the
sources is there (a fresh checkout, or a source changed since the last build); it is what the
loader calls, and it prints a line now and then while hipcc runs, so that a first call does
not look hung. The library is written beside the sources; if that folder cannot be written
(another user's checkout), a per-user folder under the system's temporary directory is used.
``build_host()`` / ``ensure_host_built()`` do the same for the host library, which needs a C++
compiler only and is what the CPU side of the engine runs on.
"""
import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import List, Optional

CSRC_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "liblmsf_hip.so"
OFFLOAD_ARCH = "gfx950"

# -packed-fp32-ops off: hipcc may otherwise form packed float32 instructions from scalar code.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=" + OFFLOAD_ARCH,
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=fast", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]

# Per source: the attention kernels rescale their accumulators with ordinary multiplications now and then, and
# with the accumulators in the registers that only the matrix cores reach the compiler copies all of them to and
# fro in every step of the loop; this keeps them where both can work on them.
EXTRA_FLAGS = {"attention_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def sources() -> List[str]:
    return sorted(f for f in os.listdir(CSRC_DIR) if f.endswith(".hip"))


def headers() -> List[str]:
    return sorted(f for f in os.listdir(CSRC_DIR) if f.endswith(".h"))


def source_digest() -> str:
    h = hashlib.sha256()
    for name in sources() + headers():
        h.update(name.encode())
        with open(os.path.join(CSRC_DIR, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(repr(sorted(EXTRA_FLAGS.items())).encode())
    return h.hexdigest()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                       "the HIP kernels of lmsf_amd cannot be built")


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, ".probe_%d" % os.getpid())
        with open(probe, "w"):
            pass
        os.unlink(probe)
        return True
    except OSError:
        return False


def _candidate_dirs() -> List[str]:
    fallback = os.path.join(tempfile.gettempdir(), "lmsf_amd_build_%d" % os.getuid())
    return [CSRC_DIR, fallback]


def _find(lib_name: str, digest: str) -> Optional[str]:
    for folder in _candidate_dirs():
        lib = os.path.join(folder, lib_name)
        stamp = lib + ".stamp"
        if os.path.isfile(lib) and os.path.isfile(stamp):
            try:
                with open(stamp) as f:
                    if f.read().strip() == digest:
                        return lib
            except OSError:
                pass
    return None


def find_library() -> Optional[str]:
    """Path of a built library whose stamp matches the current sources, or None."""
    return _find(LIB_NAME, source_digest())


def _say(msg: str) -> None:
    sys.stderr.write("[lmsf_amd build] %s\n" % msg)
    sys.stderr.flush()


def build(verbose: bool = True, jobs: Optional[int] = None) -> str:
    """Compile every .hip source and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the kernel library among %s" % _candidate_dirs())
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    if jobs is None:
        jobs = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
    digest = source_digest()
    t0 = time.time()
    if verbose:
        _say("compiling %d HIP sources for %s with %d jobs into %s" % (len(srcs), OFFLOAD_ARCH, jobs, out_dir))

    def compile_one(name: str):
        obj = os.path.join(obj_dir, name[:-4] + ".o")
        cmd = [hipcc] + HIPCC_FLAGS + EXTRA_FLAGS.get(name, []) + ["-I", CSRC_DIR, "-c", os.path.join(CSRC_DIR, name), "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        return name, obj, proc.returncode, proc.stdout

    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(compile_one, s) for s in srcs]
        pending = set(futures)
        while pending:
            done, pending = concurrent.futures.wait(pending, timeout=10.0,
                                                    return_when=concurrent.futures.FIRST_COMPLETED)
            for fut in done:
                name, obj, rc, log = fut.result()
                if rc != 0:
                    for p in pending:
                        p.cancel()
                    raise RuntimeError("hipcc failed on %s:\n%s" % (name, log))
                objs.append(obj)
                if verbose:
                    _say("compiled %s (%d/%d, %.0f s)" % (name, len(objs), len(srcs), time.time() - t0))
            if not done and verbose:
                _say("still compiling, %d of %d sources left (%.0f s)" % (len(pending), len(srcs), time.time() - t0))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + ".tmp%d" % os.getpid()
    cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=" + OFFLOAD_ARCH, "-o", tmp] + sorted(objs)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("linking %s failed:\n%s" % (LIB_NAME, proc.stdout))
    os.replace(tmp, lib)
    with open(lib + ".stamp", "w") as f:
        f.write(digest + "\n")
    if verbose:
        _say("built %s in %.0f s" % (lib, time.time() - t0))
    return lib


def ensure_built(verbose: bool = True) -> str:
    lib = find_library()
    if lib is not None:
        return lib
    return build(verbose=verbose)


# ---------------------------------------------------------------- the host library

HOST_DIR = os.path.join(CSRC_DIR, "host")
HOST_LIB_NAME = "liblmsf_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]


def host_sources() -> List[str]:
    return sorted(f for f in os.listdir(HOST_DIR) if f.endswith(".cc"))


def host_digest() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(HOST_DIR)):
        if name.endswith((".cc", ".h")):
            h.update(name.encode())
            with open(os.path.join(HOST_DIR, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()


def _cxx() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/llvm/bin/clang++"):
        if cand and (os.path.isfile(cand) or shutil.which(cand)):
            return cand
    raise RuntimeError("no C++ compiler found (looked at $CXX, g++, c++, clang++); the host library of lmsf_amd "
                       "cannot be built")


def build_host(verbose: bool = True) -> str:
    """Compile the host library; returns its path."""
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the host library among %s" % _candidate_dirs())
    digest = host_digest()
    lib = os.path.join(out_dir, HOST_LIB_NAME)
    tmp = lib + ".tmp%d" % os.getpid()
    t0 = time.time()
    cmd = [_cxx()] + HOST_FLAGS + ["-I", HOST_DIR, "-o", tmp] + [os.path.join(HOST_DIR, s) for s in host_sources()]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("compiling %s failed:\n%s" % (HOST_LIB_NAME, proc.stdout))
    os.replace(tmp, lib)
    with open(lib + ".stamp", "w") as f:
        f.write(digest + "\n")
    if verbose:
        _say("built %s in %.0f s" % (lib, time.time() - t0))
    return lib


def ensure_host_built(verbose: bool = True) -> str:
    lib = _find(HOST_LIB_NAME, host_digest())
    if lib is not None:
        return lib
    return build_host(verbose=verbose)


if __name__ == "__main__":
    print(build_host())
    print(build())
