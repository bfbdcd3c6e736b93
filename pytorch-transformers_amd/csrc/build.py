"""Compile the HIP sources in this folder into ``libpta_kernels.so`` for gfx950, and the host runtime
under ``host/`` (plain C++: slots, page lists, step layout) into ``libpta_host.so``.

``hipcc`` cross-compiles without a GPU.  Each ``.hip`` file becomes an object
(in parallel), then all are linked.  The library lies next to the sources when
that folder can be written, else in a per-user folder under the system's
temporary directory.  A text file beside it records a hash of the sources, so a
loader can tell a stale build from a current one.
"""
from __future__ import annotations

import concurrent.futures
import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libpta_kernels.so"
ARCH = "gfx950"
# packed 32-bit float instructions are switched off for every kernel of this library
# ... and matrix-core results go to ordinary vector registers: the kernels here do arithmetic on their
# accumulators between products, and copies to and from the accumulation registers cost more than they save
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-mllvm", "-amdgpu-mfma-vgpr-form", "-Wno-unused-command-line-argument"]


def sources():
    return sorted(glob.glob(os.path.join(HERE, "*.hip")))


def source_hash() -> str:
    h = hashlib.sha256()
    for p in sources() + sorted(glob.glob(os.path.join(HERE, "*.h"))):
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe{os.getpid()}")
        with open(probe, "w") as f:
            f.write("x")
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dirs():
    """Where the library may lie, in order of preference."""
    out = [HERE]
    try:
        user = str(os.getuid())
    except AttributeError:
        user = "user"
    out.append(os.path.join(tempfile.gettempdir(), f"pta_kernels_{user}_{source_hash()[:12]}"))
    return out


def find_library(require_current: bool = True):
    """Path of a built library (whose hash matches the sources if ``require_current``), or None."""
    want = source_hash()
    for d in lib_dirs():
        lib = os.path.join(d, LIB_NAME)
        if not os.path.isfile(lib):
            continue
        if not require_current:
            return lib
        try:
            with open(lib + ".hash") as f:
                if f.read().strip() == want:
                    return lib
        except OSError:
            pass
    return None


# ---- the host runtime: plain C++, no GPU code, needed on machines without a GPU too -------------
HOST_LIB_NAME = "libpta_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]


def host_sources():
    return sorted(glob.glob(os.path.join(HERE, "host", "*.cpp")))


def host_hash() -> str:
    h = hashlib.sha256()
    for p in host_sources():
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()


def host_lib_dirs():
    out = [HERE]
    try:
        user = str(os.getuid())
    except AttributeError:
        user = "user"
    out.append(os.path.join(tempfile.gettempdir(), f"pta_host_{user}_{host_hash()[:12]}"))
    return out


def find_host_library(require_current: bool = True):
    want = host_hash()
    for d in host_lib_dirs():
        lib = os.path.join(d, HOST_LIB_NAME)
        if not os.path.isfile(lib):
            continue
        if not require_current:
            return lib
        try:
            with open(lib + ".hash") as f:
                if f.read().strip() == want:
                    return lib
        except OSError:
            pass
    return None


def host_compiler() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/llvm/bin/clang++"):
        if cand and (os.path.isfile(cand) or shutil.which(cand)):
            return cand
    raise RuntimeError("no C++ compiler found for the host runtime (looked at $CXX, g++, c++, clang++)")


def build_host(verbose: bool = True) -> str:
    """Compile the host runtime (always) and return the library's path."""
    target_dir = next((d for d in host_lib_dirs() if _writable(d)), None)
    if target_dir is None:
        raise RuntimeError(f"no writable folder for {HOST_LIB_NAME}: tried {host_lib_dirs()}")
    lib = os.path.join(target_dir, HOST_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [host_compiler(), *HOST_FLAGS, "-o", tmp, *host_sources()]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"host runtime failed to compile:\n{' '.join(cmd)}\n{r.stdout}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(host_hash() + "\n")
    if verbose:
        print(f"[pta build] host runtime {lib}", file=sys.stderr, flush=True)
    return lib


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _compile_one(cc, src, obj, log):
    cmd = [cc, *FLAGS, "-I", HERE, "-c", src, "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {os.path.basename(src)}:\n{' '.join(cmd)}\n{r.stdout}")
    # the host pass does not know the packed-fp32 feature flag and says so; nothing else is expected
    noise = [ln for ln in r.stdout.splitlines() if ln.strip() and "packed-fp32-ops" not in ln and "not a recognized feature" not in ln]
    if noise and log:
        log(f"[pta build] {os.path.basename(src)}: " + " | ".join(noise[:6]))
    return obj


def build(verbose: bool = True, jobs: int | None = None) -> str:
    """Compile everything (always) and return the library's path."""
    log = (lambda s: print(s, file=sys.stderr, flush=True)) if verbose else None
    cc = hipcc()
    target_dir = next((d for d in lib_dirs() if _writable(d)), None)
    if target_dir is None:
        raise RuntimeError(f"no writable folder for {LIB_NAME}: tried {lib_dirs()}")
    obj_dir = os.path.join(target_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(16, os.cpu_count() or 1)))
    t0 = time.time()
    if log:
        log(f"[pta build] compiling {len(srcs)} HIP files for {ARCH} with {jobs} jobs into {target_dir}")
    objs = []
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        futs = {ex.submit(_compile_one, cc, s, os.path.join(obj_dir, os.path.basename(s)[:-4] + ".o"), log): s
                for s in srcs}
        for n, fut in enumerate(concurrent.futures.as_completed(futs), 1):
            objs.append(fut.result())
            if log:
                log(f"[pta build] {n}/{len(srcs)} {os.path.basename(futs[fut])} done ({time.time() - t0:.0f} s)")
    lib = os.path.join(target_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [cc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *sorted(objs)]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{' '.join(cmd)}\n{r.stdout}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(source_hash() + "\n")
    if log:
        log(f"[pta build] linked {lib} ({time.time() - t0:.0f} s)")
    return lib


if __name__ == "__main__":
    print(build_host())
    print(build())
