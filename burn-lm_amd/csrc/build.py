"""Builds the two native libraries next to their sources.

* ``libburnlm_hip.so``: the HIP kernels for gfx950, one object per ``.hip`` source compiled in
  parallel by hipcc and linked.
* ``libburnlm_host.so``: the host-side core (cache bookkeeping, step assembly) from ``host/*.cpp``
  with the C++ compiler; it needs no GPU and no ROCm.

No other build system and no torch headers are involved; a first build takes well under a minute."""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libburnlm_hip.so"
ARCH = "gfx950"
# packed-fp32 instructions are kept off for every device pass
# (-Wno-inline-asm: the direct-load statements of common.h name m0 as clobbered, which the compiler
# answers with a warning per use because it keeps that register for itself)
# -amdgpu-kernarg-preload-count: a kernel's first 16 dwords of arguments arrive in scalar registers with
# the wavefront instead of being loaded by its first instructions (every kernel keeps a prologue that
# loads them for firmware that does not preload); worth 1-2.5 % of a decode step at 32 and 64 sequences.
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wno-inline-asm",
               "-mllvm", "-amdgpu-kernarg-preload-count=16",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# The matrix-core attention takes maxima of matrix-core results; told that they are no NaNs (masked
# scores are replaced by -infinity before any maximum, stale values are zeroed as integers) the
# compiler drops a quieting instruction in front of every maximum, 13 of 130 vector instructions
# per page.
PER_FILE_FLAGS = {"attention_mfma.hip": ["-fno-honor-nans"]}


def sources():
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def source_hash():
    h = hashlib.sha256()
    for name in sources() + sorted(f for f in os.listdir(HERE) if f.endswith(".h")):
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(repr(sorted(PER_FILE_FLAGS.items())).encode())
    return h.hexdigest()


HOST_LIB_NAME = "libburnlm_host.so"
HOST_DIR = os.path.join(HERE, "host")
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]


def host_sources():
    return sorted(f for f in os.listdir(HOST_DIR) if f.endswith(".cpp"))


def host_hash():
    h = hashlib.sha256()
    for name in sorted(os.listdir(HOST_DIR)):
        if name.endswith((".cpp", ".h")):
            h.update(name.encode())
            with open(os.path.join(HOST_DIR, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()


def _writable(d):
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def out_dir():
    """In-tree when the checkout is writable, else a per-user folder under the temp dir."""
    if _writable(os.path.join(HERE, "_build")):
        return HERE
    d = os.path.join(tempfile.gettempdir(), f"burnlm_amd_{os.getuid()}_{source_hash()[:12]}")
    os.makedirs(os.path.join(d, "_build"), exist_ok=True)
    return d


def lib_path():
    return os.path.join(out_dir(), LIB_NAME)


def _hash_path():
    return os.path.join(out_dir(), "_build", "source.sha256")


def is_current():
    try:
        with open(_hash_path()) as f:
            return os.path.exists(lib_path()) and f.read().strip() == source_hash()
    except OSError:
        return False


def host_lib_path():
    return os.path.join(out_dir(), HOST_LIB_NAME)


def _host_hash_path():
    return os.path.join(out_dir(), "_build", "host.sha256")


def host_is_current():
    try:
        with open(_host_hash_path()) as f:
            return os.path.exists(host_lib_path()) and f.read().strip() == host_hash()
    except OSError:
        return False


def find_cxx():
    for cand in (os.environ.get("CXX"), "g++", "c++", "clang++", "/opt/rocm/llvm/bin/clang++"):
        path = cand and (cand if os.path.isabs(cand) and os.path.exists(cand) else shutil.which(cand))
        if path:
            return path
    raise RuntimeError("no C++ compiler found (looked at $CXX, g++, c++, clang++): the host library cannot be built")


def build_host(verbose=True):
    """Compile the host-side core.  Always compiles; returns the library path."""
    cxx = find_cxx()
    od = out_dir()
    tmp = os.path.join(od, "_build", HOST_LIB_NAME + f".{os.getpid()}.tmp")
    t0 = time.time()
    r = subprocess.run([cxx, *HOST_FLAGS, "-I", HOST_DIR, *[os.path.join(HOST_DIR, s) for s in host_sources()], "-o", tmp],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"{cxx} failed on the host library:\n{r.stdout}")
    os.replace(tmp, os.path.join(od, HOST_LIB_NAME))
    with open(_host_hash_path(), "w") as f:
        f.write(host_hash())
    if verbose:
        print(f"[burn-lm_amd build] built {os.path.join(od, HOST_LIB_NAME)} in {time.time() - t0:.1f} s",
              file=sys.stderr, flush=True)
    return os.path.join(od, HOST_LIB_NAME)


REF_LIB_NAME = "libburnlm_ref.so"
REF_DIR = os.path.join(HERE, "ref")


def ref_hash():
    h = hashlib.sha256()
    for name in sorted(os.listdir(REF_DIR)):
        if name.endswith((".cpp", ".h")):
            h.update(name.encode())
            with open(os.path.join(REF_DIR, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()


def ref_lib_path():
    return os.path.join(out_dir(), REF_LIB_NAME)


def build_ref(verbose=True):
    """Compile the plain C++ references of the kernels (ref/*.cpp; the kernel tests compare against
    them).  No GPU and no ROCm needed.  Always compiles; returns the library path."""
    cxx = find_cxx()
    od = out_dir()
    tmp = os.path.join(od, "_build", REF_LIB_NAME + f".{os.getpid()}.tmp")
    t0 = time.time()
    srcs = [os.path.join(REF_DIR, s) for s in sorted(os.listdir(REF_DIR)) if s.endswith(".cpp")]
    r = subprocess.run([cxx, *HOST_FLAGS, "-I", REF_DIR, *srcs, "-o", tmp], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"{cxx} failed on the reference library:\n{r.stdout}")
    os.replace(tmp, ref_lib_path())
    with open(os.path.join(od, "_build", "ref.sha256"), "w") as f:
        f.write(ref_hash())
    if verbose:
        print(f"[burn-lm_amd build] built {ref_lib_path()} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return ref_lib_path()


def ensure_ref_built(verbose=True):
    try:
        with open(os.path.join(out_dir(), "_build", "ref.sha256")) as f:
            if os.path.exists(ref_lib_path()) and f.read().strip() == ref_hash():
                return ref_lib_path()
    except OSError:
        pass
    return build_ref(verbose=verbose)


def ensure_host_built(verbose=True):
    if host_is_current():
        return host_lib_path()
    _refuse_under_profiler(HOST_LIB_NAME)
    return build_host(verbose=verbose)


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernel "
                       "library cannot be built, and there is no fallback path without it")


def build(verbose=True, jobs=None, with_ref=False):
    """Compile every HIP source and link the kernel library, and compile the host library.  Always
    compiles; returns the kernel library's path.  with_ref: the plain C++ references that the kernel
    tests use are compiled along (a model's first call does not need them)."""
    build_host(verbose=verbose)
    if with_ref:
        build_ref(verbose=verbose)
    hipcc = find_hipcc()
    od = out_dir()
    bdir = os.path.join(od, "_build")
    srcs = sources()
    jobs = jobs or min(len(srcs), 8)
    log = (lambda *a: print("[burn-lm_amd build]", *a, file=sys.stderr, flush=True)) if verbose else (lambda *a: None)
    log(f"compiling {len(srcs)} HIP sources for {ARCH} with {hipcc} ({jobs} at a time)")
    t0 = time.time()
    pending = list(srcs)
    running = {}
    objs = []
    last_note = time.time()
    while pending or running:
        while pending and len(running) < jobs:
            s = pending.pop(0)
            o = os.path.join(bdir, s[:-4] + ".o")
            objs.append(o)
            # the compiler writes into a file, not a pipe: nobody reads while it runs, and a pipe that
            # fills up (a warning per template instance is enough) would stop it for good
            said = open(os.path.join(bdir, s[:-4] + ".log"), "w+")
            p = subprocess.Popen([hipcc, *HIPCC_FLAGS, *PER_FILE_FLAGS.get(s, []), "-I", HERE, "-c", os.path.join(HERE, s), "-o", o],
                                 stdout=said, stderr=subprocess.STDOUT, stdin=subprocess.DEVNULL)
            running[s] = (p, said)
        for s, (p, said) in list(running.items()):
            if p.poll() is not None:
                said.seek(0)
                out = said.read()
                said.close()
                del running[s]
                if p.returncode != 0:
                    for q, _ in running.values():
                        q.kill()
                    raise RuntimeError(f"hipcc failed on {s}:\n{out}")
                log(f"  {s} done ({time.time() - t0:.0f} s)")
        if running and time.time() - last_note > 15:
            log(f"  still compiling: {', '.join(sorted(running))} ({time.time() - t0:.0f} s)")
            last_note = time.time()
        time.sleep(0.05)
    tmp = os.path.join(bdir, LIB_NAME + f".{os.getpid()}.tmp")
    r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc link failed:\n{r.stdout}")
    os.replace(tmp, os.path.join(od, LIB_NAME))
    with open(_hash_path(), "w") as f:
        f.write(source_hash())
    log(f"built {os.path.join(od, LIB_NAME)} in {time.time() - t0:.0f} s")
    return os.path.join(od, LIB_NAME)


def under_profiler():
    """Whether this process runs under a profiler that preloads a tool library into every child (rocprofv3
    does): a compiler started from here would load it too and start collecting on its own."""
    env = os.environ
    return ("rocprof" in env.get("LD_PRELOAD", "").lower() or
            any(k.startswith(("ROCPROF", "ROCP_TOOL", "ROCPROFILER")) for k in env))


def _refuse_under_profiler(what):
    if under_profiler():
        raise RuntimeError(f"{what} does not match its sources and would have to be compiled, but this process runs "
                           f"under a profiler whose preloaded library every compiler process would inherit: build first "
                           f"(python -c 'import __graft_entry__ as g; g.build()'), then profile")


def ensure_built(verbose=True):
    """Path of a library that matches the sources, building it first if there is none."""
    if is_current():
        return lib_path()
    _refuse_under_profiler(LIB_NAME)
    return build(verbose=verbose)


if __name__ == "__main__":
    print(build())
