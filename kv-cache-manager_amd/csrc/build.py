"""Compiles the two native libraries and finds them again.

  libkvcm_host.so   C++17, no GPU dependency: allocator, prefix cache, managers, scheduler
  libkvcm_hip.so    HIP kernels for gfx950, one C entry point per launch

Both are built in-tree under ``csrc/_lib`` (or, when the tree is read-only, in a per-user
folder under the temp dir).  A stamp file holds a hash of the sources and flags: a library is
loaded as it is when its stamp matches and rebuilt when it does not and a compiler is there.
"""
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

HERE = os.path.dirname(os.path.abspath(__file__))
HOST_DIR = os.path.join(HERE, "host")
HIP_DIR = os.path.join(HERE, "hip")
GPU_ARCH = "gfx950"

HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra"]
# packed fp32 instructions stay off: -O3 would otherwise form them from plain float code
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={GPU_ARCH}", "-Xclang", "-target-feature",
             "-Xclang", "-packed-fp32-ops", "-Wno-unused-result", "-ffp-contract=fast"]


# the vendor library's matrix product (prompt steps), as the reference links cuBLAS
HIP_LINK = ["-lhipblaslt"]


def _say(msg):
    print(f"[kvcm build] {msg}", file=sys.stderr, flush=True)


def _sources(folder, exts):
    return sorted(os.path.join(folder, f) for f in os.listdir(folder) if f.endswith(exts))


def _digest(paths, flags):
    h = hashlib.sha256(" ".join(flags).encode())
    for p in paths:
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _lib_dirs():
    yield os.path.join(HERE, "_lib")
    yield os.path.join(tempfile.gettempdir(), f"kvcm_lib_{os.getuid()}")


def _writable_lib_dir():
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe{os.getpid()}")
            with open(probe, "w") as f:
                f.write("x")
            os.remove(probe)
            return d
        except OSError:
            continue
    raise RuntimeError("no writable folder for the native libraries")


def _find_built(name, digest):
    for d in _lib_dirs():
        lib, stamp = os.path.join(d, name), os.path.join(d, name + ".stamp")
        if os.path.exists(lib) and os.path.exists(stamp):
            with open(stamp) as f:
                if f.read().strip() == digest:
                    return lib
    return None


def _find_any(name):
    for d in _lib_dirs():
        lib = os.path.join(d, name)
        if os.path.exists(lib):
            return lib
    return None


def _run(cmd, what):
    """Runs a compiler, printing a line every 20 s so that a long build does not look hung."""
    done = threading.Event()

    def ticker():
        t0 = time.time()
        while not done.wait(20.0):
            _say(f"still compiling {what} ({time.time() - t0:.0f} s)")

    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    try:
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    finally:
        done.set()
    if r.returncode != 0:
        raise RuntimeError(f"compiling {what} failed:\n{' '.join(cmd)}\n{r.stdout}")
    return r.stdout


def _hipcc():
    for c in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.exists(c):
            return c
    return None


def build_host(force=False):
    srcs = _sources(HOST_DIR, (".cpp",))
    deps = _sources(HOST_DIR, (".cpp", ".h"))
    digest = _digest(deps, HOST_FLAGS)
    name = "libkvcm_host.so"
    if not force:
        lib = _find_built(name, digest)
        if lib:
            return lib
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if not cxx:
        lib = _find_any(name)
        if lib:
            return lib
        raise RuntimeError("no C++ compiler found to build libkvcm_host.so")
    out_dir = _writable_lib_dir()
    lib = os.path.join(out_dir, name)
    tmp = lib + f".tmp{os.getpid()}"
    _say(f"compiling host core -> {lib}")
    _run([cxx] + HOST_FLAGS + ["-I", HOST_DIR] + srcs + ["-o", tmp], "host core")
    os.replace(tmp, lib)
    with open(lib + ".stamp", "w") as f:
        f.write(digest)
    return lib


def build_hip(force=False, jobs=None):
    srcs = _sources(HIP_DIR, (".hip",))
    deps = _sources(HIP_DIR, (".hip", ".h"))
    digest = _digest(deps, HIP_FLAGS + HIP_LINK)
    name = "libkvcm_hip.so"
    if not force:
        lib = _find_built(name, digest)
        if lib:
            return lib
    hipcc = _hipcc()
    if not hipcc:
        lib = _find_any(name)
        if lib:
            _say("hipcc not found; loading the library that is there although its sources changed")
            return lib
        raise RuntimeError("hipcc not found and libkvcm_hip.so is not built: the engine has no "
                           "fallback for its HIP kernels")
    out_dir = _writable_lib_dir()
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    lib = os.path.join(out_dir, name)
    _say(f"compiling {len(srcs)} HIP sources for {GPU_ARCH} -> {lib}")
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    objs, errors = [], []
    lock = threading.Lock()
    todo = list(srcs)

    def worker():
        while True:
            with lock:
                if not todo or errors:
                    return
                src = todo.pop()
            obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
            try:
                t0 = time.time()
                _run([hipcc] + HIP_FLAGS + ["-I", HIP_DIR, "-c", src, "-o", obj], os.path.basename(src))
                _say(f"  {os.path.basename(src)} done in {time.time() - t0:.0f} s")
                with lock:
                    objs.append(obj)
            except Exception as e:  # noqa: BLE001
                with lock:
                    errors.append(e)

    threads = [threading.Thread(target=worker) for _ in range(jobs)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    tmp = lib + f".tmp{os.getpid()}"
    _run([hipcc, "-shared", "-fPIC", f"--offload-arch={GPU_ARCH}"] + sorted(objs) + HIP_LINK + ["-o", tmp], "link")
    os.replace(tmp, lib)
    with open(lib + ".stamp", "w") as f:
        f.write(digest)
    _say("HIP library ready")
    return lib


def build_all(force=False):
    return build_host(force), build_hip(force)


if __name__ == "__main__":
    print(build_all(force="--force" in sys.argv))
