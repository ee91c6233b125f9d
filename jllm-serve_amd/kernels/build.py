"""Builds the HIP sources under csrc/ into one shared library for gfx950 with hipcc, and the host-side C++ sources
under csrc/host/ into a second one with the C++ compiler (no GPU code: it loads anywhere).

The library lives in ``<package>/_build/`` (next to the sources, so it travels with the tree); when that
folder cannot be written the build goes to a per-user folder under the system's temporary directory. A
digest of the sources and flags is stored beside the library; ``ensure_built`` compiles only when no
library with the current digest exists.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libjllm_kernels.so"
ARCH = "gfx950"
# packed fp32 VALU forms are switched off for every device compile of this project
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-unused-result",
         # the loads that write LDS directly are written out as instructions and name m0 among what they change,
         # which the compiler remarks on at every use
         "-Wno-inline-asm"]
# per source: the decode attention multiplies its MFMA accumulators by the softmax rescale now and then; kept in
# the accumulator half of the register file they would be moved there and back at every turn of the loop
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
FILE_FLAGS = {"attention_decode.hip": VGPR_FORM, "gemm_skinny.hip": VGPR_FORM}


def sources():
    return sorted(f for f in os.listdir(SRC_DIR) if f.endswith(".hip"))


def headers():
    return sorted(f for f in os.listdir(SRC_DIR) if f.endswith(".h"))


def digest() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    for f in sources() + headers():
        h.update(f.encode())
        with open(os.path.join(SRC_DIR, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def _candidates():
    yield os.path.join(PKG_DIR, "_build")
    yield os.path.join(tempfile.gettempdir(), f"jllm_serve_amd_build_{os.getuid()}")


def find_library(require_current: bool = True):
    d = digest()
    for folder in _candidates():
        lib = os.path.join(folder, LIB_NAME)
        stamp = os.path.join(folder, "digest.txt")
        if os.path.exists(lib) and (folder.startswith(PKG_DIR) or _trusted(folder)):
            if not require_current:
                return lib
            try:
                with open(stamp) as f:
                    if f.read().strip() == d:
                        return lib
            except OSError:
                pass
    return None


def _hipcc() -> str:
    for c in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.exists(c):
            return c
    raise RuntimeError("hipcc not found: the kernels of this engine are HIP sources and need the ROCm compiler")


def _trusted(folder: str) -> bool:
    """A folder under the shared temporary directory is used only when it belongs to this user and nobody else may
    write to it: a library found there is loaded into the process."""
    try:
        st = os.stat(folder)
    except OSError:
        return False
    return st.st_uid == os.getuid() and not (st.st_mode & 0o022)


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, mode=0o700, exist_ok=True)
        if not folder.startswith(PKG_DIR) and not _trusted(folder):
            return False
        probe = os.path.join(folder, f".probe_{os.getpid()}")
        with open(probe, "w") as f:
            f.write("x")
        os.remove(probe)
        return True
    except OSError:
        return False


def build(verbose: bool = True) -> str:
    """Compiles every source and links the library; returns its path."""
    hipcc = _hipcc()
    folder = next((f for f in _candidates() if _writable(f)), None)
    if folder is None:
        raise RuntimeError("no writable folder for the kernel build")
    srcs = sources()
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # hipcc wants a home for its caches

    def log(msg):
        if verbose:
            print(f"[jllm build] {msg}", file=sys.stderr, flush=True)

    log(f"compiling {len(srcs)} HIP sources for {ARCH} into {folder}")

    # objects go to a folder of this process: two first runs at once (test workers, a bench beside the tests) never
    # link each other's half-written files; only finished files are moved into place
    work = tempfile.mkdtemp(prefix=f"obj_{os.getpid()}_", dir=folder)

    def compile_one(src):
        obj = os.path.join(work, src[:-4] + ".o")
        tail = ["-I", SRC_DIR, "-c", os.path.join(SRC_DIR, src), "-o", obj]
        r = subprocess.run([hipcc] + FLAGS + FILE_FLAGS.get(src, []) + tail, stdout=subprocess.PIPE,
                           stderr=subprocess.STDOUT, text=True, env=env)
        if r.returncode != 0 and src in FILE_FLAGS and "Unknown command line argument" in r.stdout:
            # a compiler without the option: the kernel is the same, only slower
            log(f"  {src}: this hipcc does not know {' '.join(FILE_FLAGS[src])}; compiling without")
            r = subprocess.run([hipcc] + FLAGS + tail, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
        out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        log(f"  {src} done ({time.time() - t0:.0f} s)" + (("\n" + out) if out.strip() else ""))
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16))
    try:
        with concurrent.futures.ThreadPoolExecutor(workers) as ex:
            objs = list(ex.map(compile_one, srcs))
    except BaseException:
        shutil.rmtree(work, ignore_errors=True)
        raise
    lib = os.path.join(folder, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    shutil.rmtree(work, ignore_errors=True)
    if r.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{r.stdout}")
    os.replace(tmp, lib)
    stamp = os.path.join(folder, f"digest.txt.tmp{os.getpid()}")
    with open(stamp, "w") as f:
        f.write(digest())
    os.replace(stamp, os.path.join(folder, "digest.txt"))
    log(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


HOST_DIR = os.path.join(SRC_DIR, "host")
HOST_LIB_NAME = "libjllm_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"]


def host_sources():
    return sorted(f for f in os.listdir(HOST_DIR) if f.endswith(".cpp"))


def host_digest() -> str:
    h = hashlib.sha256()
    h.update(" ".join(HOST_FLAGS).encode())
    for f in sorted(os.listdir(HOST_DIR)):
        if f.endswith((".cpp", ".h")):
            h.update(f.encode())
            with open(os.path.join(HOST_DIR, f), "rb") as fh:
                h.update(fh.read())
    return h.hexdigest()


def find_host_library():
    d = host_digest()
    for folder in _candidates():
        lib = os.path.join(folder, HOST_LIB_NAME)
        if os.path.exists(lib) and (folder.startswith(PKG_DIR) or _trusted(folder)):
            try:
                with open(os.path.join(folder, "host_digest.txt")) as f:
                    if f.read().strip() == d:
                        return lib
            except OSError:
                pass
    return None


def build_host(verbose: bool = True) -> str:
    """Compiles the host-side sources (page pool, step layout) into their library; returns its path."""
    cxx = next((c for c in (shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"), "/opt/rocm/llvm/bin/clang++")
                if c and os.path.exists(c)), None)
    if cxx is None:
        raise RuntimeError("no C++ compiler found (g++, c++ or clang++): the engine's host library is C++")
    folder = next((f for f in _candidates() if _writable(f)), None)
    if folder is None:
        raise RuntimeError("no writable folder for the host library build")
    lib = os.path.join(folder, HOST_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    t0 = time.time()
    r = subprocess.run([cxx] + HOST_FLAGS + ["-I", HOST_DIR] + [os.path.join(HOST_DIR, f) for f in host_sources()] + ["-o", tmp],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building {HOST_LIB_NAME} failed:\n{r.stdout}")
    os.replace(tmp, lib)
    stamp = os.path.join(folder, f"host_digest.txt.tmp{os.getpid()}")
    with open(stamp, "w") as f:
        f.write(host_digest())
    os.replace(stamp, os.path.join(folder, "host_digest.txt"))
    if verbose:
        print(f"[jllm build] built {lib} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return lib


SANITIZE_FLAGS = ["-O1", "-g", "-std=c++17", "-Wall", "-fsanitize=address,undefined", "-fno-omit-frame-pointer",
                  "-fno-sanitize-recover=undefined"]


def build_host_check(folder: str, sanitize: bool = True) -> str:
    """Compiles the host-side sources together with their hammer (csrc/host/check/hammer.cpp) into an executable in
    ``folder``, under AddressSanitizer and UndefinedBehaviorSanitizer unless ``sanitize`` is off; returns its path.
    CPU only: the program touches no GPU."""
    cxx = next((c for c in (shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")) if c), None)
    if cxx is None:
        raise RuntimeError("no C++ compiler found (g++, c++ or clang++)")
    exe = os.path.join(folder, "jllm_host_hammer")
    flags = list(SANITIZE_FLAGS) if sanitize else ["-O1", "-std=c++17", "-Wall"]
    if sanitize and "clang" not in os.path.basename(cxx):
        flags.append("-static-libasan")  # the runtime inside the program: nothing preloaded can come before it
    srcs = [os.path.join(HOST_DIR, f) for f in host_sources()] + [os.path.join(HOST_DIR, "check", "hammer.cpp")]
    r = subprocess.run([cxx] + flags + ["-I", HOST_DIR] + srcs + ["-o", exe], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building the host hammer failed:\n{r.stdout}")
    return exe


def ensure_host_built(verbose: bool = True) -> str:
    return find_host_library() or build_host(verbose)


def ensure_built(verbose: bool = True) -> str:
    lib = find_library()
    if lib is None:
        lib = build(verbose)
    return lib


if __name__ == "__main__":
    print(build_host())
    print(build())
