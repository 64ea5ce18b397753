"""Building the kernel library with hipcc for gfx950.

The sources under ``csrc/`` are compiled one process per file and linked into
``kernels/libhfamd.so`` inside the package (or, if the package folder cannot be
written, into a per-user folder under the system's temporary directory). A build
prints a line to stderr when it starts, every few seconds while it runs, and when
it ends.
"""
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(PKG, "csrc")
LIB_NAME = "libhfamd.so"
ARCH = "gfx950"
# -packed-fp32-ops off: the compiler must not form packed fp32 instructions.
# -ffp-contract=fast-honor-pragmas: products and sums are fused, except where a source says
# `#pragma clang fp contract(off)` (the sampler's draw, the random weights: bits the host must match).
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-ffp-contract=fast-honor-pragmas",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_hash():
    h = hashlib.sha256(" ".join(FLAGS).encode())
    for f in sorted(os.listdir(CSRC)):
        if f.endswith((".hip", ".h")):
            h.update(f.encode())
            with open(os.path.join(CSRC, f), "rb") as fh:
                h.update(fh.read())
    return h.hexdigest()


def _writable(path):
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dirs():
    """Where the library may lie: in the package first, then the per-user fallback."""
    return [os.path.join(PKG, "kernels"),
            os.path.join(tempfile.gettempdir(), f"hfamd-{os.getuid()}", "kernels")]


def find_library():
    """(path, is_current) of a built library, or (None, False)."""
    want = source_hash()
    found = None
    for d in lib_dirs():
        lib = os.path.join(d, LIB_NAME)
        if os.path.exists(lib):
            try:
                with open(lib + ".hash") as f:
                    if f.read().strip() == want:
                        return lib, True
            except OSError:
                pass
            found = found or lib
    return found, False


def build_extension(srcs, lib_path, verbose=True):
    """Compiles HIP sources of a part that lives outside the package (its own kernels) into a shared
    library of its own, with the flags the package's kernels are built with. Returns ``lib_path``."""
    hipcc = hipcc_path()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    os.makedirs(os.path.dirname(os.path.abspath(lib_path)), exist_ok=True)
    tmp = lib_path + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc] + FLAGS + ["-shared", "-o", tmp] + list(srcs), stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, env=env)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + r.stdout)
    os.replace(tmp, lib_path)
    if verbose:
        print(f"[hf_cpu_amd] extension library ready: {lib_path}", file=sys.stderr, flush=True)
    return lib_path


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                       "the kernel library cannot be built")


def build(verbose=True):
    """Compiles every source and links the library; returns its path."""
    hipcc = hipcc_path()
    out_dir = next((d for d in lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the kernel library: " + ", ".join(lib_dirs()))
    obj_dir = os.path.join(os.path.dirname(out_dir), "csrc", "_build") if out_dir.startswith(PKG) \
        else os.path.join(os.path.dirname(out_dir), "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    t0 = time.time()

    def say(msg):
        if verbose:
            print(f"[hf_cpu_amd] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(srcs)} kernel files for {ARCH} with {hipcc}")
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    procs = []
    for s in srcs:
        obj = os.path.join(obj_dir, s[:-4] + ".o")
        log = open(obj + ".log", "w")
        procs.append((s, obj, log, subprocess.Popen([hipcc] + FLAGS + ["-c", os.path.join(CSRC, s), "-o", obj],
                                                    stdout=log, stderr=subprocess.STDOUT, env=env)))
    last = time.time()
    while any(p.poll() is None for _, _, _, p in procs):
        time.sleep(0.2)
        if time.time() - last > 10:
            done = sum(p.poll() is not None for _, _, _, p in procs)
            say(f"compiling: {done}/{len(procs)} files done after {time.time() - t0:.0f} s")
            last = time.time()
    failed = []
    for s, obj, log, p in procs:
        log.close()
        if p.returncode != 0:
            with open(obj + ".log") as f:
                failed.append(f"{s}:\n{f.read()}")
    if failed:
        raise RuntimeError("hipcc failed:\n" + "\n".join(failed))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + [o for _, o, _, _ in procs],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if r.returncode != 0:
        raise RuntimeError("linking the kernel library failed:\n" + r.stdout)
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(source_hash() + "\n")
    say(f"kernel library ready after {time.time() - t0:.0f} s: {lib}")
    return lib
