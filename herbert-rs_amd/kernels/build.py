"""Building the HIP modules for gfx950 and finding what is built.

Each module is one `.hip` file of `csrc/` compiled by hipcc into one shared
library with a C interface. The library's file name carries a hash of the
sources it was built from, so a library that no longer fits its source is never
loaded. A module that is not built is compiled when it is first asked for; a
line is printed when that starts and every few seconds while it runs.
"""
import hashlib
import os
import subprocess
import sys
import tempfile
import threading
import time

from ..errors import BackendError

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
MODULES = ("elementwise", "gemm_plain", "attention_plain", "sampling", "gemm_mfma", "attention_mfma",
           "random_weights")
# packed float32 instructions are kept out of every kernel
FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-shared", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
_locks = {m: threading.Lock() for m in MODULES}


def available_modules():
    return [m for m in MODULES if os.path.exists(os.path.join(CSRC, m + ".hip"))]


def _source_hash(name):
    h = hashlib.sha256()
    files = [name + ".hip"] + sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))
    for f in files:
        with open(os.path.join(CSRC, f), "rb") as fh:
            h.update(f.encode())
            h.update(fh.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:12]


def _library_name(name):
    return f"libhb_{name}.{_source_hash(name)}.so"


def _fallback_dir():
    d = os.path.join(tempfile.gettempdir(), f"herbert_rs_amd_build_{os.getuid()}")
    os.makedirs(d, exist_ok=True)
    return d


def find_library(name):
    """Path of the built library of a module, or None."""
    fname = _library_name(name)
    for d in (CSRC, _fallback_dir()):
        p = os.path.join(d, fname)
        if os.path.exists(p):
            return p
    return None


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_module(name, force=False, quiet=False):
    """Compile one module (if it is not built, or always with `force`); returns the path."""
    src = os.path.join(CSRC, name + ".hip")
    if not os.path.exists(src):
        raise BackendError(f"no kernel source {src}")
    with _locks.setdefault(name, threading.Lock()):
        if not force:
            found = find_library(name)
            if found:
                return found
        out_dir = CSRC if os.access(CSRC, os.W_OK) else _fallback_dir()
        target = os.path.join(out_dir, _library_name(name))
        tmp = target + f".tmp{os.getpid()}"
        cmd = [_hipcc()] + FLAGS + [src, "-o", tmp]
        t0 = time.time()
        if not quiet:
            print(f"[herbert_rs_amd] compiling {name}.hip for {ARCH} ...", file=sys.stderr, flush=True)
        env = dict(os.environ)
        env.setdefault("HOME", tempfile.gettempdir())
        try:
            proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env,
                                    cwd=out_dir)
        except FileNotFoundError:
            raise BackendError("hipcc not found: the HIP kernels cannot be built") from None
        chunks = []
        reader = threading.Thread(target=lambda: chunks.append(proc.stdout.read()), daemon=True)
        reader.start()
        while True:
            try:
                proc.wait(timeout=15)
                break
            except subprocess.TimeoutExpired:
                if not quiet:
                    print(f"[herbert_rs_amd] still compiling {name}.hip ({time.time() - t0:.0f} s)",
                          file=sys.stderr, flush=True)
        reader.join()
        log = (chunks[0] if chunks else b"").decode(errors="replace")
        if proc.returncode != 0:
            if os.path.exists(tmp):
                os.remove(tmp)
            lines = [l for l in log.splitlines() if "not a recognized feature" not in l]
            raise BackendError(f"hipcc failed on {name}.hip:\n" + "\n".join(lines[-40:]))
        os.replace(tmp, target)
        # older builds of this module are of no use any more
        for f in os.listdir(out_dir):
            if f.startswith(f"libhb_{name}.") and f.endswith(".so") and \
                    os.path.join(out_dir, f) != target:
                try:
                    os.remove(os.path.join(out_dir, f))
                except OSError:
                    pass
        if not quiet:
            print(f"[herbert_rs_amd] built {os.path.basename(target)} in {time.time() - t0:.0f} s",
                  file=sys.stderr, flush=True)
        return target


def build_all(force=True, quiet=False):
    """Compile every module, several hipcc processes at a time."""
    names = available_modules()
    errors = []

    def work(n):
        try:
            build_module(n, force, quiet)
        except BackendError as e:
            errors.append(str(e))

    threads = [threading.Thread(target=work, args=(n,)) for n in names]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise BackendError("\n".join(errors))
    return [find_library(n) for n in names]
