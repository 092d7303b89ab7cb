"""Compile the HIP sources under `arle_amd/csrc` into shared libraries for gfx950, and the
host-side C++ runtime core (`csrc/host/`, no GPU code) with the host compiler.

One library per source file, built with plain `hipcc` (no torch headers, so a
file compiles in seconds).  Libraries live in `arle_amd/_lib/`, or in a per-user
folder under the system temp folder when the package folder is not writable.
A library is rebuilt when the hash of its sources differs from the one recorded
beside it; otherwise it is loaded as it is.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC_DIR = os.path.join(PACKAGE_DIR, "csrc")
OFFLOAD_ARCH = "gfx950"

# library name -> source file (all include common.h)
SOURCES = {
    "elementwise": "elementwise.hip",
    "norm": "norm.hip",
    "gemm_f32": "gemm_f32.hip",
    "gemm_rows": "gemm_rows.hip",
    "gemm_tiles": "gemm_tiles.hip",
    "rope_kv": "rope_kv.hip",
    "attention_simt": "attention_simt.hip",
    "attention_mfma": "attention_mfma.hip",
    "sampling": "sampling.hip",
    "ceilings": "ceilings.hip",
    "host": "host/runtime.cpp",
}
HEADERS = ("common.h", "attention_static.h", "attention_args.h", "attention_stream.h", "attention_portions.h",
           "attention_portions_dma.h")
HOST_LIBS = ("host",)   # plain C++: page pool, block tables, step packing
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared"]

HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # Packed 32-bit float instructions are kept out of every kernel of this package.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[arle_amd build] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


_lib_dir_lock = threading.Lock()
_lib_dir_cache: dict = {}


def lib_dir() -> str:
    """Folder that holds the built libraries; created if it does not exist."""
    key = os.environ.get("ARLE_AMD_LIB_DIR", "")
    with _lib_dir_lock:
        if key not in _lib_dir_cache:
            _lib_dir_cache[key] = _find_lib_dir()
        return _lib_dir_cache[key]


def _find_lib_dir() -> str:
    override = os.environ.get("ARLE_AMD_LIB_DIR")
    primary = override or os.path.join(PACKAGE_DIR, "_lib")
    try:
        os.makedirs(primary, exist_ok=True)
        probe = os.path.join(primary, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return primary
    except OSError:
        fallback = os.path.join(tempfile.gettempdir(), f"arle_amd_lib_{os.getuid()}")
        os.makedirs(fallback, exist_ok=True)
        return fallback


def existing_lib(name: str) -> str | None:
    """Path of an already built library, wherever it may be, without creating anything."""
    fname = f"libarle_{name}.so"
    cands = []
    if os.environ.get("ARLE_AMD_LIB_DIR"):
        cands.append(os.path.join(os.environ["ARLE_AMD_LIB_DIR"], fname))
    cands.append(os.path.join(PACKAGE_DIR, "_lib", fname))
    cands.append(os.path.join(tempfile.gettempdir(), f"arle_amd_lib_{os.getuid()}", fname))
    for c in cands:
        if os.path.exists(c):
            return c
    return None


def find_host_compiler() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")):
        if cand and (os.path.exists(cand) or shutil.which(cand)):
            return cand
    return find_hipcc()   # hipcc compiles plain C++ too


def source_hash(name: str) -> str:
    h = hashlib.sha256()
    host = name in HOST_LIBS
    for fname in ((SOURCES[name],) if host else (SOURCES[name], *HEADERS)):
        with open(os.path.join(CSRC_DIR, fname), "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HOST_FLAGS if host else HIPCC_FLAGS).encode())
    return h.hexdigest()


def is_current(path: str, name: str) -> bool:
    try:
        with open(path + ".srchash") as fh:
            return fh.read().strip() == source_hash(name)
    except OSError:
        return False


def build(name: str) -> str:
    """Compile one library (always) and return its path."""
    if name not in SOURCES:
        raise BuildError(f"unknown kernel library {name!r}")
    src = os.path.join(CSRC_DIR, SOURCES[name])
    out_dir = lib_dir()
    out = os.path.join(out_dir, f"libarle_{name}.so")
    tmp = f"{out}.tmp{os.getpid()}"
    if name in HOST_LIBS:
        cmd = [find_host_compiler(), *HOST_FLAGS, src, "-o", tmp]
        _say(f"compiling {SOURCES[name]} for the host ...")
    else:
        cmd = [find_hipcc(), *HIPCC_FLAGS, f"-I{CSRC_DIR}", src, "-o", tmp]
        _say(f"compiling {SOURCES[name]} for {OFFLOAD_ARCH} ...")
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME") or not os.access(env.get("HOME", ""), os.W_OK):
        env["HOME"] = out_dir  # hipcc may want a writable home for its caches
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    done = threading.Event()

    def heartbeat():
        while not done.wait(15.0):
            _say(f"  still compiling {SOURCES[name]} ({time.time() - t0:.0f} s)")

    beat = threading.Thread(target=heartbeat, daemon=True)
    beat.start()
    try:
        output, _ = proc.communicate()
    finally:
        done.set()
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise BuildError(f"{os.path.basename(cmd[0])} failed on {SOURCES[name]} (exit {proc.returncode}):\n{output}")
    os.replace(tmp, out)
    with open(out + ".srchash", "w") as fh:
        fh.write(source_hash(name))
    _say(f"built {os.path.basename(out)} in {time.time() - t0:.1f} s")
    return out


def ensure(name: str) -> str:
    """Path of an up-to-date library: the built one if current, else compile it now."""
    path = existing_lib(name)
    if path and is_current(path, name):
        return path
    return build(name)


def build_all(names=None, jobs: int = 4) -> dict:
    """Compile every library (always), a few at a time; returns name -> path.  Libraries of sources that no
    longer exist are removed from the folder."""
    if not names:
        known = {f"libarle_{n}.so" for n in SOURCES}
        folder = lib_dir()
        for fname in os.listdir(folder):
            base = fname[:-len(".srchash")] if fname.endswith(".srchash") else fname
            if base.startswith("libarle_") and base.endswith(".so") and base not in known:
                os.remove(os.path.join(folder, fname))
    names = list(names or SOURCES)
    results: dict = {}
    errors: list = []
    lock = threading.Lock()
    queue = list(names)

    def worker():
        while True:
            with lock:
                if not queue:
                    return
                n = queue.pop(0)
            try:
                p = build(n)
                with lock:
                    results[n] = p
            except Exception as exc:  # noqa: BLE001 - reported below
                with lock:
                    errors.append((n, exc))

    threads = [threading.Thread(target=worker) for _ in range(max(1, min(jobs, len(names))))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise BuildError("; ".join(f"{n}: {e}" for n, e in errors))
    return results


if __name__ == "__main__":
    build_all(sys.argv[1:] or None)
