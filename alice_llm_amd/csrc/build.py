"""Builds the HIP library for gfx950 with hipcc: every .hip file of this folder into one shared
object next to the Python bindings.  Used by the first call that needs the library when none is
built, and by the repository's build entry point, which compiles every time."""
from __future__ import annotations

import concurrent.futures as cf
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libalice_hip.so"
ARCH = "gfx950"
# No packed 32-bit float instructions: hipcc -O3 would form them from ordinary float code.
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-unused-value"]


def sources():
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def source_digest() -> str:
    """A digest of everything the library is made from (sources, headers, compiler flags).  It is compiled
    into the library, so that a library built from other sources than the ones beside it is noticed."""
    h = hashlib.sha256(" ".join(FLAGS).encode())
    for f in sorted(f for f in os.listdir(HERE) if f.endswith((".hip", ".h"))):
        h.update(f.encode())
        with open(os.path.join(HERE, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:32]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                       "the HIP library cannot be built")


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        open(probe, "w").close()
        os.remove(probe)
        return True
    except OSError:
        return False


def output_dirs():
    """Where the library is looked for and built: in the tree first, else a per-user temp folder."""
    in_tree = os.path.join(os.path.dirname(HERE), "hip")
    fallback = os.path.join(tempfile.gettempdir(), f"alice_llm_amd_{os.getuid()}", source_digest())
    return [in_tree, fallback]


def built_libraries():
    """Every built library there is, in the order of preference."""
    return [p for p in (os.path.join(d, LIB_NAME) for d in output_dirs()) if os.path.exists(p)]


def find_library():
    libs = built_libraries()
    return libs[0] if libs else None


def _say(msg: str) -> None:
    print(f"[alice-llm_amd build] {msg}", file=sys.stderr, flush=True)


def _compile(hipcc: str, src: str, obj: str, digest: str) -> float:
    t0 = time.time()
    cmd = [hipcc, *FLAGS, f'-DALICE_SOURCE_DIGEST="{digest}"', "-c", os.path.join(HERE, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
    return time.time() - t0


def build(verbose: bool = True) -> str:
    """Compile everything and link; returns the path of the shared object."""
    hipcc = _hipcc()
    out_dir = next((d for d in output_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError(f"no writable folder for the HIP library among {output_dirs()}")
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    digest = source_digest()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    # object files carry the process id: two processes that build at once (a test runner and a program it
    # starts) do not write into each other's files; the library itself is put in place by a rename
    objs = {s: os.path.join(obj_dir, f"{s[:-4]}.{os.getpid()}.o") for s in srcs}
    t0 = time.time()
    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
    with cf.ThreadPoolExecutor(workers) as pool:
        futs = {pool.submit(_compile, hipcc, s, o, digest): s for s, o in objs.items()}
        pending = set(futs)
        while pending:
            done, pending = cf.wait(pending, timeout=15, return_when=cf.FIRST_COMPLETED)
            for f in done:
                dt = f.result()
                if verbose:
                    _say(f"  {futs[f]} compiled in {dt:.0f} s")
            if pending and verbose and not done:
                _say(f"  still compiling {len(pending)} sources ({time.time() - t0:.0f} s)")
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs.values()],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    for o in objs.values():
        try:
            os.remove(o)
        except OSError:
            pass
    if r.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, lib)
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


if __name__ == "__main__":
    print(build())
