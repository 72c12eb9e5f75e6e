"""Builds the gfx950 kernel library with hipcc, in-tree, one object per source.

``build()`` always compiles (``build_host()`` likewise, the host runtime, with
the host compiler). ``ensure_built()`` compiles only when no library
is there or its sources changed since it was built; it prints a line per file
meanwhile, since a first call in a fresh checkout takes a minute or so.
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
from typing import List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libreinfer_hip.so"
ARCH = "gfx950"

# -packed-fp32-ops off: packed float instructions are kept out of every kernel
HIPCC_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Wno-unused-result",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    for f in sources() + _headers():
        h.update(f.encode())
        with open(os.path.join(HERE, f), "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def _hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _writable_dir() -> str:
    """In-tree when possible (the library then travels with the tree), else a
    private folder under the temporary directory."""
    if os.access(HERE, os.W_OK):
        return HERE
    d = os.path.join(tempfile.gettempdir(), f"reinfer_amd_build_{os.getuid()}_{source_hash()[:12]}")
    os.makedirs(d, exist_ok=True)
    return d


def lib_candidates() -> List[str]:
    out = [os.path.join(HERE, LIB_NAME)]
    alt = os.path.join(tempfile.gettempdir(), f"reinfer_amd_build_{os.getuid()}_{source_hash()[:12]}", LIB_NAME)
    out.append(alt)
    return out


def _say(msg: str) -> None:
    print(f"[reinfer_amd] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    hipcc = _hipcc()
    if hipcc is None:
        raise RuntimeError("hipcc not found: the gfx950 kernel library cannot be built "
                           "(set HIPCC or put /opt/rocm/bin on PATH)")
    out_dir = _writable_dir()
    stamp_dir = os.path.join(out_dir, "_build")
    # objects in a folder of this process: two programs that find nothing built at the same moment
    # (two replays started side by side in a fresh tree) each build whole objects and publish the
    # library with one rename
    obj_dir = os.path.join(stamp_dir, f"obj_{os.getpid()}")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())       # hipcc wants a HOME for its caches
    if not env["HOME"] or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    t0 = time.time()

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, src[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", HERE, "-c", os.path.join(HERE, src), "-o", obj]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
        return obj

    if verbose:
        _say(f"compiling {len(srcs)} kernel sources for {ARCH} with {hipcc} ...")
    objs = []
    workers = max(1, min(len(srcs), (os.cpu_count() or 4), 8))
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as ex:
        futs = {ex.submit(compile_one, s): s for s in srcs}
        for n, fut in enumerate(concurrent.futures.as_completed(futs), 1):
            objs.append(fut.result())
            if verbose:
                _say(f"  [{n}/{len(srcs)}] {futs[fut]} done ({time.time() - t0:.0f} s)")
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".{os.getpid()}.tmp"
    r = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp, *sorted(objs)],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc link failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, lib)
    with open(os.path.join(stamp_dir, "source.sha256"), "w") as f:
        f.write(source_hash())
    shutil.rmtree(obj_dir, ignore_errors=True)
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def find_built(check_fresh: bool = True) -> Optional[str]:
    want = source_hash() if check_fresh else None
    for lib in lib_candidates():
        if not os.path.isfile(lib):
            continue
        if not check_fresh:
            return lib
        stamp = os.path.join(os.path.dirname(lib), "_build", "source.sha256")
        try:
            with open(stamp) as f:
                if f.read().strip() == want:
                    return lib
        except OSError:
            # a library without its stamp (objects not shipped): take it as it is
            return lib
    return None


def ensure_built() -> str:
    lib = find_built()
    if lib is not None:
        return lib
    stale = find_built(check_fresh=False)
    if _hipcc() is None:
        if stale is not None:
            _say(f"warning: {stale} is older than its sources and hipcc is not available; using it")
            return stale
        raise RuntimeError("the gfx950 kernel library is not built and hipcc is not available")
    _say("kernel library " + ("is older than its sources" if stale else "is not built yet") + "; building now")
    return build()


# ---------------------------------------------------------------------------
# The host runtime (cache bookkeeping, step packing, scheduler): plain C++ with
# pybind11, built with the host compiler into the extension module reinfer_amd._host.
# ---------------------------------------------------------------------------
HOST_DIR = os.path.join(HERE, "host")
HOST_SOURCES = ["host.cpp"]


def _host_name() -> str:
    import sysconfig
    return "_host" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so")


def host_hash() -> str:
    h = hashlib.sha256()
    for f in HOST_SOURCES:
        with open(os.path.join(HOST_DIR, f), "rb") as fh:
            h.update(fh.read())
    h.update(sys.version.encode())
    return h.hexdigest()


def _host_dirs() -> List[str]:
    pkg = os.path.dirname(HERE)
    return [pkg, os.path.join(tempfile.gettempdir(), f"reinfer_amd_host_{os.getuid()}_{host_hash()[:12]}")]


def build_host(verbose: bool = True) -> str:
    import sysconfig
    import pybind11
    cxx = None
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/lib/llvm/bin/clang++"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            cxx = cand
            break
    if cxx is None:
        raise RuntimeError("no C++ compiler found for the host runtime (set CXX)")
    pkg, tmp = _host_dirs()
    out_dir = pkg if os.access(pkg, os.W_OK) else tmp
    os.makedirs(out_dir, exist_ok=True)
    out = os.path.join(out_dir, _host_name())
    part = out + f".{os.getpid()}.tmp"
    cmd = [cxx, "-O2", "-shared", "-fPIC", "-std=c++17", "-fvisibility=hidden",
           "-I", sysconfig.get_paths()["include"], "-I", pybind11.get_include(),
           *[os.path.join(HOST_DIR, f) for f in HOST_SOURCES], "-o", part]
    if verbose:
        _say(f"compiling the host runtime with {cxx} (about 15 s) ...")
    t0 = time.time()
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"host runtime failed to compile:\n{r.stderr[-4000:]}")
    os.replace(part, out)
    with open(out + ".sha256", "w") as f:
        f.write(host_hash())
    if verbose:
        _say(f"built {out} in {time.time() - t0:.0f} s")
    return out


def ensure_host_built() -> str:
    want = host_hash()
    stale = None
    for d in _host_dirs():
        path = os.path.join(d, _host_name())
        if not os.path.isfile(path):
            continue
        try:
            with open(path + ".sha256") as f:
                if f.read().strip() == want:
                    return path
            stale = stale or path
        except OSError:
            return path          # a module without its stamp: take it as it is
    try:
        return build_host()
    except Exception:
        if stale is not None:
            _say(f"warning: {stale} is older than its source and could not be rebuilt; using it")
            return stale
        raise


if __name__ == "__main__":
    build()
    build_host()
