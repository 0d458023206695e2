"""Builds the HIP kernels for gfx950 with hipcc into one shared library.

The library's file name carries a hash of the sources and flags, so a library
built from other sources is never loaded by mistake. `ensure_built()` compiles
only if no library for the current sources exists; `build()` always compiles.
The library is kept next to the sources; if that folder cannot be written, in
a per-user folder under the temporary directory.
"""
from __future__ import annotations

import hashlib
import os
from pathlib import Path
import shutil
import subprocess
import sys
import tempfile
import threading
import time

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
# Packed float32 instructions are switched off: some of their forms have given
# wrong results on this hardware generation.
# MFMA results are kept in ordinary vector registers: with the default heuristic the
# compiler parks accumulators in AGPRs and moves them to VGPRs and back around every
# float32 operation on them (the online-softmax rescale), hundreds of moves per block.
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-value",
         "-mllvm", "-amdgpu-mfma-vgpr-form=1"]
# The tiled GEMM's largest tile keeps 256 accumulator registers per lane, which only fit as AGPRs.
WITHOUT = {"gemm_tiled.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def flags_for(src):
    drop = WITHOUT.get(Path(src).name, [])
    flags = list(FLAGS)
    for i in range(len(flags) - len(drop) + 1):
        if drop and flags[i:i + len(drop)] == drop:
            del flags[i:i + len(drop)]
            break
    return flags


def sources():
    return sorted(CSRC.glob("*.hip"))


def headers():
    return sorted(CSRC.glob("*.h"))


def source_hash():
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    h.update(repr(sorted(WITHOUT.items())).encode())
    for path in headers() + sources():
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()[:16]


def library_name():
    return f"libtessweave_hip_{source_hash()}.so"


def _in_tree_dir():
    return CSRC / "_lib"


def _user_dir():
    user = os.getuid() if hasattr(os, "getuid") else 0
    return Path(tempfile.gettempdir()) / f"tessweave_engine_amd_{user}"


def _candidate_dirs():
    yield _in_tree_dir()
    yield _user_dir()


def _only_ours(folder):
    """Is FOLDER (under the shared temporary directory) a real directory that belongs to this user and
    that nobody else can write to? A library is neither loaded from nor built into anything else: the
    library's name is computable from public sources, so a folder another user made could hold a planted one."""
    try:
        st = os.lstat(folder)
    except OSError:
        return False
    import stat
    if not stat.S_ISDIR(st.st_mode):
        return False
    if hasattr(os, "getuid") and st.st_uid != os.getuid():
        return False
    return not st.st_mode & (stat.S_IWGRP | stat.S_IWOTH)


def find_library():
    name = library_name()
    for folder in _candidate_dirs():
        if folder == _user_dir() and not _only_ours(folder):
            continue
        path = folder / name
        if path.exists():
            return path
    return None


def _writable_dir():
    for folder in _candidate_dirs():
        try:
            if folder == _user_dir():
                folder.mkdir(mode=0o700, exist_ok=True)
                if not _only_ours(folder):
                    raise OSError(f"{folder} is not this user's private folder")
            else:
                folder.mkdir(parents=True, exist_ok=True)
            probe = folder / f".probe_{os.getpid()}"
            probe.write_bytes(b"")
            probe.unlink()
            return folder
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel library")


def _hipcc():
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(path).exists():
        raise RuntimeError("hipcc was not found; the HIP kernels cannot be built")
    return path


def _say(text):
    print(f"[tessweave_engine_amd] {text}", file=sys.stderr, flush=True)


def build(verbose=True):
    """Compile every source for gfx950 and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = _writable_dir()
    target = out_dir / library_name()
    work = Path(tempfile.mkdtemp(prefix="tw_build_", dir=str(out_dir)))
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = str(work)
    srcs = sources()
    started = time.time()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} with {hipcc} ...")
    results = {}

    def compile_one(src):
        obj = work / (src.stem + ".o")
        cmd = [hipcc, *flags_for(src), "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
        proc = subprocess.run(cmd, capture_output=True, text=True, env=env)
        results[src] = (proc.returncode, proc.stderr, obj)

    threads = [threading.Thread(target=compile_one, args=(s,)) for s in srcs]
    for t in threads:
        t.start()
    while any(t.is_alive() for t in threads):
        for t in threads:
            t.join(timeout=15.0 / max(1, len(threads)))
        if verbose and any(t.is_alive() for t in threads):
            done = len(results)
            _say(f"  {done}/{len(srcs)} compiled, {time.time() - started:.0f} s")
    try:
        failed = [(s, r) for s, r in results.items() if r[0] != 0]
        if failed:
            text = "\n".join(f"{s.name}:\n{r[1]}" for s, r in failed)
            raise RuntimeError(f"hipcc failed:\n{text}")
        objs = [str(results[s][2]) for s in srcs]
        tmp_target = work / target.name
        link = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", str(tmp_target), *objs],
                              capture_output=True, text=True, env=env)
        if link.returncode != 0:
            raise RuntimeError(f"linking the kernel library failed:\n{link.stderr}")
        os.replace(tmp_target, target)
        for old in out_dir.glob("libtessweave_hip_*.so"):
            if old != target:
                try:
                    old.unlink()
                except OSError:
                    pass
    finally:
        shutil.rmtree(work, ignore_errors=True)
    if verbose:
        _say(f"built {target.name} in {time.time() - started:.0f} s")
    return target


def ensure_built(verbose=True):
    path = find_library()
    if path is None:
        if verbose:
            _say("no kernel library for these sources yet; building it once")
        path = build(verbose)
    return path
