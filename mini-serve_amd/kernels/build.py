"""Builds the HIP kernel library for gfx950 with hipcc and finds the built file.

The library's file name carries a hash of its sources, so a stale build is never loaded: a
changed source simply has no library yet and is compiled at the first call (in-tree under
``kernels/_lib`` when that is writable, else under a per-user temporary folder). Each source file
is compiled by its own hipcc process, then all are linked into one shared object.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
LIB_DIR = Path(__file__).resolve().parent / "_lib"
ARCH = "gfx950"
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    # Keep the compiler from forming packed float32 instructions.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
CXX_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-Wall", "-Wextra"]


def hip_sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def cpp_sources() -> list[Path]:
    return sorted(CSRC.glob("*.cpp"))


def _digest(files: list[Path], flags: list[str]) -> str:
    h = hashlib.sha256()
    for f in sorted(files + sorted(CSRC.glob("*.h"))):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    h.update(" ".join(flags).encode())
    return h.hexdigest()[:16]


def _say(msg: str) -> None:
    print(f"[miniserve_amd build] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found: the HIP kernels cannot be built (set HIPCC or install ROCm)")


def _writable_dir() -> Path:
    override = os.environ.get("MINISERVE_AMD_BUILD_DIR")
    if override:
        d = Path(override)
        d.mkdir(parents=True, exist_ok=True)
        return d
    try:
        LIB_DIR.mkdir(parents=True, exist_ok=True)
        probe = LIB_DIR / f".w{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return LIB_DIR
    except OSError:
        d = Path(tempfile.gettempdir()) / f"miniserve_amd_{os.getuid()}"
        d.mkdir(parents=True, exist_ok=True)
        return d


def _run_parallel(cmds: list[list[str]], what: str) -> None:
    """Run the commands at once. Each writes to a file of its own, never to a pipe: a compiler that
    prints more than a pipe holds would otherwise wait for a reader that only comes after its exit."""
    start = time.time()
    procs = []
    for c in cmds:
        log = tempfile.TemporaryFile(mode="w+", prefix="msamd_log_")
        procs.append((c, subprocess.Popen(c, stdout=log, stderr=subprocess.STDOUT, text=True), log))
    last = start
    try:
        while any(p.poll() is None for _, p, _ in procs):
            if time.time() - last > 10:
                last = time.time()
                left = sum(p.poll() is None for _, p, _ in procs)
                _say(f"{what}: {left} of {len(procs)} still compiling ({int(last - start)} s)")
            time.sleep(0.05)
        for c, p, log in procs:
            if p.returncode != 0:
                log.seek(0)
                raise RuntimeError(f"build failed: {' '.join(c)}\n{log.read()[-8000:]}")
    finally:
        for _, p, log in procs:
            if p.poll() is None:
                p.kill()
            log.close()


def kernel_library_name() -> str:
    return f"libmsamd_kernels_{_digest(hip_sources(), HIP_FLAGS)}.so"


def core_library_name() -> str:
    return f"libmsamd_core_{_digest(cpp_sources(), CXX_FLAGS)}.so"


def _find(name: str) -> Path | None:
    for d in (LIB_DIR, Path(os.environ.get("MINISERVE_AMD_BUILD_DIR", "/nonexistent")),
              Path(tempfile.gettempdir()) / f"miniserve_amd_{os.getuid()}"):
        if (d / name).is_file():
            return d / name
    return None


def build_kernels(force: bool = False) -> Path:
    """Compile every ``csrc/*.hip`` for gfx950 into one shared library; returns its path."""
    name = kernel_library_name()
    found = None if force else _find(name)
    if found:
        return found
    out_dir = _writable_dir()
    hipcc = _hipcc()
    srcs = hip_sources()
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir / name}")
    work = Path(tempfile.mkdtemp(prefix="msamd_obj_", dir=str(out_dir)))
    try:
        objs = [work / (s.stem + ".o") for s in srcs]
        _run_parallel([[hipcc, *HIP_FLAGS, "-c", str(s), "-o", str(o)] for s, o in zip(srcs, objs)], "kernels")
        tmp = work / name
        _run_parallel([[hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]], "link")
        # The new file takes its place in one step, and only builds of other sources are cleared away:
        # another process that builds the same sources at the same time never finds the name missing.
        os.replace(tmp, out_dir / name)
        for old in out_dir.glob("libmsamd_kernels_*.so"):
            if old.name != name:
                old.unlink(missing_ok=True)
    finally:
        shutil.rmtree(work, ignore_errors=True)
    _say("kernels built")
    return out_dir / name


def build_core(force: bool = False) -> Path:
    """Compile the C++ block core (host code) into a shared library; returns its path."""
    name = core_library_name()
    found = None if force else _find(name)
    if found:
        return found
    out_dir = _writable_dir()
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if not cxx:
        raise RuntimeError("no C++ compiler found for the block core")
    srcs = cpp_sources()
    tmp = out_dir / f".{name}.{os.getpid()}"
    _run_parallel([[cxx, *CXX_FLAGS, "-shared", "-o", str(tmp), *map(str, srcs)]], "block core")
    os.replace(tmp, out_dir / name)
    for old in out_dir.glob("libmsamd_core_*.so"):
        if old.name != name:
            old.unlink(missing_ok=True)
    return out_dir / name


def build_all(force: bool = False) -> list[Path]:
    out = [build_kernels(force)]
    if cpp_sources():
        out.append(build_core(force))
    return out


if __name__ == "__main__":
    for p in build_all(force="--force" in sys.argv):
        print(p)
