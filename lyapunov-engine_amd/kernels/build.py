"""Compiles the HIP and C++ sources under ``csrc/`` into shared libraries.

There is one library of kernels whose sizes are run-time values (``core``), one
attention library per head size (``attn_hd<N>``; the head size is a compile-time
constant there), one of host code around the vendor's GEMM library (``blas``),
and one library of host code (``runtime``: cache manager and scheduler).  A library's file name carries a hash of its sources and flags, so a
changed source is never served by an old binary; what is missing is compiled on
first use, with a progress line now and then.

The reference builds one torch extension from its .cu files
(setup.py:33-93, CMakeLists.txt:1-33); here the libraries have a C interface and
are loaded with ctypes, so nothing but hipcc and a C++ compiler is needed.
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
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent.parent
CSRC = PACKAGE_DIR / "csrc"

GPU_ARCH = "gfx950"
HIP_FLAGS = [
    f"--offload-arch={GPU_ARCH}",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
CXX_FLAGS = ["-O2", "-std=c++20", "-fPIC", "-Wall", "-Wextra"]

CORE_SOURCES = ["kernels/errors.hip", "kernels/elementwise.hip", "kernels/gemm.hip", "kernels/sampler.hip"]
ATTN_SOURCES = ["kernels/errors.hip", "kernels/attention.hip"]
BLAS_SOURCES = ["kernels/errors.hip", "kernels/library_gemm.hip"]   # host code around the vendor's GEMM library
RUNTIME_SOURCES = ["runtime/cache_manager.cpp", "runtime/scheduler.cpp", "runtime/c_api.cpp"]

# Head sizes compiled ahead of time by build_all(); any other multiple of 16 up
# to 256 is compiled when a model first asks for it.
PREBUILT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 128, 256)

_lock = threading.Lock()


def _say(msg: str) -> None:
    from ..utils import log

    log.info(msg, prefix="[lyapunov-amd build]")


def hipcc_path() -> str:
    found = shutil.which("hipcc")
    if found:
        return found
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cand = os.path.join(rocm, "bin", "hipcc")
    if os.path.exists(cand):
        return cand
    raise RuntimeError("hipcc not found: the kernels of this package cannot be compiled")


def cxx_path() -> str:
    for name in (os.environ.get("CXX"), "g++", "c++", "clang++"):
        if name and shutil.which(name):
            return shutil.which(name)
    return hipcc_path()


def library_dir() -> Path:
    """Where libraries are kept: inside the package when that is writable, so
    that they travel with the source tree, else a per-user temporary folder."""
    override = os.environ.get("LYAPUNOV_AMD_LIB_DIR")
    if override:
        p = Path(override)
        p.mkdir(parents=True, exist_ok=True)
        return p
    p = PACKAGE_DIR / "_lib"
    try:
        p.mkdir(parents=True, exist_ok=True)
        probe = p / f".probe-{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return p
    except OSError:
        p = Path(tempfile.gettempdir()) / f"lyapunov_amd_lib_{os.getuid()}"
        p.mkdir(parents=True, exist_ok=True)
        return p


def _headers() -> list[Path]:
    return sorted(CSRC.rglob("*.h")) + sorted(CSRC.rglob("*.hpp"))


def _key(sources: list[str], flags: list[str]) -> str:
    h = hashlib.sha1()
    for f in flags:
        h.update(f.encode())
    for rel in sources:
        h.update(rel.encode())
        h.update((CSRC / rel).read_bytes())
    for hdr in _headers():
        h.update(hdr.read_bytes())
    return h.hexdigest()[:12]


def _run_with_progress(cmds: list[list[str]], what: str) -> None:
    """Run the compile commands in parallel; say something every 20 s."""
    procs = [subprocess.Popen(c, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True) for c in cmds]
    outputs = [""] * len(procs)

    def drain(i: int) -> None:
        outputs[i] = procs[i].stdout.read()

    threads = [threading.Thread(target=drain, args=(i,), daemon=True) for i in range(len(procs))]
    for t in threads:
        t.start()
    t0 = last = time.time()
    while any(p.poll() is None for p in procs):
        time.sleep(0.2)
        if time.time() - last > 20:
            last = time.time()
            _say(f"still compiling {what} ({int(last - t0)} s)")
    for t in threads:
        t.join()
    for p, out, cmd in zip(procs, outputs, cmds):
        if p.returncode != 0:
            lines = [l for l in out.splitlines() if "not a recognized feature" not in l]
            raise RuntimeError("compilation failed: " + " ".join(cmd) + "\n" + "\n".join(lines[-40:]))


def build_library(name: str, sources: list[str], *, hip: bool, defines: dict[str, str] | None = None,
                  force: bool = False, link: list[str] | None = None, extra_flags: list[str] | None = None) -> Path:
    """Return the path of the library, compiling it if it is not there."""
    defines = dict(defines or {})
    # For experiments: LYAPUNOV_AMD_EXTRA_DEFINES="NAME=VALUE,OTHER=1" adds macros to every HIP compile
    # (the library's name changes with them, so the regular build is left alone).
    if hip and os.environ.get("LYAPUNOV_AMD_EXTRA_DEFINES"):
        for item in os.environ["LYAPUNOV_AMD_EXTRA_DEFINES"].split(","):
            k, _, v = item.partition("=")
            defines[k.strip()] = v.strip() or "1"
    compiler = hipcc_path() if hip else cxx_path()
    flags = (HIP_FLAGS if hip else CXX_FLAGS) + list(extra_flags or []) + [f"-D{k}={v}" for k, v in sorted(defines.items())]
    include = ["-I", str(CSRC / "kernels"), "-I", str(CSRC / "runtime")]
    out_dir = library_dir()
    target = out_dir / f"lib{name}-{_key(sources, flags + list(link or []))}.so"
    with _lock:
        if target.exists() and not force:
            return target
        _say(f"compiling {name} ({len(sources)} files) -> {target}")
        t0 = time.time()
        work = Path(tempfile.mkdtemp(prefix=f"build-{name}-", dir=out_dir))
        try:
            objs, cmds = [], []
            for rel in sources:
                obj = work / (rel.replace("/", "_") + ".o")
                objs.append(str(obj))
                cmds.append([compiler, *flags, *include, "-c", str(CSRC / rel), "-o", str(obj)])
            _run_with_progress(cmds, name)
            tmp_so = work / "out.so"
            link_cmd = [compiler, "-shared", "-fPIC", *objs, "-o", str(tmp_so), *(link or [])]
            if hip:
                link_cmd.insert(1, f"--offload-arch={GPU_ARCH}")
            _run_with_progress([link_cmd], name + " (link)")
            os.replace(tmp_so, target)
        finally:
            shutil.rmtree(work, ignore_errors=True)
        for old in out_dir.glob(f"lib{name}-*.so"):
            if old != target and not os.environ.get("LYAPUNOV_AMD_EXTRA_DEFINES"):
                try:
                    old.unlink()
                except OSError:
                    pass
        _say(f"{name} done in {time.time() - t0:.1f} s")
    return target


def core_library(force: bool = False) -> Path:
    return build_library("lyp_core", CORE_SOURCES, hip=True, force=force)


def attention_library(head_dim: int, force: bool = False) -> Path:
    if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
        raise ValueError(f"attention kernels exist for head sizes that are multiples of 16 up to 256, not {head_dim}")
    return build_library(f"lyp_attn_hd{head_dim}", ATTN_SOURCES, hip=True,
                         defines={"LYP_HEAD_DIM": str(head_dim)}, force=force)


def blas_library(force: bool = False) -> Path:
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    return build_library("lyp_blas", BLAS_SOURCES, hip=True, force=force,
                         link=[f"-L{os.path.join(rocm, 'lib')}", "-lhipblaslt"])


SANITIZE_FLAGS = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-g", "-O1"]


def sanitizing() -> bool:
    """LYAPUNOV_AMD_SANITIZE=1: host code (the cache manager and the scheduler) is compiled with the
    address and undefined-behaviour sanitizers.  The self-test program then runs under them as it
    is; the library so built can only be loaded by a process that has the sanitizer's runtime
    loaded first."""
    return os.environ.get("LYAPUNOV_AMD_SANITIZE", "0") not in ("", "0")


def runtime_library(force: bool = False) -> Path:
    if sanitizing():
        return build_library("lyp_runtime_sanitized", RUNTIME_SOURCES, hip=False, force=force,
                             link=["-fsanitize=address,undefined"], extra_flags=SANITIZE_FLAGS)
    return build_library("lyp_runtime", RUNTIME_SOURCES, hip=False, force=force)


def runtime_selftest(force: bool = False) -> Path:
    """The program of csrc/runtime/selftest.cpp (random requests through the scheduler and the
    cache manager, invariants checked after every step), with the sanitizers when
    LYAPUNOV_AMD_SANITIZE=1.  Returns the executable's path."""
    sources = [s for s in RUNTIME_SOURCES if not s.endswith("c_api.cpp")] + ["runtime/selftest.cpp"]
    flags = CXX_FLAGS + (SANITIZE_FLAGS if sanitizing() else [])
    out_dir = library_dir()
    target = out_dir / f"runtime_selftest{'_sanitized' if sanitizing() else ''}-{_key(sources, flags)}"
    with _lock:
        if target.exists() and not force:
            return target
        _say(f"compiling the runtime's self-test -> {target}")
        tmp = target.with_suffix(f".tmp{os.getpid()}")
        cmd = [cxx_path(), *flags, "-I", str(CSRC / "runtime"), *[str(CSRC / rel) for rel in sources], "-o", str(tmp)]
        _run_with_progress([cmd], "runtime self-test")
        os.replace(tmp, target)
        for old in out_dir.glob(f"{target.name.rsplit('-', 1)[0]}-*"):
            if old != target:
                try:
                    old.unlink()
                except OSError:
                    pass
    return target


def build_all(force: bool = True) -> list[Path]:
    """Compile every library (what ``__graft_entry__.build`` calls)."""
    out = [runtime_library(force), core_library(force), blas_library(force)]
    for hd in PREBUILT_HEAD_DIMS:
        out.append(attention_library(hd, force))
    return out
