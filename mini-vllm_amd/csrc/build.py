"""Builds the HIP kernel libraries for gfx950 with hipcc.

Two libraries are made from the same sources, one per activation type, so that a process
compiles only what its model needs: ``libmvk_f32.so`` (everything in IEEE float) and
``libmvk_bf16.so`` (bfloat16 activations and cache, the serving path). Object files are
compiled in parallel and a progress line is printed as each one finishes.

The libraries are written next to the sources in ``_build/``; when that folder cannot be
written (a read-only checkout) a per-user folder under the system's temporary directory is
used. A library is rebuilt when the hash of the sources and flags it was made from differs
from the current one.
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
from typing import Dict, List, Optional

CSRC = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"

# translation units of each variant
COMMON_SOURCES = ["runtime.hip", "elementwise.hip", "gemm_ref.hip", "attention_ref.hip", "sampling.hip"]
VARIANT_SOURCES: Dict[str, List[str]] = {
    "f32": COMMON_SOURCES,
    "bf16": COMMON_SOURCES + ["gemm_skinny.hip", "gemm_mid.hip", "gemm_tile.hip", "gemm_lt.hip", "attention_fast.hip",
                              "attention_prefill.hip"],
}
# libraries a variant links against
VARIANT_LIBS: Dict[str, List[str]] = {
    "f32": [],
    "bf16": ["-lhipblaslt"],
}
VARIANT_DEFINES: Dict[str, List[str]] = {
    "f32": ["-DMV_WITH_F32"],
    "bf16": ["-DMV_WITH_BF16"],
}

BASE_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option",
]


def _log(msg: str) -> None:
    print(f"[mini-vllm_amd build] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _sources(variant: str) -> List[str]:
    return [s for s in VARIANT_SOURCES[variant] if os.path.isfile(os.path.join(CSRC, s))]


def source_hash(variant: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(BASE_FLAGS + VARIANT_DEFINES[variant] + VARIANT_LIBS[variant]).encode())
    names = sorted(set(_sources(variant)) | {f for f in os.listdir(CSRC) if f.endswith(".h")})
    for name in names:
        h.update(name.encode())
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _writable_dir(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w") as f:
            f.write("x")
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dirs() -> List[str]:
    """Folders searched for built libraries, the first writable one receives new builds."""
    dirs = [os.path.join(CSRC, "_build")]
    env = os.environ.get("MINIVLLM_AMD_BUILD_DIR")
    if env:
        dirs.insert(0, env)
    dirs.append(os.path.join(tempfile.gettempdir(), f"mini-vllm_amd-build-{os.getuid()}"))
    return dirs


def library_name(variant: str) -> str:
    return f"libmvk_{variant}.so"


def find_library(variant: str, require_fresh: bool = True) -> Optional[str]:
    """Path of a built library whose recorded source hash is current (or any, if not
    ``require_fresh``)."""
    want = source_hash(variant)
    for d in build_dirs():
        lib = os.path.join(d, library_name(variant))
        stamp = lib + ".hash"
        if os.path.isfile(lib):
            if not require_fresh:
                return lib
            try:
                with open(stamp) as f:
                    if f.read().strip() == want:
                        return lib
            except OSError:
                pass
    return None


def _compile_one(hipcc: str, src: str, obj: str, defines: List[str]) -> float:
    t0 = time.time()
    cmd = [hipcc] + BASE_FLAGS + defines + ["-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    return time.time() - t0


def build(variant: str, force: bool = False, jobs: Optional[int] = None) -> str:
    """Compile one variant and return the library's path."""
    if variant not in VARIANT_SOURCES:
        raise ValueError(f"unknown kernel library variant {variant!r}")
    if not force:
        lib = find_library(variant)
        if lib:
            return lib
    hipcc = find_hipcc()
    if hipcc is None:
        raise RuntimeError("the HIP kernel library is not built and hipcc was not found "
                           "(looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")
    out_dir = next((d for d in build_dirs() if _writable_dir(d)), None)
    if out_dir is None:
        raise RuntimeError(f"no writable folder for the kernel library among {build_dirs()}")
    obj_dir = os.path.join(out_dir, f"obj_{variant}")
    os.makedirs(obj_dir, exist_ok=True)
    sources = _sources(variant)
    defines = VARIANT_DEFINES[variant]
    jobs = jobs or min(len(sources), max(1, min(16, (os.cpu_count() or 4))))
    _log(f"compiling {len(sources)} files for {ARCH} ({variant}) into {out_dir} with {jobs} jobs ...")
    t0 = time.time()
    objs = [os.path.join(obj_dir, os.path.splitext(s)[0] + ".o") for s in sources]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futs = {pool.submit(_compile_one, hipcc, s, o, defines): s for s, o in zip(sources, objs)}
        done = 0
        pending = set(futs)
        while pending:
            finished, pending = concurrent.futures.wait(pending, timeout=20,
                                                        return_when=concurrent.futures.FIRST_COMPLETED)
            if not finished:
                _log(f"  still compiling ({done}/{len(sources)} done, {time.time() - t0:.0f} s) ...")
            for fut in finished:
                dt = fut.result()
                done += 1
                _log(f"  [{done}/{len(sources)}] {futs[fut]} ({dt:.1f} s)")
    lib = os.path.join(out_dir, library_name(variant))
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", tmp] + objs + VARIANT_LIBS[variant]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"linking {lib} failed:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(source_hash(variant))
    _log(f"built {lib} in {time.time() - t0:.1f} s")
    return lib


def build_all(force: bool = True) -> List[str]:
    return [build(v, force=force) for v in VARIANT_SOURCES]


if __name__ == "__main__":
    variants = sys.argv[1:] or list(VARIANT_SOURCES)
    for v in variants:
        print(build(v, force=True))
