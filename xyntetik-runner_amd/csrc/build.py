"""Compiling the gfx950 kernel library with hipcc.

One shared object per *unit*: the unit "kernels" holds everything whose code does
not depend on the model's sizes; a unit "attn_d<D>" holds the MFMA attention kernels
specialised for head size D and is compiled when a model with that head size is
first built.  Objects and libraries live beside the sources (``_build/`` and
``lib*.so``); if that folder cannot be written, under ``$XR_BUILD_DIR`` or a
per-user folder in the temporary directory.

A library is rebuilt when the hash of its sources and flags differs from the one
stored beside it.  While hipcc runs, a line goes to stderr every few seconds.
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
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List, Optional, Sequence

SRC_DIR = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
# -packed-fp32-ops off: hipcc must not form packed 32-bit float instructions.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

UNITS: Dict[str, dict] = {
    "kernels": {
        "sources": ["errors.hip", "basic_kernels.hip", "gemm_ref.hip", "attention_ref.hip",
                    "sampling.hip", "gemm_mfma.hip"],
        "defines": [],
    },
}
ATTN_SOURCES = ["errors.hip", "attention_mfma.hip"]
HEADERS = ["common.h", "async_copy.h", "no_alloc.h"]


class BuildError(RuntimeError):
    pass


def unit_spec(unit: str) -> dict:
    if unit in UNITS:
        return UNITS[unit]
    if unit.startswith("attn_d"):
        d = int(unit[len("attn_d"):])
        return {"sources": ATTN_SOURCES, "defines": [f"-DXR_HEAD_DIM={d}"]}
    raise BuildError(f"unknown kernel unit {unit!r}")


def _log(msg: str) -> None:
    sys.stderr.write(f"[xyntetik-runner build] {msg}\n")
    sys.stderr.flush()


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the kernel library cannot be built")


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def output_dir() -> str:
    """Where libraries are written and looked for first."""
    env = os.environ.get("XR_BUILD_DIR")
    if env:
        os.makedirs(env, exist_ok=True)
        return env
    if _writable(SRC_DIR):
        return SRC_DIR
    d = os.path.join(tempfile.gettempdir(), f"xyntetik-runner-build-{os.getuid()}")
    os.makedirs(d, exist_ok=True)
    return d


def source_hash(unit: str) -> str:
    spec = unit_spec(unit)
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS + spec["defines"]).encode())
    for name in list(spec["sources"]) + HEADERS:
        h.update(name.encode())
        with open(os.path.join(SRC_DIR, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def lib_name(unit: str) -> str:
    return f"libxr_{unit}.so"


def find_built(unit: str) -> Optional[str]:
    """Path of an up-to-date library for ``unit``, or None."""
    want = source_hash(unit)
    dirs = [SRC_DIR]
    try:
        od = output_dir()
        if od not in dirs:
            dirs.append(od)
    except OSError:
        pass
    for d in dirs:
        lib = os.path.join(d, lib_name(unit))
        try:
            with open(lib + ".hash", "r") as f:
                have = f.read().strip()
        except OSError:
            continue
        if have == want and os.path.exists(lib):
            return lib
    return None


def _run(cmd: Sequence[str], what: str) -> None:
    done = threading.Event()

    def beat():
        t0 = time.time()
        while not done.wait(15.0):
            _log(f"still compiling {what} ({time.time() - t0:.0f} s)")

    th = threading.Thread(target=beat, daemon=True)
    th.start()
    try:
        p = subprocess.run(list(cmd), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    finally:
        done.set()
    if p.returncode != 0:
        raise BuildError(f"hipcc failed on {what} (exit {p.returncode}):\n{' '.join(cmd)}\n{p.stdout}")


def build_unit(unit: str, force: bool = False, jobs: int = 8) -> str:
    """Compile ``unit`` (if stale or ``force``) and return the library's path."""
    if not force:
        have = find_built(unit)
        if have:
            return have
    spec = unit_spec(unit)
    hipcc = find_hipcc()
    out = output_dir()
    obj_dir = os.path.join(out, "_build", unit)
    os.makedirs(obj_dir, exist_ok=True)
    env_home = os.environ.get("HOME")
    if not env_home or not os.path.isdir(env_home) or not os.access(env_home, os.W_OK):
        os.environ["HOME"] = out      # hipcc wants a home it can write a cache into
    _log(f"compiling unit '{unit}' for {ARCH} ({len(spec['sources'])} files) into {out}")
    t0 = time.time()
    objs: List[str] = []
    jobs_list = []
    for src in spec["sources"]:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        cmd = [hipcc] + HIPCC_FLAGS + spec["defines"] + ["-I", SRC_DIR, "-c", os.path.join(SRC_DIR, src), "-o", obj]
        jobs_list.append((cmd, src))
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(jobs_list)))) as ex:
        futs = [ex.submit(_run, cmd, src) for cmd, src in jobs_list]
        for f in futs:
            f.result()
    lib = os.path.join(out, lib_name(unit))
    tmp = lib + f".tmp{os.getpid()}"
    _run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp] + objs, f"link {lib_name(unit)}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(source_hash(unit))
    _log(f"unit '{unit}' built in {time.time() - t0:.1f} s")
    return lib


def default_units(head_dims: Sequence[int] = (16, 32, 64, 128)) -> List[str]:
    return ["kernels"] + [f"attn_d{d}" for d in head_dims]


if __name__ == "__main__":
    units = sys.argv[1:] or default_units()
    for u in units:
        print(build_unit(u, force=True))
