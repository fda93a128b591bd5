"""Compile one group of HIP sources of ``csrc/`` into its shared library next to this file.

The package's kernels come in groups that build and load independently, so that a process pays only for what its model uses:
``pc_*.hip`` -> ``libpromptcache_hip.so`` (the split-precision fp16 stacks of the Llama / Falcon / MPT adapters) and
``pb_*.hip`` -> ``libpromptcache_blocks.so`` (the bf16 / fp32 building blocks).  One hipcc per translation unit, all at once.
"""
from __future__ import annotations

import fcntl
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(PKG), "csrc")
INCLUDE = os.path.join(os.path.dirname(os.path.dirname(PKG)), "include")

GROUPS = {
    # group -> (source glob, library, extra flags)
    "blocks": ("pb_*.hip", "libpromptcache_blocks.so",
               # no packed-fp32 instructions: hipcc forms them from scalar float code by itself
               ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]),
}


def hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def lib_path(group: str) -> str:
    return os.path.join(PKG, GROUPS[group][1])


def stale(group: str) -> bool:
    pattern, _, _ = GROUPS[group]
    lib = lib_path(group)
    if not os.path.exists(lib):
        return True
    prefix = pattern.split("*")[0]
    deps = glob.glob(os.path.join(CSRC, pattern)) + glob.glob(os.path.join(CSRC, prefix + "*.h")) + \
        glob.glob(os.path.join(INCLUDE, "*.h"))
    return any(os.path.getmtime(d) > os.path.getmtime(lib) for d in deps)


def build(group: str, force: bool = False) -> str:
    """Build the group's library when it is missing or older than its sources (always with ``force``); returns its path.
    Concurrent callers serialise on a lock file, and the library appears under its name only when it is complete."""
    pattern, _, extra = GROUPS[group]
    lib = lib_path(group)
    objdir = os.path.join(CSRC, "_build")
    os.makedirs(objdir, exist_ok=True)
    with open(os.path.join(objdir, f".{group}.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if not force and not stale(group):
            return lib
        srcs = sorted(glob.glob(os.path.join(CSRC, pattern)))
        if not srcs:
            raise RuntimeError(f"no sources match {pattern} under {CSRC}")
        flags = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-mllvm", "-amdgpu-mfma-vgpr-form",
                 *extra, *os.environ.get("PC_BUILD_FLAGS", "").split()]
        jobs = []
        for src in srcs:
            obj = os.path.join(objdir, os.path.basename(src) + ".o")
            cmd = [hipcc(), *flags, "-c", src, "-o", obj]
            print("[build]", " ".join(cmd), file=sys.stderr, flush=True)
            jobs.append((obj, cmd, subprocess.Popen(cmd, cwd=os.path.dirname(CSRC), stdout=sys.stderr)))
        for obj, cmd, proc in jobs:
            if proc.wait() != 0:
                raise subprocess.CalledProcessError(proc.returncode, cmd)
        tmp = lib + f".{os.getpid()}.tmp"
        link = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *[o for o, _, _ in jobs], "-o", tmp]
        print("[build]", " ".join(link), file=sys.stderr, flush=True)
        subprocess.check_call(link, cwd=os.path.dirname(CSRC), stdout=sys.stderr)
        os.replace(tmp, lib)
    return lib
