"""Compiles the HIP sources under csrc/ into distca_amd/libdistca_ca.so for gfx950.

Run on a machine with hipcc (no GPU needed: hipcc cross-compiles).  The library is
loaded by distca_amd._lib; tests, smoke and bench only load what is already built.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libdistca_ca.so")
SOURCES = ["api.cpp", "pack.hip", "sched.hip", "attn_fwd.hip", "attn_bwd.hip", "attn_bwd_dkdv64.hip", "attn_bwd_dq64.hip", "probe.hip"]
# The attention kernels exist once per element type: the same sources compiled again with -DDISTCA_F16 give the fp16
# kernels and their launchers under names of their own; the entry points (compiled once) pick by distca_ca_params.dtype.
F16_SOURCES = ["attn_fwd.hip", "attn_bwd.hip", "attn_bwd_dkdv64.hip", "attn_bwd_dq64.hip"]

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-x", "hip",
    # scalar fp32 only: keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # select MFMAs with VGPR accumulators; the allocator moves long-lived ones to AGPRs itself.
    # (AGPR-form selection, the default above 256 registers, copies every accumulator the VALU
    # touches between the two files each loop iteration.)
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-munsafe-fp-atomics",  # float atomic add as one hardware instruction, not a CAS loop
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: cannot build libdistca_ca.so")
    return exe


# Flags a source must not be compiled with.  attn_bwd_dkdv64.hip wants the compiler's default MFMA form (results in
# the accumulation registers) for its 256 dK/dV accumulators; the accumulators its vector ALU touches are pinned
# to vector registers in the source.
DROP_FLAGS = {"attn_bwd_dkdv64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"], "attn_bwd_dq64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def _compile(src: str, obj: str, extra: list[str]) -> None:
    flags = list(HIPCC_FLAGS)
    drop = DROP_FLAGS.get(src, [])
    for i in range(len(flags) - len(drop) + 1):
        if drop and flags[i:i + len(drop)] == drop:
            del flags[i:i + len(drop)]
            break
    cmd = [_hipcc(), *flags, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the gfx950 feature name and says so; drop that line
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build_library(extra_flags: list[str] | None = None, verbose: bool = False, out_path: str | None = None) -> str:
    """Compiles and links into `out_path` (default distca_amd/libdistca_ca.so, the only path
    the loader reads)."""
    extra = list(extra_flags or [])
    lib_path = out_path or LIB_PATH
    obj_dir = os.path.join(PKG_DIR, "build", os.path.basename(lib_path))
    os.makedirs(obj_dir, exist_ok=True)
    jobs = [(s, os.path.join(obj_dir, os.path.splitext(s)[0] + ".o"), extra) for s in SOURCES]
    jobs += [(s, os.path.join(obj_dir, os.path.splitext(s)[0] + "_f16.o"), extra + ["-DDISTCA_F16"]) for s in F16_SOURCES]
    objs = [j[1] for j in jobs]
    with ThreadPoolExecutor(max_workers=min(len(jobs), 8)) as ex:
        list(ex.map(lambda j: _compile(*j), jobs))
    tmp = lib_path + ".tmp"
    cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    os.replace(tmp, lib_path)
    if verbose:
        print("built", lib_path)
    return lib_path


if __name__ == "__main__":
    argv = sys.argv[1:]
    out = None
    if "-o" in argv:
        i = argv.index("-o")
        out = os.path.abspath(argv[i + 1])
        del argv[i:i + 2]
    build_library(argv, verbose=True, out_path=out)
