"""Compile the HIP sources under ``csrc/`` into ``csrc/libchr_nf4_amd.so`` for gfx950.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is
installed.  The library is built in-tree; nothing is installed.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libchr_nf4_amd.so")
SOURCES = ("nf4_gemv.hip", "nf4_codec.hip", "nf4_attn.hip", "nf4_gemm.hip", "dv2_state.hip",
           "dv2_prefill.hip")
HEADERS = ("nf4_common.h", "nf4_gemv_ring_regs.h", os.path.join("..", "..", "include", "chr_nf4_amd.h"))

#: -packed-fp32-ops is switched off on purpose: the kernels are written for
#: scalar fp32 VALU ops only.
HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the ring GEMV's asm names registers that its kernels keep away from the compiler;
    # clang remarks on every such clobber list
    "-Wno-inline-asm",
)


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the NF4 kernels need the ROCm toolchain to build")
    return exe


def have_hipcc() -> bool:
    return bool(shutil.which("hipcc")) or os.path.exists("/opt/rocm/bin/hipcc")


def stale() -> bool:
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, s) for s in SOURCES + HEADERS]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = True, verbose: bool = False) -> str:
    """Run hipcc.  ``force=False`` skips the compile when the library is newer
    than every source."""
    if not force and not stale():
        return LIB
    cmd = [hipcc(), *HIPCC_FLAGS, "-o", LIB, *[os.path.join(CSRC, s) for s in SOURCES]]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the device-only target feature and says so
    # once per source; that line is noise, everything else is shown.
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    # the ring GEMV kernels rely on what the compiler did with their asm: read it back
    from . import ring_asm_check

    ring_asm_check.check_source(hipcc(), HIPCC_FLAGS, os.path.join(CSRC, "nf4_gemv.hip"))
    build_host_check()
    build_launch_probe()
    return LIB


#: A caller of the C-ABI written in C++ with no Python in the process; the tests run it.
HOST_CHECK_SRC = os.path.join(CSRC, "..", "..", "tests", "cabi", "host_check.cpp")
HOST_CHECK = os.path.splitext(HOST_CHECK_SRC)[0]


def build_host_check() -> str | None:
    """Link ``tests/cabi/host_check`` against the library just built (skipped when the
    package is used without its test tree)."""
    if not os.path.exists(HOST_CHECK_SRC):
        return None
    include = os.path.join(CSRC, "..", "..", "include")
    cmd = [hipcc(), "-O2", "-std=c++17", "-I", include, "-o", HOST_CHECK, HOST_CHECK_SRC,
           "-L", CSRC, "-lchr_nf4_amd", "-Wl,-rpath,$ORIGIN/../../deep-fold_amd/csrc"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on host_check.cpp ({proc.returncode}):\n{proc.stderr}")
    return HOST_CHECK


#: A stand-alone measurement program (no library code, no torch): launch floor, streaming-read
#: ceiling, where the time before a launch's first product goes, and chains of launches that
#: overlap through device words.  ``profiles/launch_*.txt`` are its output.
LAUNCH_PROBE_SRC = os.path.join(CSRC, "launch_probe.hip")
LAUNCH_PROBE = os.path.splitext(LAUNCH_PROBE_SRC)[0]


def build_launch_probe() -> str:
    cmd = [hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           # scalar kernel arguments arrive in registers (one of the things the program measures)
           "-mllvm", "-amdgpu-kernarg-preload-count=16",
           "-o", LAUNCH_PROBE, LAUNCH_PROBE_SRC]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on launch_probe.hip ({proc.returncode}):\n{proc.stderr}")
    return LAUNCH_PROBE


if __name__ == "__main__":
    print(build(force=True, verbose=True))
