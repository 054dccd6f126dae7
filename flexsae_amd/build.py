"""Builds libflexsae_amd.so (the C-ABI library of HIP kernels) in-tree with hipcc for gfx950.

Usage: python -m flexsae_amd.build
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libflexsae_amd.so")

# gfx950 only: some kernels use more LDS per workgroup than the 64 KiB of earlier gfx9 parts
# (csr_sort_long_kernel 65 600 bytes, the hot-latent variant of the training-step kernel more), the
# gfx950 lane-swap and bf16 conversion instructions, and buffer loads with the LDS as destination.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-munsafe-fp-atomics",
    # keep the compiler from forming packed-fp32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def source_id(extra_flags=()) -> str:
    """Identifier of what the library is built from: a hash over the kernel sources, the header and
    the compiler flags (not over the binary, so that rebuilding the same sources gives the same id).
    The library reports it through flexsae_build_id(); measurements kept under profiles/ carry it."""
    import hashlib

    h = hashlib.sha256()
    files = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".hpp")))
    files.append(os.path.join(os.path.dirname(HERE), "include", "flexsae_amd.h"))
    for path in files:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as fh:
            h.update(fh.read())
    h.update(" ".join([*HIPCC_FLAGS, *extra_flags]).encode())
    return h.hexdigest()[:16]


def build(verbose: bool = False, extra_flags=()) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, f'-DFLEXSAE_BUILD_ID="{source_id(extra_flags)}"', "-o", LIB_PATH,
           os.path.join(CSRC, "flexsae_amd.hip")]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building libflexsae_amd.so")
    if verbose and proc.stderr:
        sys.stderr.write(proc.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
