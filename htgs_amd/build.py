"""Builds ``libhtgs_amd.so`` (gfx950 only) from ``csrc/*.hip`` with hipcc, and the separate counter-calibration library
``diagnostics/libhtgs_copy.so`` (a plain copy kernel) from ``diagnostics/copy_kernel.hip``.

Both are built in-tree.  ``python -m htgs_amd.build`` rebuilds them.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libhtgs_amd.so")
OBJ_DIR = os.path.join(HERE, "build")
COPY_SRC = os.path.join(HERE, "diagnostics", "copy_kernel.hip")
COPY_LIB_PATH = os.path.join(HERE, "diagnostics", "libhtgs_copy.so")

# -ffp-contract=off: a fused multiply-add exists only where the sources write __builtin_fmaf, which is what
#   makes tile counts and accept/reject decisions reproducible (see csrc/common.h).
# -packed-fp32-ops disabled: no v_pk_{add,mul,fma}_f32.
# -disable-promote-alloca-to-vector: the K-buffer arrays of the blend kernels (constant indices once the loops are
#   unrolled) must end up as individual registers; promoted early to one 16- or 32-wide vector value they are allocated
#   as a register tuple and spilled around the insertion chain.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-disable-promote-alloca-to-vector=1",
    "-Wno-unused-command-line-argument",
]


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def csrc_digest() -> str:
    """SHA-256 over the kernel sources and the C ABI header: the code version a profile-derived figure is tied to."""
    import hashlib
    h = hashlib.sha256()
    for path in [*sources(), *sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")),
                 os.path.join(os.path.dirname(HERE), "include", "htgs_amd.h")]:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; that line is noise
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def build(verbose: bool = False) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = _hipcc()
    srcs = sources()
    objs = [os.path.join(OBJ_DIR, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        cmd = [hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd))
        _run(cmd)

    copy_obj = os.path.join(OBJ_DIR, "copy_kernel.o")
    with ThreadPoolExecutor(max_workers=min(8, len(srcs) + 1)) as pool:
        list(pool.map(compile_one, [*zip(srcs, objs), (COPY_SRC, copy_obj)]))
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wno-unused-command-line-argument"]
    for lib_objs, path in ((objs, LIB_PATH), ([copy_obj], COPY_LIB_PATH)):
        tmp = path + ".tmp"
        _run([*link, *lib_objs, "-o", tmp])
        os.replace(tmp, path)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
