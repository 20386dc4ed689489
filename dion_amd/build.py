"""Builds the gfx950 shared library `dion_amd/libdion_amd.so` from `dion_amd/csrc/*.hip`.

Run as `python -m dion_amd.build`.  hipcc cross-compiles without a GPU present.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
# Measurement builds: DION_AMD_BUILD_DEFINES holds extra compiler options (e.g. "-DDA_MI=32"), DION_AMD_BUILD_LIB the
# library to write instead of the in-tree one (its objects go beside it); load it with DION_AMD_LIB.
LIB = os.environ.get("DION_AMD_BUILD_LIB") or os.path.join(HERE, "libdion_amd.so")
if os.environ.get("DION_AMD_BUILD_LIB"):
    OBJ = LIB + ".obj"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # the elementwise passes and GEMM epilogues reproduce the reference's separate
    # multiply / add roundings: no fused multiply-add contraction
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    *os.environ.get("DION_AMD_BUILD_DEFINES", "").split(),
]


# MFMA accumulators of the fp64 / fp32 kernels stay in ordinary VGPRs: left to its heuristic the compiler
# keeps them in AGPRs only inside the MFMA blocks and copies all of them over and back on every loop
# iteration (32 v_accvgpr_write + 32 v_accvgpr_read per 16 MFMAs; 4-6 % of the orthonormaliser).  The bf16
# kernel, whose K loop has no such copies, measured 2 % slower with the option and is built without it.
PER_FILE_FLAGS = {
    "gemm_f64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_f32.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    # (cholesky.hip also: without the second option the compiler merges the stores of two branches into different
    # named register tiles into one store through a selected pointer, and both tiles then live in scratch memory)
    "cholesky.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1", "-mllvm", "-simplifycfg-sink-common=false"],
}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ, src[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, *PER_FILE_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, res


def build(verbose=True, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), 8)
    objs = []
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, obj, res in pool.map(_compile, srcs):
            err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
            if res.returncode != 0:
                raise RuntimeError(f"hipcc failed on {src}:\n{err}")
            if verbose and err.strip():
                print(err, file=sys.stderr)
            objs.append(obj)
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    res = subprocess.run(link, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build()
