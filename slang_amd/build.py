"""Build recipe for the gfx950 library and (optionally) the CPU oracle.

    python -m slang_amd.build            # compile slang_amd/libcoopvec_mi355x.so
    python -m slang_amd.build --oracle   # also oracle/libcoopvec_oracle.so

hipcc cross-compiles for gfx950 without a GPU.  Objects go to build/ (git-ignored), the
shared library next to this file so that it travels with the source tree.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libcoopvec_mi355x.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)
ORACLE_DIR = os.path.join(REPO_DIR, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "libcoopvec_oracle.so")

HIP_SOURCES = ["cv_abi.hip", "cv_convert.hip", "cv_matmul_f16.hip", "cv_matmul_fp8.hip",
               "cv_matmul_i8.hip", "cv_matmul_fp8b.hip", "cv_matmul_bf16.hip", "cv_matmul_f32.hip", "cv_mlp_f16.hip", "cv_mlp_fp8.hip", "cv_mlp_fp8n.hip", "cv_mlp_generic.hip", "cv_train.hip", "cv_train_general.hip", "cv_accum.hip", "cv_adam.hip", "cv_elementwise.hip", "cv_permuto.hip", "cv_neural.hip"]

# packed-fp32 instructions are switched off on purpose (see the flag below): hipcc would
# otherwise form v_pk_*_f32 from ordinary float code.  -ffp-contract=off: the kernels state every
# rounding point of the Slang source (each half product and sum rounded on its own); hipcc's default
# would fuse a rounded product and a following sum into one fma with a single rounding.  Where a
# fused multiply-add is wanted it is written as one.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fvisibility=hidden", "-fno-strict-aliasing",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# Forward kernels read every MFMA result with the VALU right away, so their MFMAs write VGPRs
# directly; left to its heuristics the compiler parks results in AGPRs and copies them back.
# (The training kernel pins its gradient accumulators to AGPRs itself.)
PER_FILE_FLAGS = {
    name: ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]
    for name in ("cv_matmul_f16.hip", "cv_matmul_fp8.hip", "cv_matmul_i8.hip", "cv_matmul_fp8b.hip", "cv_matmul_bf16.hip", "cv_matmul_f32.hip",
                 "cv_mlp_f16.hip", "cv_mlp_fp8.hip", "cv_mlp_fp8n.hip", "cv_mlp_generic.hip", "cv_train.hip", "cv_accum.hip")
}


# Kernels that must compile without register spills (a substring of the mangled name, per source file):
# mlpWideKernel keeps loads in flight in registers the compiler does not know to be pending, so a spill or
# reload of such a register would move stale data.  Checked from hipcc's kernel-resource-usage remarks.
NO_SPILL_KERNELS = {"cv_mlp_fp8.hip": "mlpWideKernel"}


def _check_no_spills(src: str, needle: str, remarks: str) -> None:
    name = None
    for line in remarks.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif name and needle in name:
            for key in ("VGPRs Spill:", "SGPRs Spill:", "ScratchSize [bytes/lane]:"):
                if key in line and int(line.split(key)[1].split()[0]) != 0:
                    raise RuntimeError("%s: %s of %s is not zero (%s)" % (src, key.rstrip(":"), name, line.strip()))


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    src = os.path.basename(next((c for c in cmd if c.endswith(".hip")), ""))
    if src in NO_SPILL_KERNELS:
        _check_no_spills(src, NO_SPILL_KERNELS[src], proc.stdout)


def build_library(jobs: int = 8, verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 and link the shared library.  Always recompiles."""
    hipcc = _hipcc()
    obj_dir = os.path.join(REPO_DIR, "build", "obj")
    os.makedirs(obj_dir, exist_ok=True)
    sources = [s for s in HIP_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = []
    cmds = []
    for src in sources:
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        objs.append(obj)
        remarks = ["-Rpass-analysis=kernel-resource-usage"] if src in NO_SPILL_KERNELS else []
        cmds.append([hipcc, *HIPCC_FLAGS, *PER_FILE_FLAGS.get(src, []), *remarks, "-I", os.path.join(REPO_DIR, "include"), "-c",
                     os.path.join(CSRC, src), "-o", obj])
    with cf.ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        for cmd, _ in zip(cmds, pool.map(_run, cmds)):
            if verbose:
                print(" ".join(cmd))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


HOST_SRC = os.path.join(PKG_DIR, "host", "mlp_training_host.cpp")
HOST_BIN = os.path.join(PKG_DIR, "host", "mlp_training_host")


def build_host_example() -> str:
    """Compile the host program that trains the example network through the C-ABI."""
    _run([_hipcc(), "-O2", "-std=c++17", "-I", os.path.join(REPO_DIR, "include"), HOST_SRC, "-o", HOST_BIN,
          "-L", PKG_DIR, "-l:" + LIB_NAME, "-Wl,-rpath,$ORIGIN/.."])
    return HOST_BIN


def build_oracle() -> str:
    """Compile the CPU oracle (test infrastructure) with the host C compiler."""
    _run(["make", "-C", ORACLE_DIR, "-B", "libcoopvec_oracle.so"])
    return ORACLE_LIB


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--oracle", action="store_true", help="also build the CPU oracle")
    ap.add_argument("-j", "--jobs", type=int, default=8)
    ap.add_argument("-v", "--verbose", action="store_true")
    args = ap.parse_args(argv)
    print(build_library(args.jobs, args.verbose))
    print(build_host_example())
    if args.oracle:
        print(build_oracle())
    return 0


if __name__ == "__main__":
    sys.exit(main())
