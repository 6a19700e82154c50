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
               "cv_matmul_i8.hip", "cv_matmul_fp8b.hip", "cv_matmul_bf16.hip", "cv_matmul_f32.hip", "cv_matmul_scalar.hip", "cv_mlp_f16.hip", "cv_mlp_f16w8.hip", "cv_mlp_f16w16.hip", "cv_mlp_f16w32.hip", "cv_mlp_fp8.hip", "cv_mlp_fp8n.hip", "cv_mlp_generic.hip", "cv_mlp_float.hip", "cv_train.hip", "cv_train_team.hip", "cv_train_quad.hip", "cv_train_general.hip", "cv_accum.hip", "cv_accum_f32.hip", "cv_accum_scalar.hip", "cv_adam.hip", "cv_elementwise.hip", "cv_permuto.hip", "cv_permuto_mlp.hip", "cv_permuto_w16.hip", "cv_permuto_w32.hip", "cv_neural.hip"]

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
                 "cv_mlp_f16.hip", "cv_mlp_f16w8.hip", "cv_mlp_f16w16.hip", "cv_mlp_f16w32.hip", "cv_mlp_fp8.hip", "cv_mlp_fp8n.hip", "cv_mlp_generic.hip", "cv_mlp_float.hip", "cv_train.hip", "cv_train_team.hip", "cv_train_quad.hip", "cv_accum.hip", "cv_permuto_mlp.hip", "cv_permuto_w16.hip", "cv_permuto_w32.hip")
}


# Kernels that keep loads in flight in registers the compiler does not know to be pending (a substring of
# the mangled name, per source file): mlpWideKernel issues its input loads and waits for them in inline
# assembly.  For these the build checks, on the generated code, that
#   - nothing spills (hipcc's kernel-resource-usage remarks): a spill or reload of such a register would
#     move stale data;
#   - between a hand-issued load (`global_load_dwordx4 ... nt` into v[a:b]) and the `s_waitcnt vmcnt(n)` that
#     covers it no instruction reads or writes v[a:b] (the device assembly, scanned in program order and once
#     around the loop; see _check_inflight_registers).
HAND_PIPELINED_KERNELS = {"cv_mlp_fp8.hip": "mlpWideKernel"}


def _check_no_spills(src: str, needle: str, remarks: str) -> None:
    name = None
    for line in remarks.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif name and needle in name:
            for key in ("VGPRs Spill:", "SGPRs Spill:", "ScratchSize [bytes/lane]:"):
                if key in line and int(line.split(key)[1].split()[0]) != 0:
                    raise RuntimeError("%s: %s of %s is not zero (%s)" % (src, key.rstrip(":"), name, line.strip()))


_VECTOR_PREFIXES = ("v_", "ds_", "global_", "scratch_", "buffer_", "flat_")
_VMEM_PREFIXES = ("global_", "scratch_", "buffer_", "flat_")


def _check_inflight_registers(src: str, needle: str, asm_text: str) -> int:
    """Returns the number of hand-issued loads checked; raises if a pending register is touched.

    From a hand-issued load (`global_load_dwordx4 v[a:b], ... nt`) every path of the function's control flow is followed
    (both sides of a conditional branch, around the loop) until the wait that covers the load: an `s_waitcnt vmcnt(n)`
    with n no larger than the number of vector-memory instructions issued on that path since the load (a larger n can
    return while the load is still on its way), or until the program ends.  On the way no instruction may name a
    register of v[a:b].  The scan fails closed: a line it cannot classify, a vector instruction whose register operands
    it cannot parse, an indirect jump or a path that runs off the end of the function is an error."""
    import re
    lines = asm_text.split("\n")
    checked = 0
    i = 0
    while i < len(lines):
        m = re.match(r"^(_Z\w+):", lines[i])
        if not (m and needle in m.group(1)):
            i += 1
            continue
        name = m.group(1)
        end = i + 1
        while end < len(lines) and not lines[end].startswith(".Lfunc_end"):
            end += 1
        # the function as a list of instructions; a label points at the instruction that follows it
        insts, labels = [], {}
        for line in lines[i + 1:end]:
            text = line.split(";")[0].strip()
            lm = re.match(r"^(\.?\w+):$", text)
            if lm:
                labels[lm.group(1)] = len(insts)
            elif text and not text.startswith("."):
                insts.append(text)
        for j, text in enumerate(insts):
            lm = re.match(r"global_load_dwordx4 v\[(\d+):(\d+)\],.* nt\b", text)
            if not lm:
                continue
            lo, hi = int(lm.group(1)), int(lm.group(2))
            checked += 1
            fewest = {}                      # instruction index -> fewest younger vector-memory instructions seen there
            work = [(j + 1, 0)]
            while work:
                k, younger = work.pop()
                while True:
                    if k >= len(insts):
                        raise RuntimeError("%s: %s: a path from the load into v[%d:%d] runs off the end of the function" % (src, name, lo, hi))
                    if k in fewest and fewest[k] <= younger:
                        break                # been here with no more vector-memory instructions behind the load
                    fewest[k] = younger
                    text = insts[k]
                    op = text.split()[0]
                    wm = re.match(r"s_waitcnt\b.*vmcnt\((\d+)\)", text)
                    if wm and int(wm.group(1)) <= younger:
                        break                # the load has landed
                    if op == "s_endpgm":
                        break
                    if op == "s_branch" or op.startswith("s_cbranch"):
                        target = text.split()[-1]
                        if target not in labels:
                            raise RuntimeError("%s: %s: branch to an unknown label: %s" % (src, name, text))
                        if op == "s_branch":
                            k = labels[target]
                            continue
                        work.append((labels[target], younger))
                    elif op.startswith(("s_setpc", "s_swappc", "s_call")):
                        raise RuntimeError("%s: %s: indirect control flow while a load is pending: %s" % (src, name, text))
                    elif op.startswith("s_"):
                        pass                 # scalar instructions cannot name a vector register
                    elif op.startswith(_VECTOR_PREFIXES):
                        operands = text[len(op):]
                        stripped = re.sub(r"\b[vas]\[\d+:\d+\]|\b[vas]\d+\b", "", operands)
                        if re.search(r"\bv\[|\bv\d", stripped):
                            raise RuntimeError("%s: %s: cannot parse the vector registers of '%s'" % (src, name, text))
                        for rm in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", operands):
                            a, b = (int(rm.group(3)),) * 2 if rm.group(3) else (int(rm.group(1)), int(rm.group(2)))
                            if not (b < lo or a > hi):
                                raise RuntimeError("%s: %s touches v[%d:%d] while its load is pending: %s" % (src, name, lo, hi, text))
                        if op.startswith(_VMEM_PREFIXES):
                            younger += 1
                    else:
                        raise RuntimeError("%s: %s: the scan does not know the instruction form '%s' (between a hand-issued "
                                           "load and its wait)" % (src, name, text))
                    k += 1
        i = end
    if checked == 0:
        raise RuntimeError("%s: no hand-issued load found in any %s (the check no longer matches the code)" % (src, needle))
    return checked


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
    if src in HAND_PIPELINED_KERNELS and "-c" in cmd:
        _check_no_spills(src, HAND_PIPELINED_KERNELS[src], proc.stdout)
        # the same translation unit once more as device assembly, for the scan of pending registers
        asm_path = cmd[cmd.index("-o") + 1][:-2] + ".s"
        asm_cmd = [c for c in cmd if not c.startswith("-Rpass-analysis")]
        asm_cmd[asm_cmd.index("-c")] = "-S"
        asm_cmd[asm_cmd.index("-o") + 1] = asm_path
        asm_cmd.insert(1, "--cuda-device-only")
        asm = subprocess.run(asm_cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if asm.returncode != 0:
            raise RuntimeError("command failed: %s\n%s" % (" ".join(asm_cmd), asm.stdout))
        with open(asm_path) as f:
            _check_inflight_registers(src, HAND_PIPELINED_KERNELS[src], f.read())
        os.remove(asm_path)


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
        remarks = ["-Rpass-analysis=kernel-resource-usage"] if src in HAND_PIPELINED_KERNELS else []
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
