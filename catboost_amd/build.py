"""Builds libcatboostmodel.so (host C++ + HIP kernels for gfx950) in-tree with hipcc.

    python -m catboost_amd.build          # rebuild
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libcatboostmodel.so")

HOST_SOURCES = ["model.cpp", "cbm_format.cpp", "json_model.cpp", "model_builder.cpp", "cat_hash.cpp", "fast_exp.cpp", "c_api.cpp"]
HIP_SOURCES = ["hip_evaluator.hip"]

COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter", "-ffp-contract=off"]
# packed fp32 VALU forms are kept off for every device function of this library
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc():
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        raise RuntimeError("hipcc not found: the evaluator cannot be built without ROCm")
    return path


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass of hipcc does not know the packed-fp32 target feature and says so; harmless
    out = "\n".join(line for line in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in line and "is not a recognized feature" not in line)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return out


def _build_eval_reg_code_object():
    """gen_eval_reg_kernel.py -> assembly -> gfx950 code object -> byte list included by hip_evaluator.hip"""
    llvm = os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(_hipcc()))), "llvm", "bin")
    if not os.path.isdir(llvm):
        llvm = "/opt/rocm/llvm/bin"
    asm = os.path.join(OBJ_DIR, "eval_reg_kernel.s")
    obj = os.path.join(OBJ_DIR, "eval_reg_kernel.o")
    co = os.path.join(OBJ_DIR, "eval_reg_kernel.co")
    _run([sys.executable, os.path.join(CSRC, "gen_eval_reg_kernel.py"), asm])
    _run([os.path.join(llvm, "clang"), "-x", "assembler", "-target", "amdgcn-amd-amdhsa", "-mcpu=gfx950", "-c", asm,
          "-o", obj])
    _run([os.path.join(llvm, "ld.lld"), "-shared", "-o", co, obj])
    with open(co, "rb") as f:
        data = f.read()
    with open(os.path.join(OBJ_DIR, "eval_reg_kernel_co.inc"), "w") as f:
        for i in range(0, len(data), 32):
            f.write(",".join(str(b) for b in data[i:i + 32]) + ",\n")


def build(verbose=False):
    hipcc = _hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    _build_eval_reg_code_object()
    jobs = []
    for src in HOST_SOURCES:
        obj = os.path.join(OBJ_DIR, src + ".o")
        jobs.append((obj, [hipcc, "-x", "c++"] + COMMON + ["-c", os.path.join(CSRC, src), "-o", obj]))
    for src in HIP_SOURCES:
        obj = os.path.join(OBJ_DIR, src + ".o")
        jobs.append((obj, [hipcc, "-x", "hip"] + COMMON + DEVICE + ["-I", OBJ_DIR, "-c", os.path.join(CSRC, src), "-o", obj]))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        for out in pool.map(lambda j: _run(j[1]), jobs):
            if verbose and out.strip():
                print(out)
    objs = [j[0] for j in jobs]
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "-shared", "-fPIC", "-o", tmp] + objs + ["--offload-arch=gfx950"])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
