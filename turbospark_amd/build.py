"""Builds turbospark_amd/libtsverify.so (HIP kernels + C ABI) for gfx950 with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, os.environ.get("TSV_LIB_NAME", "libtsverify.so"))
SOURCES = ["gemm.hip", "moe.hip", "moe_fp4.hip", "misc.hip", "attn.hip", "kvquant.hip", "accept.hip", "host_utils.hip", "runtime.hip", "mtp.hip", "testing.hip", "loop.hip", "gguf.hip"]
# host_utils.hip is host-only code; clang 22 -O3 does not terminate on it, -O2 does.
OPT = {"host_utils.hip": "-O2", "gguf.hip": "-O2"}
# MFMA results straight into VGPRs (no v_accvgpr_read copies before the scaling FMAs)
EXTRA = {"gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"] + os.environ.get("TSV_GEMM_DEFS", "").split(),
         "moe.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
         "moe_fp4.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}
FLAGS = [
    "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # no implicit multiply-add fusion: the compiler picks the fused operand per template instantiation, and
    # kernels are instantiated by row count, so a row's bits would depend on the width of its pass; the
    # hot loops write their fmaf out, everything else rounds like the reference's unfused f32 / f64 code
    "-ffp-contract=off",
    # packed-fp32 VALU forms are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-pthread",
]
# TSV_HOST_UBSAN=1: the host pass of every source under the undefined-behaviour sanitizer in trap mode (no runtime
# to link; device code is compiled as always), objects kept apart.  With TSV_LIB_NAME=libtsverify_ubsan.so for both
# the build and the tests, every host path the suites reach either is clean or stops the process where it is not.
HOST_UBSAN = os.environ.get("TSV_HOST_UBSAN", "0") == "1"
if HOST_UBSAN:
    FLAGS += ["-Xarch_host", "-fsanitize=undefined,bounds", "-Xarch_host", "-fsanitize-trap=all", "-g"]
OBJ_DIR = "build_ubsan" if HOST_UBSAN else "build"


def build(verbose=False):
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, OBJ_DIR), exist_ok=True)
    for src in SOURCES:
        obj = os.path.join(HERE, OBJ_DIR, src.replace(".hip", ".o"))
        cmd = ["hipcc", OPT.get(src, "-O3"), *FLAGS, *EXTRA.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        try:
            out, _ = p.communicate(timeout=900)
        except subprocess.TimeoutExpired:
            p.kill()
            out, _ = p.communicate()
            out += b"\n(compiler killed after 900 s)"
            p.returncode = -9
        text = out.decode(errors="replace")
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"--- {src} failed ---\n{text}\n")
        elif verbose and text.strip():
            print(f"--- {src} ---\n{text}")
    if failed:
        raise RuntimeError("hipcc failed")
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-pthread", *objs, "-o", LIB])
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
