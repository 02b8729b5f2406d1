"""Builds libgq_hip.so (gfx950) from csrc/*.hip with hipcc.  Usage: python build.py [--check-isa]

Takes the place of the reference's cppimport-on-first-import build
(popxl_addons/ops/group_quantize_decompress/group_quantize_decompress_binding.cpp:57-66):
here the library is compiled ahead of time, in-tree, and loaded with ctypes.
"""
import concurrent.futures
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libgq_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

SOURCES = ["gq_api.hip", "gq_decompress.hip", "gq_compress.hip", "gq_gemv.hip", "gq_gemv_stream.hip", "gq_gemv_flow.hip", "gq_gemm.hip", "gq_linear_kn.hip",
           "gq_gemv_kn.hip", "gq_gemv_sums.hip", "gq_gemv_rows.hip"]

# -ffp-contract=off: the decompress contract is "fp16 multiply, then fp16 add" (two roundings);
# kernels that want an fma ask for one explicitly.  Packed-fp32 instruction selection is disabled.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
    "-I", INCLUDE, "-I", CSRC,
]

# kernels whose result must be bit-exact: no fused fp16 multiply-add may appear in their ISA
NO_FMA_SOURCES = {"gq_decompress.hip": r"v_(pk_)?(fma|mad|fmac)_f16|v_fma_mix"}
# kernels that count their outstanding vector-memory operations by hand (s_waitcnt vmcnt(N) with
# direct-to-LDS loads): a register spill would add scratch accesses to that count
NO_SCRATCH_SOURCES = ["gq_gemv_stream.hip", "gq_gemv_flow.hip", "gq_gemm.hip", "gq_linear_kn.hip",
           "gq_gemv_kn.hip", "gq_gemv_sums.hip", "gq_gemv_rows.hip"]


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError(f"command failed: {cmd[0]} ... {cmd[-1]}")
    return proc


def _compile(src):
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    _run([HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    return obj


def check_isa():
    """Disassembly of our own kernels: the bit-exact ones must keep multiply and add apart."""
    for src, pattern in NO_FMA_SOURCES.items():
        asm = os.path.join(OBJ_DIR, src.replace(".hip", ".s"))
        _run([HIPCC, *FLAGS, "-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", asm])
        text = open(asm).read()
        hits = re.findall(pattern, text)
        if hits:
            raise RuntimeError(f"{src}: fused fp16 multiply-add in ISA ({sorted(set(map(str, hits)))})")
        if "v_pk_mul_f16" not in text or "v_pk_add_f16" not in text:
            raise RuntimeError(f"{src}: expected v_pk_mul_f16 and v_pk_add_f16 in ISA")
    for src in NO_SCRATCH_SOURCES:
        asm = os.path.join(OBJ_DIR, src.replace(".hip", ".s"))
        _run([HIPCC, *FLAGS, "-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", asm])
        text = open(asm).read()
        if re.search(r"^\s*scratch_(load|store)", text, re.M):
            raise RuntimeError(f"{src}: registers spill to scratch memory")


def build(check=True, jobs=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs or min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    if check:
        check_isa()
    return LIB_PATH


if __name__ == "__main__":
    print(build(check="--no-check-isa" not in sys.argv))
