"""Builds libaion_hip.so (gfx950) in-tree with hipcc: python -m aion_amd.build"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libaion_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
SOURCES = ["ctx.hip", "quant.hip", "weights.hip", "gemv.hip", "gemv_fused.hip", "gemv_ksplit.hip", "gemv_mfma.hip", "gemm.hip", "matmul.hip", "matmul_nt_f32.hip", "attention.hip", "attention_prefill.hip", "decode_stack.hip", "glue.hip", "program.hip", "session.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result",
    # hipcc -O3 may otherwise form packed-f32 instructions, which have given wrong results on this pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first 16 dwords of a kernel's arguments arrive in SGPRs with the wavefront instead of through a scalar load: one
    # memory round trip less at the head of every latency-bound kernel
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


# per-file additions: the prefill attention kernel keeps MFMA results in vector registers (its softmax reads the scores
# where the MFMA wrote them; with the default form every score passes through an accumulation-register copy)
EXTRA_FLAGS = {"attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _compile(src):
    obj = os.path.join(CSRC, src[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=False):
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
