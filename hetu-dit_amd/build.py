"""Builds ``libhdit.so`` (the C-ABI library of hand-written gfx950 kernels)
in-tree with hipcc.  Cross-compiles without a GPU."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libhdit.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-fno-honor-nans",  # no kernel relies on NaN propagation; lets fmax chains become v_max3 without canonicalisation
    # packed-fp32 VALU forms are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# Per-file additions.  attention_bf16.hip: its pipelined kernel runs one wave per SIMD with 512 registers, where
# the compiler would otherwise keep every MFMA accumulator in the AGPR half -- and the softmax (VALU) cannot read
# those without a copy per score.  In the VGPR form the allocator decides per value.
EXTRA_FLAGS = {
    "attention_bf16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def build_library(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in sources():
        obj = os.path.join(CSRC, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc] + HIPCC_FLAGS + EXTRA_FLAGS.get(os.path.basename(src), []) + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        if verbose and text.strip():
            print(text)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
