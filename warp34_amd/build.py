"""Builds libwarp34_kernels.so (HIP kernels + C ABI + host-side C++ mirror) for gfx950.

hipcc cross-compiles without a GPU.  Objects are compiled one source at a time because the
quantize-on-append kernel needs -ffp-contract=off (its bits are part of the contract) while
the attention kernels want contraction.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
BUILD = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libwarp34_kernels.so")

ARCH = "gfx950"
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function"]
# packed fp32 VALU forms are kept out of every device object
DEVICE = ["--offload-arch=" + ARCH, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

SOURCES = [
    # (path, extra flags)
    (os.path.join(CSRC, "kv_write.hip"), ["-ffp-contract=off"]),
    (os.path.join(CSRC, "qk_norm_rope.hip"), ["-ffp-contract=off"]),
    (os.path.join(CSRC, "attn_output_gate.hip"), ["-ffp-contract=off"]),
    (os.path.join(CSRC, "fused_qk_norm.hip"), ["-ffp-contract=off"]),
    # leading scalar kernel arguments are preloaded into SGPRs at wave launch (gfx950 feature;
    # firmware without it runs the compatibility prologue the compiler emits)
    (os.path.join(CSRC, "paged_attn.hip"), ["-mllvm", "-amdgpu-kernarg-preload-count=12"]),
    (os.path.join(CSRC, "runtime.hip"), []),
    (os.path.join(HOST, "kv_host.cpp"), []),
    (os.path.join(HOST, "prefix_cache.cpp"), []),
    (os.path.join(HOST, "graph_io.cpp"), []),
    (os.path.join(HOST, "kv_host_runtime.cpp"), []),
    (os.path.join(HOST, "synth.cpp"), ["-pthread"]),
]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        sys.stderr.write(out + "\n")


def build(verbose=False):
    os.makedirs(BUILD, exist_ok=True)
    objs = []
    for src, extra in SOURCES:
        obj = os.path.join(BUILD, os.path.basename(src) + ".o")
        is_hip = src.endswith(".hip")
        cmd = ["hipcc"] + COMMON + (DEVICE if is_hip else ["-x", "c++"]) + extra + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd))
        _run(cmd)
        objs.append(obj)
    _run(["hipcc", "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
