"""Builds libneura_hip.so (gfx950 only) in-tree with hipcc.

    python -m neura_amd.build          # compile every .hip file and link

-ffp-contract=off: every fused multiply-add in the kernels is written as fmaf(); plain
a*b+c stays two roundings, which the bit-exact dequantisation and the norm's sum of squares
depend on.  Packed fp32 arithmetic is switched off for the device pass.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBRARY = os.path.join(HERE, "libneura_hip.so")
SOURCES = ["runtime.hip", "codec.hip", "gemv.hip", "gemv_tile16.hip", "gemv_q6k_tile16.hip", "gemm.hip", "rowops.hip", "attention.hip", "argmax.hip", "sample.hip", "model.hip"]
# -amdgpu-kernarg-preload-count: the hardware hands a kernel's leading plain arguments (up to 14 words) to every wave in scalar
# registers as it starts it, so a kernel's first loads need not wait for a load of its arguments (about 0.5 us a launch);
# kernels that take a parameter struct name what they need first as leading arguments for this
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-lambda-capture",
]


def hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


# per file: the 16-row tile product and the attention kernels work on their matrix-core sums where they land, in vector registers
EXTRA_FLAGS = {"gemv_tile16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "gemv_q6k_tile16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _compile(source):
    obj = os.path.join(CSRC, source.replace(".hip", ".o"))
    cmd = [hipcc(), *FLAGS, *EXTRA_FLAGS.get(source, []), "-c", os.path.join(CSRC, source), "-o", obj]
    done = subprocess.run(cmd, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (source, " ".join(cmd), done.stderr))
    noise = "'-packed-fp32-ops' is not a recognized feature"
    warnings = "\n".join(line for line in done.stderr.splitlines() if noise not in line)
    return obj, warnings


def build_library(verbose=True):
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        results = list(pool.map(_compile, SOURCES))
    objects = [obj for obj, _ in results]
    if verbose:
        for source, (_, warnings) in zip(SOURCES, results):
            if warnings.strip():
                print("[%s]\n%s" % (source, warnings), file=sys.stderr)
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIBRARY, *objects]
    done = subprocess.run(cmd, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), done.stderr))
    return LIBRARY


HOST_LIBRARY = os.path.join(HERE, "libneura_host.so")


def build_host(verbose=True):
    """The C++ host layer (GGUF reader, decoder declarations, generation batch) over the C ABI,
    with its flat C surface; plain g++, no device code.  Links against libneura_hip.so."""
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-Wall", "-Wextra", "-fPIC", "-shared",
           os.path.join(HERE, "host", "capi.cpp"), "-o", HOST_LIBRARY,
           "-L" + HERE, "-lneura_hip", "-Wl,-rpath,$ORIGIN"]
    done = subprocess.run(cmd, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError("host build failed:\n%s\n%s" % (" ".join(cmd), done.stderr))
    if verbose and done.stderr.strip():
        print(done.stderr, file=sys.stderr)
    return HOST_LIBRARY


if __name__ == "__main__":
    print(build_library())
    print(build_host())
