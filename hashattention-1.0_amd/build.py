"""Build the HIP library for gfx950:  python build.py  ->  hashattention/libhashattn.so

hipcc cross-compiles without a GPU.  Packed-FP32 instruction selection is switched off for all
device code (`-packed-fp32-ops`), see the flags below.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCES = ["ha_core.hip", "ha_encode.hip", "ha_encode_mfma.hip", "ha_encode_mfma_f32.hip", "ha_select.hip", "ha_select_sampled.hip", "ha_attend.hip", "ha_decoder.hip"]
LIB = os.path.join(HERE, "hashattention", "libhashattn.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def build(verbose: bool = True, extra_flags=()) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(HERE, "csrc", s) for s in SOURCES if os.path.exists(os.path.join(HERE, "csrc", s))]
    cmd = [hipcc, *FLAGS, *extra_flags, "-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc"), *srcs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
