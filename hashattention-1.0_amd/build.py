"""Build the HIP library for gfx950:  python build.py  ->  hashattention/libhashattn.so

hipcc cross-compiles without a GPU.  Packed-FP32 instruction selection is switched off for all
device code (`-packed-fp32-ops`), see the flags below.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SOURCES = ["ha_core.hip", "ha_encode.hip", "ha_encode_mfma.hip", "ha_encode_mfma_f32.hip", "ha_select.hip", "ha_select_sampled.hip", "ha_attend.hip", "ha_decoder.hip", "ha_linear_tiled.hip"]
LIB = os.path.join(HERE, "hashattention", "libhashattn.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


# The same library with -DHASHATTN_STAGE_WAIT_ALL: the fused attention launch then waits for ALL of a wave's outstanding
# requests wherever the shipped build waits for "all but the eight youngest" (the hand-counted wait for the codes staged
# through LDS).  A test runs both builds on the same inputs and demands identical bits, so a change that breaks what the
# counted wait relies on shows up as a difference instead of as a wrong selection on some shape.
LIB_WAIT_ALL = os.path.join(HERE, "hashattention", "libhashattn_waitall.so")


def _command(out: str, extra_flags=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(HERE, "csrc", s) for s in SOURCES if os.path.exists(os.path.join(HERE, "csrc", s))]
    return [hipcc, *FLAGS, *extra_flags, "-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc"), *srcs, "-o", out]


def build(verbose: bool = True, extra_flags=(), variants: bool = True) -> str:
    """Compile the library (and, side by side, its HASHATTN_STAGE_WAIT_ALL twin for the tests)."""
    cmds = [_command(LIB, extra_flags)]
    if variants:
        cmds.append(_command(LIB_WAIT_ALL, (*extra_flags, "-DHASHATTN_STAGE_WAIT_ALL")))
    procs = []
    for cmd in cmds:
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append(subprocess.Popen(cmd))
    codes = [p.wait() for p in procs]
    if any(codes):
        raise subprocess.CalledProcessError(next(c for c in codes if c), cmds[0])
    return LIB


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
