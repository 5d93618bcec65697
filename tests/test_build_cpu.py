"""Compile-time properties of the device code, checked without a GPU (hipcc cross-compiles gfx950)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "hashattention-1.0_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.mark.skipif(not (os.path.exists(HIPCC) or shutil.which("hipcc")), reason="hipcc not available")
def test_attention_and_selection_kernels_keep_their_registers():
    # A register of the gather loop that is spilled to scratch costs the headline launch several microseconds (every reload
    # is a vector-memory operation whose wait drains the row loads the loop keeps in flight), and it happens silently when
    # a kernel that sits at its register budget gains one more live value.  The compiler reports scratch per kernel.
    from importlib import util
    spec = util.spec_from_file_location("hashattn_build", os.path.join(ROOT, "hashattention-1.0_amd", "build.py"))
    mod = util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    flags = [f for f in mod.FLAGS if f not in ("-shared",)]
    for src in ("ha_attend.hip", "ha_select.hip"):
        cmd = [HIPCC if os.path.exists(HIPCC) else "hipcc", *flags, "-c", "-Rpass-analysis=kernel-resource-usage", "-I",
               os.path.join(ROOT, "include"), "-I", CSRC, os.path.join(CSRC, src), "-o", os.devnull]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        names = re.findall(r"Function Name: (\S+)", r.stderr)
        scratch = [int(x) for x in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", r.stderr)]
        assert names and len(names) == len(scratch)
        spilled = {n: s for n, s in zip(names, scratch) if s and "kernel" in n}
        assert not spilled, f"{src}: kernels with registers spilled to scratch: {spilled}"
