"""The f16 kernels must round the fold to binary32 before narrowing.  hipcc is able to fuse the
fold's last multiply with the narrowing into one v_fma_mixlo_f16 (one rounding of the exact
product instead of two), which differs from the CPU checker on exact ties.  This compiles the
f16 instances to assembly (device pass only, no GPU needed) and looks for what must not be there."""
import os
import re
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "pccl_amd", "csrc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-I" + os.path.join(ROOT, "include"),
         "-I" + os.path.join(CSRC, "hip"), "--cuda-device-only", "-S"]
FORBIDDEN = re.compile(r"\b(v_fma_mix\w*|v_mad_mix\w*|v_pk_(?:add|mul|fma)_f32|v_cvt_pkrtz_f16_f32)\b")


def _assembly(name, out_dir):
    out = os.path.join(out_dir, name + ".s")
    subprocess.run(["hipcc"] + FLAGS + ["-o", out, os.path.join(CSRC, "hip", name + ".hip")], check=True,
                   stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=600)
    with open(out) as f:
        return f.read()


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_f16_kernels_hold_no_fused_or_packed_float_arithmetic():
    with open(os.path.join(CSRC, "Makefile")) as f:
        assert "-ffp-contract=off" in f.read(), "the build must not contract a*b+c"
    with tempfile.TemporaryDirectory() as d, ThreadPoolExecutor(2) as pool:
        texts = list(pool.map(lambda n: _assembly(n, d), ["reduce_copy_inst_f16", "graph_queue_inst_f16"]))
    for name, text in zip(["reduce_copy_inst_f16", "graph_queue_inst_f16"], texts):
        assert "v_cvt_f16_f32" in text, name + ": expected the plain narrowing instruction"
        found = sorted(set(FORBIDDEN.findall(text)))
        assert not found, "%s: %s" % (name, found)
