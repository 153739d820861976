"""Compiler-level property of the bits top-k kernel: its streaming loop is wave-uniform.

A lane-dependent branch next to a loop exit is enough for LLVM's uniformity analysis to treat the
loop state as differing between lanes; the streaming loop then becomes an exec-masked loop with
its counters in vector registers and a flat load for the merge flag.  The analysis of the
kernel's IR must therefore report no cycle with a divergent exit.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "bits-knn-jpdc2024_amd", "csrc")
OPT = "/opt/rocm/llvm/bin/opt"

SOURCE = """
#include "topk_bits_kernel.hpp"
namespace bitsknn {
template __global__ void bits_topk_kernel<256, 1, 2, true>(const topk_args a);
template __global__ void bits_topk_kernel<512, 4, 1, true>(const topk_args a);
template __global__ void bits_topk_kernel<128, 2, 2, false>(const topk_args a);
}
"""


@pytest.mark.skipif(shutil.which("hipcc") is None or not os.path.exists(OPT),
                    reason="needs hipcc and LLVM's opt")
def test_streaming_loop_of_the_bits_kernel_is_wave_uniform(tmp_path):
    src = tmp_path / "inst.hip"
    src.write_text(SOURCE)
    ir = tmp_path / "inst.ll"
    subprocess.run(["hipcc", "-O3", "-std=c++20", "--offload-arch=gfx950", "-I", os.path.join(ROOT, "include"),
                    "-I", CSRC, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                    "-Wno-unused-command-line-argument", "-S", "-emit-llvm", "--cuda-device-only",
                    "-o", str(ir), str(src)], check=True, capture_output=True, timeout=600)
    report = subprocess.run([OPT, "-mtriple=amdgcn-amd-amdhsa", "-mcpu=gfx950", "-passes=print<uniformity>",
                             "-disable-output", str(ir)], check=True, capture_output=True, text=True,
                            timeout=600).stderr
    assert report.count("UniformityInfo for function") == 3
    assert "CYCLES WITH DIVERGENT EXIT" not in report
