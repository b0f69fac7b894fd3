"""Runs the C++ testbench-style harness (flexllm_amd/host/tb/modules_tb.cpp): the reference's module call surface
(pref_/dec_ quant, Linear_Layer, FHT, Layer_Norm, Swish, Gate, Residual, Softmax, RoPE, the prefill and decode MHA
module chains and their fused tops, the decode top launched through the invoke shim on the reference's cache lines,
the int4 weight-word and cache-line adapters, the linear testbench tops launched through the invoke shim on the
testbenches' packed int4 weight words, the prefill int4 linear module, the top-k and sampling + embedding layers) driven through stream packings exactly as the reference's *_tb.cpp files
drive theirs, with in-process goldens."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "flexllm_amd", "host", "tb", "modules_tb")


def test_cpp_module_harness_passes():
    assert os.path.exists(BIN), "build it with `python -m flexllm_amd.build` (or __graft_entry__.build())"
    out = subprocess.run([BIN], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(out.stdout)
    assert out.returncode == 0, out.stdout
    assert out.stdout.count("passed correctness check") == 17 and "failed" not in out.stdout
