"""Builds libflexllm_hip.so (gfx950) in-tree with hipcc.  `python -m flexllm_amd.build`."""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libflexllm_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # the reference's arithmetic has no fused multiply-add: keep mul and add separate
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", *os.environ.get("FLEXLLM_EXTRA_FLAGS", "").split(),
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose=False, jobs=8):
    objs = []
    procs = []
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    for src in sources():
        obj = os.path.join(CSRC, "build", os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("link failed:\n" + out.stdout)
    return LIB


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, "\n".join(lines)))
        if lines:
            print("\n".join(lines), file=sys.stderr)


TB_SRC = os.path.join(HERE, "host", "tb", "modules_tb.cpp")
TB_BIN = os.path.join(HERE, "host", "tb", "modules_tb")


def build_harness():
    """Compile the C++ testbench-style harness of the host-side module mirror against the built library."""
    cmd = [HIPCC, "-std=c++17", "-O2", "-x", "c++", TB_SRC, "-o", TB_BIN, "-D__HIP_PLATFORM_AMD__",
           "-I/opt/rocm/include", "-L" + HERE, "-lflexllm_hip", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath," + HERE, "-Wl,-rpath,/opt/rocm/lib"]
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("harness build failed:\n" + out.stdout)
    return TB_BIN


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_harness())
