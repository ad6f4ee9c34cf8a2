"""Builds the measurement-only libraries that bench.py loads beside the product library (never by quamba_amd itself):

  libqa_bench_probes.so    register-only loops that give the rates the matrix cores and the vector ALUs sustain
  libquamba_amd_clk.so     the product library with the W8A8 GEMM kernel compiled with -DQA_GEMM_CLK: every workgroup
                           records the shader clock and the 100 MHz clock at the boundaries of its prologue, main loop
                           and epilogue (bench.py --gemm-phase-clocks)

Usage: python -m bench_probes.build [--force]     (after python -m quamba_amd.build: the second library links the
product's objects)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, ROOT)
from quamba_amd import build as qbuild  # noqa: E402

PROBES_SRC = os.path.join(HERE, "bench_probes.hip")
PROBES_LIB = os.path.join(HERE, "libqa_bench_probes.so")
CLK_LIB = os.path.join(HERE, "libquamba_amd_clk.so")
CLK_OBJ = os.path.join(HERE, "build", "gemm_w8a8_clk.o")


def _run(cmd, what):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {what}:\n{r.stdout}\n{r.stderr}")


def _deps():
    csrc = qbuild.CSRC
    return [os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith(".hpp")] + \
           [os.path.join(ROOT, "include", "quamba_amd.h")]


def build(force=False):
    os.makedirs(os.path.dirname(CLK_OBJ), exist_ok=True)
    newer = qbuild._newer
    if force or any(newer(d, PROBES_LIB) for d in [PROBES_SRC, *_deps()]):
        _run([qbuild.HIPCC, *qbuild.FLAGS, "-shared", PROBES_SRC, "-o", PROBES_LIB], "the bench probes")
    gemm_src = os.path.join(qbuild.CSRC, "gemm_w8a8.hip")
    if force or any(newer(d, CLK_OBJ) for d in [gemm_src, *_deps()]):
        _run([qbuild.HIPCC, *qbuild.FLAGS, "-DQA_GEMM_CLK", "-c", gemm_src, "-o", CLK_OBJ], "the clocked GEMM")
    others = [os.path.join(qbuild.BUILD, s[:-4] + ".o") for s in qbuild.sources() if s != "gemm_w8a8.hip"]
    if force or any(newer(o, CLK_LIB) for o in [CLK_OBJ, *others]):
        _run([qbuild.HIPCC, "-shared", "-fPIC", f"--offload-arch={qbuild.ARCH}", CLK_OBJ, *others, "-o", CLK_LIB],
             "libquamba_amd_clk.so")
    return PROBES_LIB, CLK_LIB


if __name__ == "__main__":
    print(*build(force="--force" in sys.argv))
