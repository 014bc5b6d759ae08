"""Builds libmctsnc_hip.so (search engine) and libpuct_hip.so (PUCT select/backup) for gfx950 with hipcc, in-tree,
next to this file."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmctsnc_hip.so")
PUCT_LIB = os.path.join(HERE, "libpuct_hip.so")
LIBRARIES = {LIB: ["mctsnc_engine.hip"], PUCT_LIB: ["puct_kernels.hip", "puct_gomoku.hip"]}
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
               # UCB values must be bit-reproducible: no fused multiply-add contraction anywhere
               "-ffp-contract=off",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               # the playout loops are a few hundred bytes run by a lone wavefront: where they start relative to the
               # instruction cache lines moved measured rates by 3 % between otherwise identical builds
               "-falign-loops=64",
               "-Wno-unknown-warning-option"]
# The PUCT kernels claim with one lane of a wavefront (`if (lane == 0) atomicAdd(...)`).  The compiler's pass that turns a
# wavefront's atomics on one address into one atomic of the sum does not see that a single lane is active, and wraps
# each claim in a lane count and a broadcast (a dozen instructions per claim in kernels bound by instruction issue;
# the node-level winner-recalc selection is 4-5 % faster without it).
EXTRA_FLAGS = {PUCT_LIB: ["-mllvm", "-amdgpu-atomic-optimizer-strategy=None"]}


def build_one(lib, sources, verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + EXTRA_FLAGS.get(lib, []) + ["-o", lib] + [os.path.join(CSRC, s) for s in sources]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return lib


def build(verbose=False, only=None):
    """Compiles every library (or the one whose path is `only`); returns the search engine's path."""
    for lib, sources in LIBRARIES.items():
        if only is None or only == lib:
            build_one(lib, sources, verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
