"""Build recipe for the HIP libraries: one hipcc call each, gfx950 only, output in-tree.

libltr_attn.so   the product: the attention path behind include/ltr_attn.h.
libltr_probe.so  measurement helpers for bench.py (include/ltr_probe.h); nothing on the attention path uses it."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRCS = [os.path.join(HERE, "csrc", f) for f in ("ltr_attn.hip", "ltr_rope.hip")]
LIB = os.path.join(HERE, "csrc", "libltr_attn.so")
PROBE_SRCS = [os.path.join(HERE, "csrc", "ltr_probe.hip")]
PROBE_LIB = os.path.join(HERE, "csrc", "libltr_probe.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-shared", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",       # MFMA results in VGPRs: no accvgpr copies around the softmax
    "-I", os.path.join(ROOT, "include"),
]


def _hipcc(out: str, srcs, verbose: bool) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", out] + list(srcs)
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed building %s" % " ".join(srcs))
    return out


def build(verbose: bool = False) -> str:
    """Compiles both libraries; returns the path of the product library."""
    _hipcc(PROBE_LIB, PROBE_SRCS, verbose)
    return _hipcc(LIB, SRCS, verbose)


if __name__ == "__main__":
    print(build(verbose=True))
