"""Build recipe for the HIP extension: one hipcc call, gfx950 only, output in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRCS = [os.path.join(HERE, "csrc", f) for f in ("ltr_attn.hip", "ltr_rope.hip", "ltr_probe.hip")]
LIB = os.path.join(HERE, "csrc", "libltr_attn.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-shared", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",       # MFMA results in VGPRs: no accvgpr copies around the softmax
    "-I", os.path.join(ROOT, "include"),
]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", LIB] + SRCS
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed building %s" % " ".join(SRCS))
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
