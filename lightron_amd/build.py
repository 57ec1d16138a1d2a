"""Build recipe for the HIP libraries: one hipcc call each, gfx950 only, output in-tree.

libltr_attn.so   the product: the attention path behind include/ltr_attn.h.
libltr_probe.so  measurement helpers for bench.py (include/ltr_probe.h); nothing on the attention path uses it.
_ltr_node.so     host code only (g++, no device code): a C++ autograd node around ltr_attn_fwd / ltr_attn_bwd for the
                 single-chunk bf16 call, so that the backward of the most frequent call does not run through Python."""
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


NODE_SRC = os.path.join(HERE, "csrc", "ltr_autograd.cpp")
NODE_LIB = os.path.join(HERE, "_ltr_node.so")


def build_node(verbose: bool = False) -> str:
    """The C++ autograd node: plain g++ against the installed torch's headers and libraries and against libltr_attn.so
    (found at run time beside this package through an $ORIGIN rpath)."""
    import sysconfig
    import pybind11
    import torch
    from torch.utils import cpp_extension as ce
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-shared", "-fPIC", "-std=c++17", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-DTORCH_EXTENSION_NAME=_ltr_node", "-DTORCH_API_INCLUDE_EXTENSION_H"]
    for inc in ce.include_paths() + [sysconfig.get_paths()["include"], pybind11.get_include(), os.path.join(ROOT, "include")]:
        cmd += ["-I", inc]
    cmd += [NODE_SRC, "-o", NODE_LIB]
    for lib in ce.library_paths():
        cmd += ["-L", lib]
    cmd += ["-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python", "-L", os.path.join(HERE, "csrc"), "-lltr_attn",
            "-Wl,-rpath,$ORIGIN/csrc"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("%s failed building %s" % (cxx, NODE_SRC))
    return NODE_LIB


def build(verbose: bool = False) -> str:
    """Compiles the two HIP libraries and the host-only autograd node; returns the path of the product library."""
    _hipcc(PROBE_LIB, PROBE_SRCS, verbose)
    lib = _hipcc(LIB, SRCS, verbose)
    build_node(verbose)
    return lib


if __name__ == "__main__":
    print(build(verbose=True))
