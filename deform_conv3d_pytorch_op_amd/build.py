"""Builds csrc/libdcn_amd.so with hipcc for gfx950 (in-tree, no JIT cache).

    python -m deform_conv3d_pytorch_op_amd.build
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
SO = os.path.join(CSRC, "libdcn_amd.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed fp32 math is switched off on purpose for this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # float/double atomic adds lower to global_atomic_add_f32/f64 instead of CAS loops
    "-munsafe-fp-atomics",
]


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", SO, os.path.join(CSRC, "dcn_amd.hip")]
    if verbose:
        print(" ".join(cmd))
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return SO


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
