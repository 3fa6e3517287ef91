"""Builds libredmetal_hip.so (gfx950) in-tree with hipcc. Run on the CPU-only build machine; the GPU box loads the
prebuilt library."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libredmetal_hip.so")
SOURCES = ["redhip_kernels.hip", "redhip_fused.hip", "redhip_prefill.hip", "redhip_pool_abi.hip", "redhip_moe_abi.hip", "redhip_gguf.hip", "redhip_profile.hip"]
# -packed-fp32-ops off: v_pk_*_f32 forms are not used on this pool of machines
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-shared", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wextra", "-Wno-unused-parameter"]


def build_library(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-o", LIB] + [os.path.join(CSRC, s) for s in SOURCES]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
