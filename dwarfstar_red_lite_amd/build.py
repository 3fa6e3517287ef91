"""Builds libredmetal_hip.so (gfx950) in-tree with hipcc. Run on the CPU-only build machine; the GPU box loads the
prebuilt library. Every source is compiled to an object of its own (in parallel), then linked."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libredmetal_hip.so")
SOURCES = ["redhip_kernels.hip", "redhip_fused.hip", "redhip_prefill.hip", "redhip_pool_abi.hip", "redhip_moe_abi.hip",
           "redhip_gguf.hip", "redhip_profile.hip", "redhip_topk_abi.hip"]
# -packed-fp32-ops off: v_pk_*_f32 forms are not used on this pool of machines
# -amdgpu-kernarg-preload-count: the leading scalar / pointer arguments of a kernel (up to 14 dwords) are handed to every wave in
# registers at its start instead of being fetched from the argument block in memory; the latency-bound kernels name what their first
# requests need in leading arguments for this reason (one-token layer 16.4 -> 15.5 us)
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-mllvm", "-amdgpu-kernarg-preload-count=16",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wextra", "-Wno-unused-parameter"]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd[-3:]), out))
    return out


def _stale(obj, src, deps):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(d) > t for d in [src] + deps)


ABLATIONS = {"no_mfma": "REDHIP_ABLATE_NO_MFMA", "no_lds": "REDHIP_ABLATE_NO_LDS", "no_sign": "REDHIP_ABLATE_NO_SIGN"}


def build_library(verbose=False, incremental=False, timeline=False, ablate=()):
    """incremental: recompile only the sources that changed (or whose headers did) since their object was built.
    timeline: a second library, libredmetal_hip_timeline.so, whose expert kernels store phase stamps (-DREDHIP_TIMELINE; see
    redhip_timeline_read); load it by pointing REDHIP_LIBRARY at it. The ordinary library is not touched.
    ablate (with timeline): names from ABLATIONS; the slice kernels of libredmetal_hip_timeline_<names>.so leave that part of the decode
    out (matrix instructions, table reads, sign placement). Their results are wrong on purpose: for `timeline.py` only, which times
    phases and checks no values."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if ablate and not timeline:
        raise ValueError("--ablate builds are measurement builds: combine with --timeline")
    tag = "_timeline" + "".join("_" + a for a in ablate) if timeline else ""
    OBJ = os.path.join(HERE, "build" + tag)
    LIB = os.path.join(HERE, "libredmetal_hip%s.so" % tag)
    FLAGS = globals()["FLAGS"] + (["-DREDHIP_TIMELINE"] if timeline else []) + ["-D" + ABLATIONS[a] for a in ablate]
    FLAGS = FLAGS + os.environ.get("REDHIP_EXTRA_HIPCC_FLAGS", "").split()      # (for trying a compiler option without editing this file)
    os.makedirs(OBJ, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers += [os.path.join(HERE, "..", "include", f) for f in os.listdir(os.path.join(HERE, "..", "include")) if f.endswith(".h")]
    jobs = []
    for s in SOURCES:
        src, obj = os.path.join(CSRC, s), os.path.join(OBJ, s[:-4] + ".o")
        if not incremental or _stale(obj, src, headers):
            jobs.append([hipcc] + FLAGS + ["-c", "-o", obj, src])
    with ThreadPoolExecutor(max(1, min(8, len(jobs) or 1))) as ex:
        outs = list(ex.map(_run, jobs))
    outs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + [os.path.join(OBJ, s[:-4] + ".o") for s in SOURCES]))
    if verbose:
        text = "\n".join(o for o in outs if o.strip())
        if text:
            print(text)
    return LIB


if __name__ == "__main__":
    _ablate = tuple(sys.argv[i + 1] for i, a in enumerate(sys.argv[:-1]) if a == "--ablate")
    print(build_library(verbose=True, incremental="--incremental" in sys.argv, timeline="--timeline" in sys.argv, ablate=_ablate))
