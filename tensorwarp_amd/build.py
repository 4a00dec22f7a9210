"""Builds libtwmarlin_hip.so (gfx950 code objects + C ABI) in-tree with hipcc."""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtwmarlin_hip.so")
SOURCES = ["twm_kernels.hip", "twm_decode.hip", "twm_gemv4.hip", "twm_prefill.hip", "twm_api.hip"]
# -packed-fp32-ops off: v_pk_{add,mul,fma}_f32 are not to be generated on this hardware pool.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def build(verbose=False):
    """Compile every HIP source for gfx950 and link the shared library. Always recompiles."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    tmp = LIB + ".tmp"
    cmd = [hipcc] + FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", tmp]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    os.replace(tmp, LIB)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
