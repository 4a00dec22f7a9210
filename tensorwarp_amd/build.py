"""Builds libtwmarlin_hip.so (gfx950 code objects + C ABI) in-tree with hipcc."""
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtwmarlin_hip.so")
SOURCES = ["twm_kernels.hip", "twm_gemv4.hip", "twm_gemv4s.hip", "twm_moe.hip", "twm_stream.hip", "twm_batch.hip", "twm_prefill.hip", "twm_debug_mix.hip", "twm_noalloc.hip", "twm_api.hip",
           "twm_api_weights.hip", "twm_api_gemm.hip", "twm_api_moe.hip"]
# The batched-decode kernels read every MFMA result with vector instructions right away (scale, add):
# with the default choice the results land in AGPRs and each costs a v_accvgpr_read first.
# The decode kernels' first argument words (thirteen fit the user scalar registers) arrive preloaded (see k_gemv4s).
PRELOAD = ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
PER_FILE_FLAGS = {"twm_gemv4s.hip": PRELOAD, "twm_gemv4.hip": PRELOAD, "twm_moe.hip": PRELOAD, "twm_stream.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"] + PRELOAD,
                  "twm_batch.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"] + PRELOAD}
# -packed-fp32-ops off: v_pk_{add,mul,fma}_f32 are not to be generated on this hardware pool.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def build(verbose=False):
    """Compile every HIP source for gfx950 and link the shared library. Always recompiles."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    tmp = LIB + ".tmp"
    objdir = os.path.join(HERE, "_build")
    os.makedirs(objdir, exist_ok=True)

    def run(cmd):
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in res.stdout.splitlines() if "not a recognized feature" not in l)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
        return out

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        return obj, run([hipcc] + FLAGS + PER_FILE_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as pool:
        results = list(pool.map(compile_one, SOURCES))
    out = "\n".join(o for _, o in results if o.strip())
    out += run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc"] + [o for o, _ in results] + ["-o", tmp])
    os.replace(tmp, LIB)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
