"""Compiles liboxinfer_hip.so for gfx950 with hipcc, in-tree (oxinfer_amd/liboxinfer_hip.so)."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "liboxinfer_hip.so")
OBJ = os.path.join(HERE, "build")

SOURCES = ["act.hip", "dequant.hip", "decode.hip", "decode_mfma.hip", "decode_fp8.hip", "moe.hip", "moe_bf16.hip", "gemm.hip", "gemm_fp8.hip", "gemm_i8.hip", "backend.hip", "backend_moe.hip", "backend_gemm.hip", "graph_ops.hip", "backend_graph.hip", "backend_plan.hip"]

# -ffp-contract=off: multiply-adds fuse only where the source says fmaf (the bit-exact dequantizers
# need the reference's unfused operations). Packed-FP32 instructions are switched off.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
]

# Per-file extras. The prefill GEMMs keep 128 accumulator registers per wave; in the compiler's default form for a
# kernel with one wave per SIMD the matrix instructions take them from the accumulation registers and are never
# allocated in place (each accumulator moves to a new register at every instruction and is copied back around the
# loop: more copies than useful VALU work). With the VGPR form they accumulate in place.
EXTRA = {
    "gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_fp8.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def hipcc():
    for p in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if p and (os.path.sep not in p or os.path.exists(p)):
            return p
    raise RuntimeError("hipcc not found")


def build(verbose=False, tuning=False):
    """tuning=True compiles the developer overrides in (-DOXHIP_TUNING: environment variables that override tile shapes
    and orders, for measurement scripts); the library that ships is always built without them."""
    os.makedirs(OBJ, exist_ok=True)
    cc = hipcc()
    extra_all = (["-DOXHIP_TUNING"] + os.environ.get("OXHIP_EXP_FLAGS", "").split()) if tuning else []

    def one(src):
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        cmd = [cc, *FLAGS, *extra_all, *EXTRA.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        # the host pass does not know the device-only target feature; that warning is harmless
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(one, SOURCES))
    r = subprocess.run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return OUT


if __name__ == "__main__":
    print(build(verbose=True, tuning="--tuning" in sys.argv[1:]))
