"""Compiles the HIP sources under csrc/ into librlt_rocm.so for gfx950 (cross-compiles without a GPU).

Each source becomes an object file under build/ (compiled in parallel), then one link. `build(force=True)` recompiles everything;
without it only the objects older than their source or any header are redone.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
OUT = os.path.join(HERE, "librlt_rocm.so")
SOURCES = ["device.hip", "tensor_ops.hip", "gemm.hip", "mlp.hip", "mlp_fused.hip", "mlp_small.hip", "mlp_rows.hip", "optim.hip", "sac.hip", "sac_fused.hip", "sac_update.hip", "sac_wide.hip", "runner.hip",
           "ppo.hip", "pad.hip", "gru.hip", "td3.hip", "normalize.hip", "envs.hip", "seq.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # keep the compiler from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def build(verbose=True, force=True, jobs=8):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ, exist_ok=True)
    headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    todo = []
    for s in sources:
        src, obj = os.path.join(CSRC, s), os.path.join(OBJ, s.replace(".hip", ".o"))
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), newest_header):
            todo.append([hipcc] + FLAGS + ["-c", src, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(run, todo))
    run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc"] + [os.path.join(OBJ, s.replace(".hip", ".o")) for s in sources] + ["-o", OUT])
    return OUT


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    sys.exit(0)
