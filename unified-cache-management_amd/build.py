"""Builds libucm_hip.so (the C-ABI library) for gfx950 with hipcc.

    python build.py            # compile into ./lib/libucm_hip.so

hipcc cross-compiles without a GPU.  The library links only against the HIP runtime; when it
is loaded into a process that already imported torch, the runtime torch loaded is reused.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = ["common.hip", "hamming_topk.hip", "hash_encode.hip", "trans.hip", "cache_store.hip", "dot_topk.hip", "kvstar_topk.hip",
       "posix_store.hip"]
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libucm_hip.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-FP32 VALU forms are kept out of generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def build(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "csrc")]
    cmd += [os.path.join(HERE, "csrc", s) for s in SRC] + ["-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out:
        print(out)
    return LIB


if __name__ == "__main__":
    print(build())
    sys.exit(0)
