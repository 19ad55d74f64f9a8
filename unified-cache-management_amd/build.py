"""Builds libucm_hip.so (the C-ABI library) for gfx950 with hipcc.

    python build.py            # compile into ./lib/libucm_hip.so
    python build.py --changed  # recompile only the sources newer than their objects

hipcc cross-compiles without a GPU.  Every source file is compiled to its own object (in
parallel), then linked.  The library links only against the HIP runtime; when it is loaded into
a process that already imported torch, the runtime torch loaded is reused.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = ["common.hip", "hamming_topk.hip", "hash_encode.hip", "trans.hip", "cache_store.hip", "dot_topk.hip", "kvstar_topk.hip",
       "posix_store.hip"]
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")
LIB = os.path.join(LIB_DIR, "libucm_hip.so")
TORCH_OPS_SRC = os.path.join(HERE, "csrc", "torch_ops.cpp")
TORCH_OPS_LIB = os.path.join(LIB_DIR, "libucm_torch_ops.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 VALU forms are kept out of generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out:
        print(out)


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src] + [os.path.join(HERE, "csrc", f) for f in os.listdir(os.path.join(HERE, "csrc"))
                    if f.endswith(".h")] + [os.path.join(ROOT, "include", "ucm_hip.h")]
    return any(os.path.getmtime(d) > t for d in deps)


def build(verbose=True, only_changed=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    base = [hipcc] + FLAGS + ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "csrc")]
    jobs = []
    objs = []
    for s in SRC:
        src = os.path.join(HERE, "csrc", s)
        obj = os.path.join(OBJ_DIR, s.replace(".hip", ".o"))
        objs.append(obj)
        if not only_changed or _stale(src, obj):
            jobs.append(base + ["-c", src, "-o", obj])
    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "8"))))
    with ThreadPoolExecutor(workers) as ex:
        list(ex.map(lambda c: _run(c, verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB], verbose)
    if not only_changed or _stale(TORCH_OPS_SRC, TORCH_OPS_LIB):
        build_torch_ops(verbose)
    return LIB


def build_torch_ops(verbose=True):
    """libucm_torch_ops.so: the TORCH_LIBRARY registration (torch.ops.ucm_amd.*) over the C ABI.  Host
    code only (g++), linked against libucm_hip.so and the installed PyTorch."""
    import torch
    from torch.utils import cpp_extension as ce

    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "csrc")]
    cmd += ["-I" + p for p in ce.include_paths()] + ["-I/opt/rocm/include", "-w"]
    cmd += [TORCH_OPS_SRC, "-o", TORCH_OPS_LIB, "-L" + LIB_DIR, "-lucm_hip", "-L" + tlib, "-ltorch", "-ltorch_cpu",
            "-lc10", "-lc10_hip", "-ltorch_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    _run(cmd, verbose)
    return TORCH_OPS_LIB


if __name__ == "__main__":
    print(build(only_changed="--changed" in sys.argv))
    sys.exit(0)
