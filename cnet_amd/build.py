"""Builds cnet_amd/lib/libcnet_hip.so (the C-ABI device library) for gfx950 with hipcc.

    python -m cnet_amd.build            # compile what changed, link
    python -m cnet_amd.build --force    # recompile everything

hipcc cross-compiles without a GPU.  Objects go to cnet_amd/build/, the library to cnet_amd/lib/ (in-tree, so
it travels with the source tree to the machine that runs it).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib", "libcnet_hip.so")
SOURCES = ["runtime.hip", "cgemm.hip", "cdft.hip", "elementwise.hip", "reduce.hip", "embedding.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
         # no fused multiply-add contraction: the elementwise kernels then round like the CPU path
         # (mul, then add), e.g. the SGD step is bit-identical to it; the GEMMs use MFMA either way
         "-ffp-contract=off",
         # packed-fp32 VALU forms are kept out of every kernel
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-DCNET_SCHED_RECIPE=" + os.environ.get("CNET_SCHED_RECIPE", "1"),
         "-Wno-unused-result", "-Wno-inline-asm", "-Wno-unused-value", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    newest = max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC) if f.endswith(".hpp"))
    newest = max(newest, os.path.getmtime(src), os.path.getmtime(os.path.join(ROOT, "include", "cnet_hip.h")))
    return os.path.getmtime(obj) < newest


def _compile(name, force):
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ, name.replace(".hip", ".o"))
    if not force and not _stale(src, obj):
        return obj
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (name, out))
    if out:
        print(out)
    return obj


def build(force=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 4)
    with ThreadPoolExecutor(jobs) as pool:
        objs = list(pool.map(lambda n: _compile(n, force), SOURCES))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc"] + objs + ["-o", LIB]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("link failed:\n" + res.stdout)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
