"""Builds the native pieces in-tree (no JIT cache):

  khan_amd/csrc/libkhan_aev.so      HIP kernels + C ABI, compiled for gfx950 with hipcc
  khan_amd/csrc/libkhan_datagen.so  host-only synthetic batch generator (gcc)
  khan_amd/csrc/libkhan_host.so     host-only batch assembly (gcc, OpenMP)

Run as ``python -m khan_amd.build`` or through ``__graft_entry__.build()``.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)

HIP_SOURCES = ["capi.hip", "aev_generic.hip", "aev_small.hip", "aev_small_bwd.hip", "aev_medium.hip", "aev_medium_bwd.hip", "sort_offsets.hip", "charges.hip"]
HIP_HEADERS = ["khan_internal.h", "khan_params.h", "aev_generic_center.h", "aev_small_common.h", "aev_fwd_batch.h", "aev_bwd_batch.h", os.path.join(ROOT, "include", "khan_aev.h")]

# packed-FP32 instruction selection is switched off on purpose (target feature -packed-fp32-ops)
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _run(cmd, cwd=None):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, cwd=cwd, check=True)


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libkhan_aev.so cannot be built")
    return exe


def build_hip(jobs=4):
    """Compile every HIP translation unit for gfx950 and link libkhan_aev.so."""
    hipcc = _hipcc()
    objs = []
    procs = []
    for src in HIP_SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append(subprocess.Popen(cmd))
        if len(procs) >= jobs:
            for p in procs:
                if p.wait() != 0:
                    raise RuntimeError("hipcc failed")
            procs = []
    for p in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed")
    out = os.path.join(CSRC, "libkhan_aev.so")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs)
    return out


def build_datagen():
    out = os.path.join(CSRC, "libkhan_datagen.so")
    _run(["gcc", "-std=gnu99", "-O2", "-fPIC", "-shared", "-o", out, os.path.join(CSRC, "datagen.c"), "-lm"])
    return out


def build_host():
    out = os.path.join(CSRC, "libkhan_host.so")
    _run(["gcc", "-std=gnu99", "-O2", "-fPIC", "-fopenmp", "-fvisibility=hidden", "-shared", "-o", out,
          os.path.join(CSRC, "host_batch.c")])
    return out


def build_all():
    return [build_hip(), build_datagen(), build_host()]


if __name__ == "__main__":
    build_all()
    sys.exit(0)
