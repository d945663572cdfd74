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


DPP_SOURCES = ["aev_small.hip", "aev_medium.hip"]     # translation units that use fma_quad (aev_small_common.h)


def check_dpp_operands(asm_text, name="<asm>"):
    """The multiply-add with a lane-exchange operand (written as inline asm, which the compiler's hazard
    handling does not look into) needs two wait states between a vector instruction that writes the exchanged
    register and itself.  Checks every use in the generated code: none of the two instructions before it -- on
    the fall-through path and before every branch to a label in between -- may be a vector instruction that
    writes that register.  Raises on a violation (the remedy is an `s_nop 1` in front of the instruction)."""
    import re
    lines = [l.strip() for l in asm_text.split("\n")]
    code = [(i, l) for i, l in enumerate(lines) if l and not l.startswith((";", ".", "//")) or re.match(r"^\.LBB\d+_\d+:", l or "")]
    is_label = lambda l: re.match(r"^\.LBB\d+_\d+:", l) is not None
    branches = {}
    for k, (_, l) in enumerate(code):
        m = re.match(r"^s_c?branch\S*\s+(\.LBB\d+_\d+)", l)
        if m:
            branches.setdefault(m.group(1) + ":", []).append(k)

    def writes(l, reg):
        m = re.match(r"^(v_\S+)\s+([^,\s]+)", l)
        if not m or m.group(1).startswith(("v_cmp", "v_readlane", "v_readfirstlane")):
            return False
        dst = m.group(2)
        r = re.match(r"^v\[(\d+):(\d+)\]$", dst)
        n = int(reg[1:])
        if r:
            return int(r.group(1)) <= n <= int(r.group(2))
        return dst == reg

    def hazard_before(k, reg, budget):
        """True if a vector write of `reg` lies within `budget` instructions before position k on any path."""
        j = k - 1
        while budget > 0 and j >= 0:
            l = code[j][1]
            if is_label(l):
                for b in branches.get(l.split()[0], []):
                    if hazard_before(b, reg, budget):
                        return True
                j -= 1
                continue
            if writes(l, reg):
                return True
            budget -= 1
            j -= 1
        return False

    uses = 0
    for k, (i, l) in enumerate(code):
        m = re.match(r"^v_fmac_f32_dpp\s+v\d+,\s*(v\d+),", l)
        if m:
            uses += 1
            if hazard_before(k, m.group(1), 2):
                raise RuntimeError("%s line %d: a vector instruction writes %s within two instructions of its "
                                   "lane-exchange read" % (name, i + 1, m.group(1)))
    return uses


def check_dpp_sources():
    """Compiles the translation units that use the lane-exchange multiply-add to assembly and checks them."""
    hipcc = _hipcc()
    total = 0
    for src in DPP_SOURCES:
        cmd = [hipcc] + [f for f in HIPCC_FLAGS if f != "-Wall"] + ["-S", "--cuda-device-only", "-o", "-", os.path.join(CSRC, src)]
        print("+", " ".join(cmd), flush=True)
        out = subprocess.run(cmd, check=True, capture_output=True, text=True).stdout
        total += check_dpp_operands(out, src)
    if total == 0:
        raise RuntimeError("no lane-exchange multiply-add found in %s: the check looks at the wrong files" % DPP_SOURCES)
    print("lane-exchange operands: %d uses checked" % total, flush=True)
    return total


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
    outs = [build_hip(), build_datagen(), build_host()]
    check_dpp_sources()
    return outs


if __name__ == "__main__":
    build_all()
    sys.exit(0)
