"""Builds the native pieces in-tree (no JIT cache):

  khan_amd/csrc/libkhan_aev.so      HIP kernels + C ABI, compiled for gfx950 with hipcc
  khan_amd/csrc/libkhan_datagen.so  host-only synthetic batch generator (gcc)
  khan_amd/csrc/libkhan_host.so     host-only batch assembly (gcc, OpenMP)

plus csrc/check_build/libkhan_aev.so, the same library with the check switches compiled in (`build_check_variant`),
which only the tests of those switches load.

Run as ``python -m khan_amd.build`` or through ``__graft_entry__.build()``.
``python -m khan_amd.build --stage-variants`` builds the measurement libraries of `build_stage_variants`.

Every libkhan_aev.so gets a stamp beside it (``libkhan_aev.so.digest``): the digest of the sources and flags it was
built from, written after the generated code has passed `check_dpp_sources` and the link has succeeded.
`library_is_current()` compares it with the sources in the tree.
"""
import hashlib
import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)

HIP_SOURCES = ["capi.hip", "aev_generic.hip", "aev_small.hip", "aev_small_bwd.hip", "aev_medium.hip", "aev_medium_bwd.hip", "aev_large_sort.hip", "sort_offsets.hip", "charges.hip", "dense_first.hip", "dense_fused.hip", "mol_sum.hip"]
HIP_HEADERS = ["khan_internal.h", "khan_params.h", "aev_generic_center.h", "aev_small_common.h", "aev_fwd_batch.h", "aev_bwd_batch.h", "aev_large.h", os.path.join(ROOT, "include", "khan_aev.h")]

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


def _code_only(text):
    """Source text without comments and with runs of white space collapsed: what a digest is taken over, so that
    rewording a comment changes nothing."""
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    return " ".join(text.split())


def sources_digest(names=None, defines=()):
    """sha256 (16 hex digits) over the code of the HIP sources and headers (`names`: a subset of their file names;
    default all of them), the compiler flags and the defines."""
    h = hashlib.sha256()
    paths = [os.path.join(CSRC, n) for n in HIP_SOURCES] + [n if os.path.isabs(n) else os.path.join(CSRC, n) for n in HIP_HEADERS]
    for path in sorted(paths, key=os.path.basename):
        name = os.path.basename(path)
        if names is not None and name not in names:
            continue
        h.update(name.encode())
        with open(path, "r") as f:
            h.update(_code_only(f.read()).encode())
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(" ".join(sorted(defines)).encode())
    return h.hexdigest()[:16]


LIBRARY = os.path.join(CSRC, "libkhan_aev.so")


def stamp_path(library=LIBRARY):
    return library + ".digest"


def library_stamp(library=LIBRARY):
    """The digest written beside `library` when it was built, or None."""
    try:
        with open(stamp_path(library)) as f:
            return f.read().strip()
    except OSError:
        return None


def library_is_current(library=LIBRARY, defines=()):
    """True if `library` exists and was built from the sources, flags and defines in the tree."""
    return os.path.exists(library) and library_stamp(library) == sources_digest(defines=defines)


def build_hip(jobs=4, defines=(), out_dir=None, sources=None):
    """Compile the HIP translation units for gfx950 and link libkhan_aev.so (into `out_dir`, default csrc/).
    `sources`: the translation units to compile with `defines`; the others' objects are taken from csrc/ as the
    default build left them (for a variant whose defines touch only those files)."""
    hipcc = _hipcc()
    out_dir = out_dir or CSRC
    os.makedirs(out_dir, exist_ok=True)
    stamp = stamp_path(os.path.join(out_dir, "libkhan_aev.so"))
    if os.path.exists(stamp):
        os.remove(stamp)                 # no stamp while the library and the sources may disagree
    objs = []
    procs = []
    for src in HIP_SOURCES:
        shared = sources is not None and src not in sources
        default_obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        if shared and os.path.exists(default_obj) and os.path.getmtime(default_obj) >= os.path.getmtime(os.path.join(CSRC, src)):
            objs.append(default_obj)
            continue
        obj = os.path.join(out_dir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [hipcc] + HIPCC_FLAGS + ["-D" + d for d in (() if shared else defines)] + ["-c", os.path.join(CSRC, src), "-o", obj]
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
    # the generated code of the inline-asm users is checked before anything is linked: no library without it
    check_dpp_sources(defines)
    out = os.path.join(out_dir, "libkhan_aev.so")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs)
    with open(stamp, "w") as f:
        f.write(sources_digest(defines=defines) + "\n")
    return out


# The check switches (-DKHAN_CHECK_BUILD): environment variables, read once per process, that route every molecule
# through the general-shape kernels (KHAN_AEV_FORCE_GENERIC=1), withhold the large molecules' scratch
# (KHAN_AEV_LARGE_SCRATCH=0) or sum the forward kernel's angular records on the matrix cores (KHAN_AEV_PHASE2=matrix,
# a measured-and-dropped variant).  They are compiled into csrc/check_build/libkhan_aev.so only, which the tests of
# those paths name in KHAN_AEV_LIBRARY; the default library reads no such variable.
CHECK_DEFINES = ("KHAN_CHECK_BUILD=1",)
CHECK_SOURCES = ("capi.hip", "aev_small.hip")
CHECK_LIBRARY = os.path.join(CSRC, "check_build", "libkhan_aev.so")


def build_check_variant():
    """csrc/check_build/libkhan_aev.so: the default build's objects, with the translation units that hold the check
    switches compiled again with them.  Call after `build_hip()`."""
    return build_hip(defines=CHECK_DEFINES, out_dir=os.path.dirname(CHECK_LIBRARY), sources=CHECK_SOURCES)


STAGE_BUILDS = os.path.join(CSRC, "stage_builds")


def stage_variant_path(skip):
    return os.path.join(STAGE_BUILDS, "skip%d" % skip, "libkhan_aev.so")


STAGE_SKIPS = (1, 2, 3, 4, 8)
STAGE_SOURCES = ("aev_small.hip", "aev_small_bwd.hip", "aev_medium.hip", "aev_medium_bwd.hip")


def build_stage_variants():
    """Measurement builds of libkhan_aev.so with a stage of the AEV kernels compiled out (KHAN_PROFILE_SKIP = 1:
    no angular part, 2: no radial part, 3: neither, 4: the forward kernels store no feature rows, 8: the backward
    kernels read every upstream row from one cached row), for `python bench_profiling.py stages`.  Their results
    are wrong by design; they are loaded only when KHAN_AEV_LIBRARY names them.  Call after `build_hip()`."""
    return [build_hip(defines=("KHAN_PROFILE_SKIP=%d" % k,), out_dir=os.path.dirname(stage_variant_path(k)), sources=STAGE_SOURCES)
            for k in STAGE_SKIPS]


DPP_SOURCES = ["aev_small.hip", "aev_medium.hip"]     # translation units that use fma_quad (aev_small_common.h)


def check_dpp_operands(asm_text, name="<asm>"):
    """The multiply-add with a lane-exchange operand (v_fmac_f32_dpp, written as inline asm, which the compiler's
    hazard handling does not look into) reads its exchanged register early: two wait states have to lie between a
    vector instruction that writes that register and the multiply-add, and five between a vector instruction
    that writes EXEC (v_cmpx) and it.  Checks every use in the generated code, on the fall-through path and
    backwards through every branch to a label in between.  Every vector destination counts (register ranges,
    both operands of the swap instructions); `s_nop N` counts as N + 1 wait states, any other instruction as one.
    Raises on a violation (the remedy is an `s_nop` in front of the instruction)."""
    import re
    label_re = re.compile(r"^(\.LBB\d+_\d+):")
    code = []
    for i, raw in enumerate(asm_text.split("\n")):
        l = raw.split(";")[0].strip()            # drop comments (also the ';;#ASMSTART' markers)
        if not l or l.startswith("//"):
            continue
        if label_re.match(l) or not l.startswith("."):
            code.append((i, l))
    is_label = lambda l: label_re.match(l) is not None
    branches = {}
    for k, (_, l) in enumerate(code):
        m = re.match(r"^s_c?branch\S*\s+(\.LBB\d+_\d+)", l)
        if m:
            branches.setdefault(m.group(1), []).append(k)

    two_dest = ("v_swap_b32", "v_permlane32_swap", "v_permlane16_swap")

    def vgpr_dests(l):
        """VGPR numbers a vector-ALU instruction writes."""
        m = re.match(r"^(v_\S+)\s+(.*)$", l)
        if not m:
            return set()
        op, args = m.group(1), [a.strip() for a in m.group(2).split(",")]
        if op.startswith(("v_cmp", "v_readlane", "v_readfirstlane")):
            return set()
        out = set()
        for a in args[:2 if op.startswith(two_dest) else 1]:
            r = re.match(r"^v\[(\d+):(\d+)\]", a)
            if r:
                out.update(range(int(r.group(1)), int(r.group(2)) + 1))
            else:
                r = re.match(r"^v(\d+)\b", a)
                if r:
                    out.add(int(r.group(1)))
        return out

    def writes_exec(l):
        return l.startswith("v_cmpx") or re.match(r"^v_\S+\s+exec\b", l) is not None

    def wait_states(l):
        m = re.match(r"^s_nop\s+(\d+)", l)
        return int(m.group(1)) + 1 if m else 1

    def hazard_before(k, pred, budget, seen):
        """True if an instruction satisfying `pred` lies within `budget` wait states before position k on any path."""
        j = k - 1
        while budget > 0 and j >= 0:
            l = code[j][1]
            if is_label(l):
                lab = label_re.match(l).group(1)
                for b in branches.get(lab, []):
                    if (b, budget) not in seen:
                        seen.add((b, budget))
                        # the branch itself is an instruction on that path
                        if hazard_before(b, pred, budget - 1, seen):
                            return True
                j -= 1
                continue
            if re.match(r"^s_branch\b", l):
                return False                     # nothing falls through an unconditional branch
            if pred(l):
                return True
            budget -= wait_states(l)
            j -= 1
        return False

    uses = 0
    for k, (i, l) in enumerate(code):
        m = re.match(r"^v_fmac_f32_dpp\s+v\d+,\s*v(\d+),", l)
        if m:
            uses += 1
            reg = int(m.group(1))
            if hazard_before(k, lambda x: reg in vgpr_dests(x), 2, set()):
                raise RuntimeError("%s line %d: a vector instruction writes v%d within two wait states of its "
                                   "lane-exchange read" % (name, i + 1, reg))
            if hazard_before(k, writes_exec, 5, set()):
                raise RuntimeError("%s line %d: a vector instruction writes EXEC within five wait states of a "
                                   "lane-exchange multiply-add" % (name, i + 1))
    return uses


def check_dpp_sources(defines=()):
    """Compiles the translation units that use the lane-exchange multiply-add to assembly and checks them."""
    hipcc = _hipcc()
    total = 0
    procs = []
    for src in DPP_SOURCES:
        cmd = ([hipcc] + [f for f in HIPCC_FLAGS if f != "-Wall"] + ["-D" + d for d in defines] +
               ["-S", "--cuda-device-only", "-o", "-", os.path.join(CSRC, src)])
        print("+", " ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)))
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("hipcc -S failed on " + src)
        total += check_dpp_operands(out, src)
    if total == 0 and not defines:       # a measurement build may have compiled every use out
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
    return [build_hip(), build_check_variant(), build_datagen(), build_host()]


if __name__ == "__main__":
    if "--stage-variants" in sys.argv[1:]:
        build_stage_variants()
    else:
        build_all()
    sys.exit(0)
