"""Record of measured HBM traffic per kernel launch, kept beside the rocprofv3 summaries it comes from.

`bench.py` reports `roofline.traffic` from `profiles/hbm_traffic.json`, never from a literal: every entry carries
a digest of the kernel sources it was measured on, and an entry whose digest differs from the sources in the tree
is reported as stale (traffic null) instead of being passed on.

Refreshing an entry (on a GPU box; four counter passes, one counter each, each a run of its own):

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d OUT/fwd_fetch -o p -- python3 bench.py --workload W --traffic-probe fwd
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d OUT/fwd_write -o p -- python3 bench.py --workload W --traffic-probe fwd
    (the same two with --traffic-probe bwd)
    python3 bench_profiling.py traffic --workload W --dir OUT

`bench.py --traffic-probe` launches the pass twice and then a plain 64 MiB device-to-device copy whose traffic is
known; the counters of the pass are scaled by what they read for that copy.

Time by stage (`python bench_profiling.py stages --workload W`): the passes are timed on the default library and on
measurement builds with the angular part, the radial part or both compiled out, with the forward kernels' stores of
the feature rows compiled out, and with the backward kernels reading every upstream row from one cached row
(`python -m khan_amd.build --stage-variants`, built beforehand); differences of those times are the stages.

`--traffic-probe networks` (on an AEV workload, whose feature rows it takes) and `--traffic-probe charges` (on a
charges workload) do the same for khan_atomic_networks_f32 and khan_ani_charge_all; `python3 bench_profiling.py
traffic --workload W --dir OUT --passes networks` reads OUT/networks_fetch and OUT/networks_write.
"""
import csv
import glob
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
RECORD = os.path.join(ROOT, "profiles", "hbm_traffic.json")
COPY_BYTES = 64 * 1024 * 1024

# the kernel that dominates each pass of each bench workload (substring of the name rocprofv3 prints)
DOMINANT = {
    ("organic65536", "fwd"): "aev_fwd_small_kernel<float, false, false>",
    ("organic65536", "bwd"): "aev_bwd_small_kernel<float>",
    ("organic16384", "fwd"): "aev_fwd_small_kernel<float, false, false>",
    ("organic16384", "bwd"): "aev_bwd_small_kernel<float>",
    ("organic1024", "fwd"): "aev_fwd_small_kernel<float, false, false>",
    ("organic1024", "bwd"): "aev_bwd_small_kernel<float>",
    ("organic16384_f64", "fwd"): "aev_fwd_small_kernel<double, false, false>",
    ("organic16384_f64", "bwd"): "aev_bwd_small_kernel<double>",
    ("boxes4096", "fwd"): "aev_fwd_medium_kernel<float, false, false>",
    ("boxes4096", "bwd"): "aev_bwd_medium_kernel<float, false, false>",
    ("organic65536", "networks"): "networks_fused_kernel<true, true>",
    ("organic65536", "jvp"): "aev_fwd_small_kernel<float, true, false>",
    ("charges_boxes4096_f64", "charges"): "charge_tile_kernel<double",
}
# the sources an entry's digest covers, by pass
_DIGEST_SOURCES = {"networks": ("dense_fused.hip", "khan_internal.h"), "charges": ("charges.hip", "khan_internal.h")}


def kernel_sources_digest(which="fwd"):
    """Digest of the code of the kernels the record is about (for the AEV passes csrc/aev_*.hip, csrc/aev_*.h and
    the two shared headers; for `networks` and `charges` their translation unit; comments left out) and of the
    build flags, 16 hex digits."""
    from khan_amd import build
    if which in _DIGEST_SOURCES:
        return build.sources_digest(list(_DIGEST_SOURCES[which]))
    names = [os.path.basename(n) for n in build.HIP_SOURCES + build.HIP_HEADERS]
    return build.sources_digest([n for n in names if n.startswith("aev_") or n in ("khan_internal.h", "khan_params.h")])


def load_records():
    if not os.path.exists(RECORD):
        return {}
    with open(RECORD) as f:
        return json.load(f)


def measured_traffic(workload, which):
    """-> (bytes per launch or None, stale flag, entry or None) for pass `which` ('fwd' / 'bwd') of a workload."""
    e = load_records().get("%s/%s" % (workload, which))
    if e is None:
        return None, False, None
    if e.get("sources_digest") != kernel_sources_digest(which):
        return None, True, e
    return e["bytes"], False, e


def _counter_rows(directory, counter):
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise RuntimeError("no counter_collection.csv under " + directory)
    rows = []
    for path in files:
        with open(path) as f:
            rows += [r for r in csv.DictReader(f) if r["Counter_Name"] == counter]
    return rows


def _last_value(rows, name_part):
    """Counter value of the LAST dispatch whose kernel name contains `name_part` (the warm launch)."""
    best = None
    for r in rows:
        if name_part in r["Kernel_Name"]:
            key = int(r["Dispatch_Id"])
            if best is None or key > best[0]:
                best = (key, float(r["Counter_Value"]))
    if best is None:
        raise RuntimeError("no dispatch of %r in the counter file" % name_part)
    return best[1]


def refresh(workload, directory, passes=("fwd", "bwd")):
    """Reads the counter passes under `directory` ({fwd,bwd}_{fetch,write}/, or those of `passes`) and rewrites the
    workload's entries of the record.  Returns the entries."""
    rec = load_records()
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        head = ""
    out = {}
    for which in passes:
        kernel = DOMINANT[(workload, which)]
        digest = kernel_sources_digest(which)
        vals = {}
        for counter, sub in (("FETCH_SIZE", "fetch"), ("WRITE_SIZE", "write")):
            rows = _counter_rows(os.path.join(directory, "%s_%s" % (which, sub)), counter)
            vals[sub] = _last_value(rows, kernel)
            vals["copy_" + sub] = _last_value(rows, "copyBuffer")
        # counters are KiB per dispatch; the copy moved COPY_BYTES each way
        fetch_scale = (COPY_BYTES / 1024.0) / vals["copy_fetch"]
        write_scale = (COPY_BYTES / 1024.0) / vals["copy_write"]
        fetch_b = vals["fetch"] * 1024.0 * fetch_scale
        write_b = vals["write"] * 1024.0 * write_scale
        e = {
            "kernel": kernel, "workload": workload, "pass": which,
            "fetch_kib": vals["fetch"], "write_kib": vals["write"],
            "copy_fetch_kib": vals["copy_fetch"], "copy_write_kib": vals["copy_write"],
            "fetch_scale": fetch_scale, "write_scale": write_scale,
            "fetch_bytes": fetch_b, "write_bytes": write_b, "bytes": fetch_b + write_b,
            "sources_digest": digest, "git_head": head,
        }
        rec["%s/%s" % (workload, which)] = e
        out[which] = e
    os.makedirs(os.path.dirname(RECORD), exist_ok=True)
    with open(RECORD, "w") as f:
        json.dump(rec, f, indent=1, sort_keys=True)
        f.write("\n")
    return out


BENCH_SHAPES = {"organic65536": ("organic", 65536), "organic16384": ("organic", 16384), "organic1024": ("organic", 1024),
                "boxes4096": ("boxes", 4096)}


def time_passes(workload, repeats=20):
    """Average time of the forward and of the backward pass (ms) of a bench workload on the library this process
    loaded, each pass launched with the batch's size order and size classes as bench.py does."""
    import torch
    from khan_amd import datagen, ops
    kind, n_mols = BENCH_SHAPES[workload[:-4] if workload.endswith("_f64") else workload]
    tdt = torch.float64 if workload.endswith("_f64") else torch.float32
    b = datagen.make_batch(kind, n_mols)
    dev = torch.device("cuda:0")
    X, Y, Z = (torch.from_numpy(v).to(dev).to(tdt) for v in (b.X, b.Y, b.Z))
    A = torch.from_numpy(b.A).to(dev)
    macs, mos = ops.mol_offsets(torch.from_numpy(b.mol_idxs).to(dev), b.n_mols)
    sc, ga, ac = ops.ani_sort(A)
    acs = ac.cpu()
    order = ops.size_order(macs)
    classes = order[-4:].cpu()
    up = torch.randn(b.n_atoms * 384, dtype=tdt, device=dev)
    g, s0 = [], 0
    for c in acs.tolist():
        g.append(up[s0 * 384:(s0 + c) * 384])
        s0 += c
    out = {}
    passes = (("fwd", lambda: ops.featurize(X, Y, Z, A, mos, macs, sc, acs, order=order, size_classes=classes)),
              ("bwd", lambda: ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *g, order=order, size_classes=classes)))
    for _ in range(30):            # the first milliseconds of a process run below the clock the rest runs at
        for name, fn in passes:
            fn()
    for name, fn in passes:
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(repeats):
            fn()
        e1.record()
        torch.cuda.synchronize()
        out[name] = e0.elapsed_time(e1) / repeats
    return out


def stage_times(workload):
    """Time of the passes with the angular part, the radial part or both compiled out (the measurement builds of
    khan_amd.build.build_stage_variants), each library in a process of its own.  Returns {build: {fwd, bwd}}."""
    from khan_amd import build
    res = {}
    for name, skip in (("full", 0), ("no angular part", 1), ("no radial part", 2), ("neither (skeleton)", 3),
                       ("forward stores nothing", 4), ("backward reads one cached upstream row", 8)):
        env = dict(os.environ)
        env.pop("KHAN_AEV_LIBRARY", None)
        if skip:
            lib = build.stage_variant_path(skip)
            if not os.path.exists(lib):
                raise RuntimeError(lib + " is missing: python -m khan_amd.build --stage-variants")
            env["KHAN_AEV_LIBRARY"] = lib
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench_profiling.py"), "time", "--workload", workload],
                           env=env, cwd=ROOT, capture_output=True, text=True, timeout=300)
        if r.returncode != 0:
            raise RuntimeError("timing %s failed: %s" % (name, r.stderr[-2000:]))
        res[name] = json.loads(r.stdout.strip().splitlines()[-1])
    return res


def print_stage_table(workload, res):
    full = res["full"]
    print("workload %s, kernel sources digest %s; ms per pass (HIP events, 20 launches after 30 warm-up passes)" % (workload, kernel_sources_digest()))
    print("| build | forward | backward |")
    print("|---|---|---|")
    for name, r in res.items():
        print("| %s | %.3f | %.3f |" % (name, r["fwd"], r["bwd"]))
    print("| => forward: feature-row stores not hidden under the arithmetic | %.3f (%.0f %%) | |" % (
        full["fwd"] - res["forward stores nothing"]["fwd"], 100 * (full["fwd"] - res["forward stores nothing"]["fwd"]) / full["fwd"]))
    b1 = res["backward reads one cached upstream row"]["bwd"]
    print("| => backward: upstream-row reads from HBM not hidden under the arithmetic | | %.3f (%.0f %%) |" % (
        full["bwd"] - b1, 100 * (full["bwd"] - b1) / full["bwd"]))
    print("| => angular part (full - no angular) | %.3f (%.0f %%) | %.3f (%.0f %%) |" % tuple(
        x for w in ("fwd", "bwd") for x in (full[w] - res["no angular part"][w], 100 * (full[w] - res["no angular part"][w]) / full[w])))
    print("| => radial part (full - no radial) | %.3f (%.0f %%) | %.3f (%.0f %%) |" % tuple(
        x for w in ("fwd", "bwd") for x in (full[w] - res["no radial part"][w], 100 * (full[w] - res["no radial part"][w]) / full[w])))
    print("| => skeleton (sort, scan, lists, staging, segment tables, stores) | %.3f (%.0f %%) | %.3f (%.0f %%) |" % tuple(
        x for w in ("fwd", "bwd") for x in (res["neither (skeleton)"][w], 100 * res["neither (skeleton)"][w] / full[w])))


def main(argv=None):
    import argparse
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    t = sub.add_parser("traffic", help="rewrite a workload's entries of profiles/hbm_traffic.json from counter runs")
    t.add_argument("--workload", required=True)
    t.add_argument("--dir", required=True, help="directory holding fwd_fetch/ fwd_write/ bwd_fetch/ bwd_write/")
    t.add_argument("--passes", nargs="+", default=["fwd", "bwd"], choices=("fwd", "bwd", "jvp", "networks", "charges"))
    sub.add_parser("digest", help="print the digest of the kernel sources in the tree")
    st = sub.add_parser("stages", help="time by stage of the AEV passes, from the measurement builds "
                                       "(python -m khan_amd.build --stage-variants)")
    st.add_argument("--workload", required=True, choices=sorted(BENCH_SHAPES) + [k + "_f64" for k in sorted(BENCH_SHAPES)])
    tm = sub.add_parser("time", help="time the two passes on the library this process loads; prints one JSON line")
    tm.add_argument("--workload", required=True)
    sub.add_parser("show", help="print the record and which entries are stale")
    args = ap.parse_args(argv)
    if args.cmd == "digest":
        print(kernel_sources_digest())
    elif args.cmd == "time":
        print(json.dumps(time_passes(args.workload)))
    elif args.cmd == "stages":
        print_stage_table(args.workload, stage_times(args.workload))
    elif args.cmd == "show":
        for k, e in sorted(load_records().items()):
            print("%-24s %-40s %8.1f MB  (fetch %.1f + write %.1f)  %s" % (
                k, e["kernel"], e["bytes"] / 1e6, e["fetch_bytes"] / 1e6, e["write_bytes"] / 1e6,
                "current" if e["sources_digest"] == kernel_sources_digest(e["pass"]) else "STALE (measured on %s)" % e["sources_digest"]))
    else:
        for which, e in refresh(args.workload, args.dir, tuple(args.passes)).items():
            print("%s/%s  %s: fetch %.1f MB + write %.1f MB = %.1f MB per launch" % (
                args.workload, which, e["kernel"], e["fetch_bytes"] / 1e6, e["write_bytes"] / 1e6, e["bytes"] / 1e6))


if __name__ == "__main__":
    main(sys.argv[1:])
