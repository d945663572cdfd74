"""Record of measured HBM traffic per kernel launch, kept beside the rocprofv3 summaries it comes from.

`bench.py` reports `roofline.traffic` from `profiles/hbm_traffic.json`, never from a literal: every entry carries
a digest of the kernel sources it was measured on, and an entry whose digest differs from the sources in the tree
is reported as stale (traffic null) instead of being passed on.

Refreshing an entry (on a GPU box; four counter passes, one counter each, each a run of its own):

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d OUT/fwd_fetch -o p -- python3 bench.py --workload W --traffic-probe fwd
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d OUT/fwd_write -o p -- python3 bench.py --workload W --traffic-probe fwd
    (the same two with --traffic-probe bwd)
    python3 -m khan_amd.profiling traffic --workload W --dir OUT

`bench.py --traffic-probe` launches the pass twice and then a plain 64 MiB device-to-device copy whose traffic is
known; the counters of the pass are scaled by what they read for that copy.
"""
import csv
import glob
import hashlib
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
RECORD = os.path.join(ROOT, "profiles", "hbm_traffic.json")
COPY_BYTES = 64 * 1024 * 1024

# the kernel that dominates each pass of each bench workload (substring of the name rocprofv3 prints)
DOMINANT = {
    ("organic65536", "fwd"): "aev_fwd_small_kernel<float, false>",
    ("organic65536", "bwd"): "aev_bwd_small_kernel<float>",
    ("organic16384", "fwd"): "aev_fwd_small_kernel<float, false>",
    ("organic16384", "bwd"): "aev_bwd_small_kernel<float>",
    ("organic1024", "fwd"): "aev_fwd_small_kernel<float, false>",
    ("organic1024", "bwd"): "aev_bwd_small_kernel<float>",
    ("organic16384_f64", "fwd"): "aev_fwd_small_kernel<double, false>",
    ("organic16384_f64", "bwd"): "aev_bwd_small_kernel<double>",
    ("boxes4096", "fwd"): "aev_fwd_medium_kernel<float, false>",
    ("boxes4096", "bwd"): "aev_bwd_medium_kernel<float>",
}


def kernel_sources_digest():
    """sha256 over the kernel sources (csrc/*.hip, csrc/*.h, the build flags), 16 hex digits."""
    from . import build
    h = hashlib.sha256()
    csrc = os.path.join(HERE, "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(build.HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


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
    if e.get("sources_digest") != kernel_sources_digest():
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


def refresh(workload, directory):
    """Reads the four counter passes under `directory` ({fwd,bwd}_{fetch,write}/) and rewrites the workload's
    two entries of the record.  Returns the entries."""
    rec = load_records()
    digest = kernel_sources_digest()
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        head = ""
    out = {}
    for which in ("fwd", "bwd"):
        kernel = DOMINANT[(workload, which)]
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


def main(argv=None):
    import argparse
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    t = sub.add_parser("traffic", help="rewrite a workload's entries of profiles/hbm_traffic.json from counter runs")
    t.add_argument("--workload", required=True)
    t.add_argument("--dir", required=True, help="directory holding fwd_fetch/ fwd_write/ bwd_fetch/ bwd_write/")
    sub.add_parser("digest", help="print the digest of the kernel sources in the tree")
    sub.add_parser("show", help="print the record and which entries are stale")
    args = ap.parse_args(argv)
    if args.cmd == "digest":
        print(kernel_sources_digest())
    elif args.cmd == "show":
        d = kernel_sources_digest()
        for k, e in sorted(load_records().items()):
            print("%-24s %-40s %8.1f MB  (fetch %.1f + write %.1f)  %s" % (
                k, e["kernel"], e["bytes"] / 1e6, e["fetch_bytes"] / 1e6, e["write_bytes"] / 1e6,
                "current" if e["sources_digest"] == d else "STALE (measured on %s)" % e["sources_digest"]))
    else:
        for which, e in refresh(args.workload, args.dir).items():
            print("%s/%s  %s: fetch %.1f MB + write %.1f MB = %.1f MB per launch" % (
                args.workload, which, e["kernel"], e["fetch_bytes"] / 1e6, e["write_bytes"] / 1e6, e["bytes"] / 1e6))


if __name__ == "__main__":
    main(sys.argv[1:])
