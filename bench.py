#!/usr/bin/env python3
"""Benchmark of the ANI-1 featurization hot path on one MI355X.

One "step" = one pass of the hot path over one synthetic batch that is already resident in HBM:
    mol_offsets + ani_sort + size_order  ->  featurize (float32 forward)  ->  featurize_grad (float32 backward)
on the 65,536-molecule organic batch (the configuration the headline metric is quoted on).  The sort runs one
batch ahead of the passes that use it (its four atom counts have to reach the host first), as a feeder would
run it; every step still holds exactly one sort, one forward and one backward pass.
Prints ONE JSON line: atoms/s for forward+gradient, with the roofline position of the dominant
kernel and a CPU baseline (the reference's own CPU kernels compiled in place when available,
else this repo's CPU port) timed on a bounded sample of the same batch.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload organic65536|organic16384_f64|boxes4096|...]
"""
import argparse
import collections
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
FP32_PEAK_TFLOPS = 157.3       # MI355X vector FP32, published
FP64_PEAK_TFLOPS = 78.6

# roofline.traffic (HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) comes from the record
# profiles/hbm_traffic.json through bench_profiling: an entry measured on other kernel sources than the ones in
# the tree is reported as stale (traffic null), never passed on.

# name: (generator, molecules, float width in bytes, charges kernels in the step)
WORKLOADS = {
    "organic65536": ("organic", 65536, 4, False),        # the configuration the metric is quoted on
    "organic16384": ("organic", 16384, 4, False),
    "organic1024": ("organic", 1024, 4, False),
    "organic16384_f64": ("organic", 16384, 8, True),     # double precision forward + backward + ani_charge
    "boxes4096": ("boxes", 4096, 4, False),              # dense boxes of 64..256 atoms
    # not a line of the headline metric: boxes of 1,024..4,096 atoms (several workgroups per molecule, the atoms read
    # type-sorted from device memory)
    "bigboxes64": ("bigboxes", 64, 4, False),
    # not a line of the headline metric: energies and coordinate gradients through the atomic networks
    # (384-128-128-64-1 per type, random weights), the caller either side of the hot path
    "inference65536": ("organic", 65536, 4, False),
    # not a line of the headline metric either: featurize_grad_inverse (the Jacobian applied to per-atom vectors)
    "grad_inverse65536": ("organic", 65536, 4, False),
    "grad_inverse_boxes4096": ("boxes", 4096, 4, False),
    "grad_inverse_boxes4096_f64": ("boxes", 4096, 8, False),
    # nor these: the charge kernels alone (energy, then dE/dq and dE/dxyz), float64
    "charges_boxes4096_f64": ("boxes", 4096, 8, True),
    "charges_organic16384_f64": ("organic", 16384, 8, True),
}


def algorithmic_work(counts, n_atoms, n_mols, w):
    """Contract figures: minimal flops / compulsory HBM bytes per pass (D, P_R, P_A, T = pair and
    triple counts of the batch, w = bytes per float)."""
    D, PR, PA, T = counts["D"], counts["P_R"], counts["P_A"], counts["T"]
    return {
        "flops_fwd": 9 * D + 100 * PR + 5 * PA + 150 * T,
        "flops_bwd": 9 * D + 220 * PR + 8 * PA + 390 * T,
        "bytes_fwd": n_atoms * (384 * w + 3 * w + 8) + 8 * n_mols,
        "bytes_bwd": n_atoms * (384 * w + 3 * w + 8 + 3 * w) + 8 * n_mols,
        "bytes_sort": n_atoms * (4 + 8) + 8 * n_mols + 4 * n_atoms,
    }


def cpu_baseline(batch, sample_mols_fwd, sample_mols_bwd, w=4):
    """Forward+gradient on the host, single thread, bounded sample (rank 0, N=1 only)."""
    import numpy as np
    dtype = np.float32 if w == 4 else np.float64
    from oracle import binding as ob
    from khan_amd import datagen

    have_ref = ob.ref_lib(fast=True) is not None
    impl = "ref" if have_ref else "oracle"

    def sub(n_mols):
        b = datagen.make_batch(batch.kind, n_mols, seed=batch.seed)
        sc, ga, ac = ob.ani_sort(b.A)
        return b, sc, ac

    def fwd_job(b, sc, ac):
        ob.featurize(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, dtype=dtype, impl=impl, fast=True)

    def bwd_job(b, sc, ac):
        up = datagen.normal(b.n_atoms * 384).reshape(-1, 384)
        g = ob.scatter_rows(up, b.A, sc, ac)
        t0 = time.perf_counter()
        ob.featurize_grad(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, g, dtype=dtype, impl=impl, fast=True)
        return time.perf_counter() - t0

    b, sc, ac = sub(sample_mols_fwd)
    t0 = time.perf_counter()
    fwd_job(b, sc, ac)
    t_fwd = (time.perf_counter() - t0) / b.n_atoms
    b2, sc2, ac2 = sub(sample_mols_bwd)
    t_bwd = bwd_job(b2, sc2, ac2) / b2.n_atoms

    # the same kernels sharded by molecule over the host cores (one slice of molecules per thread; the
    # reference runs one CPU tower per core this way, gdb8.py:73-76)
    import concurrent.futures
    # a one-GPU box gives a job 16 host cores whatever os.cpu_count() shows there: at most that many threads
    host_cores = os.cpu_count() or 1
    threads = max(1, min(16, host_cores))

    def shards(n_mols):
        per = max(1, n_mols // threads)
        out = []
        for t in range(threads):
            bb = datagen.make_batch(batch.kind, per, seed=batch.seed, first_mol=t * per)
            s_, _, a_ = ob.ani_sort(bb.A)
            out.append((bb, s_, a_))
        return out

    with concurrent.futures.ThreadPoolExecutor(threads) as pool:
        sh = shards(sample_mols_fwd * threads // 2)
        t0 = time.perf_counter()
        list(pool.map(lambda a: fwd_job(*a), sh))
        tf_all = (time.perf_counter() - t0) / sum(x[0].n_atoms for x in sh)
        sh = shards(sample_mols_bwd * threads // 2)
        t0 = time.perf_counter()
        inner = list(pool.map(lambda a: bwd_job(*a), sh))
        wall = time.perf_counter() - t0
        # scatter of the upstream rows happens inside the jobs but outside their timers: charge the longest timer
        tb_all = max(inner) / sum(x[0].n_atoms for x in sh) if wall > 0 else 0.0
    return {
        "value": 1.0 / (t_fwd + t_bwd),
        "unit": "atoms/s",
        "cores": 1,
        "kind": "reference" if have_ref else "port",
        "sample": "forward on the first %d molecules (%d atoms), gradient on the first %d molecules (%d atoms) "
                  "of the same batch; per-atom times added; built -O3 -Ofast" % (
                      sample_mols_fwd, b.n_atoms, sample_mols_bwd, b2.n_atoms),
        "fwd_atoms_per_s": 1.0 / t_fwd,
        "bwd_atoms_per_s": 1.0 / t_bwd,
        "all_cores": {"value": 1.0 / (tf_all + tb_all), "unit": "atoms/s", "cores": threads,
                      "host_cpu_count": host_cores,
                      "sample": "the same kernels sharded by molecule, one slice per thread; %d threads = the job's "
                                "share of the host (os.cpu_count() reports %d); forward: wall time of the pool; "
                                "gradient: the slowest thread's timer (the scatter of its upstream rows is outside it)"
                                % (threads, host_cores)},
    }


def inference_bench(args, batch):
    """Energy + coordinate-gradient inference: featurize -> per-type networks -> segment sum, then back through the
    networks and featurize_grad; timed with every layer a library (rocBLAS) product and with the CELU layers in this
    package's matrix-core kernel.  One JSON line; the roofline object describes the step's
    dense layers, which dominate it (their flops against the fp32 matrix peak)."""
    import numpy as np
    import torch
    from khan_amd import model, ops
    from khan_amd.batching import DeviceBatch
    dev = torch.device("cuda:0")
    N, n_mols = batch.n_atoms, batch.n_mols
    xs, ys, zs = (torch.from_numpy(v).to(dev) for v in (batch.X, batch.Y, batch.Z))
    b = DeviceBatch.from_device_arrays(xs, ys, zs, torch.from_numpy(batch.A).to(dev),
                                       torch.from_numpy(batch.mol_idxs).to(dev), n_mols)
    def timed(first_layer_kernel, whole_network=True):
        m = model.AniModel(model.DEFAULT_LAYERS, model.celu, torch.float32, dev, seed=1, first_layer_kernel=first_layer_kernel)
        m.near.whole_network_kernel = whole_network
        for _ in range(args.warmup):
            m.batch_energies(b, need_grad=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            e, g = m.batch_energies(b, need_grad=True)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3, e, g

    ms_library, e_lib, g_lib = timed(False)      # every dense layer a library (rocBLAS) product
    ms_layers, e_l, g_l = timed(True, False)     # CELU layers, forward and backward, one launch per layer and direction
    ms_per_step, e_k, g_k = timed(True)          # the whole network and its gradient back to the rows in one launch
    agree = float((e_k - e_lib).abs().max() / e_lib.abs().max())
    agree_g = float((g_k - g_lib).abs().max() / g_lib.abs().max())
    sizes = (384,) + tuple(model.DEFAULT_LAYERS)
    macs_per_atom = sum(x * y for x, y in zip(sizes[:-1], sizes[1:]))
    gemm_flops = 2 * macs_per_atom * N * 2            # forward, and the data gradient on the way back
    import bench_profiling as profiling
    net_traffic, net_stale, _ = profiling.measured_traffic("organic%d" % n_mols, "networks")
    return ({
        "metric": "ANI-1 energy + coordinate-gradient inference atoms/sec, fp32, 1 MI355X",
        "value": N / (ms_per_step * 1e-3), "unit": "atoms/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "inference65536: featurize + 4 atomic networks 384-128-128-64-1 (random weights) + "
                               "segment sum, gradient back to the coordinates; %d molecules, %d atoms" % (n_mols, N)},
        "molecules_per_s": n_mols / (ms_per_step * 1e-3),
        "networks": {"one_launch_ms_per_step": ms_per_step, "layer_by_layer_kernels_ms_per_step": ms_layers,
                     "library_ms_per_step": ms_library, "max_relative_energy_difference_to_library": agree,
                     "max_relative_gradient_difference_to_library": agree_g,
                     # khan_atomic_networks_f32 with the gradient: feature rows read, gradient rows written
                     "algorithmic_bytes_per_launch": 2 * N * 384 * 4 + N * 4,
                     "hbm_bytes_per_launch": net_traffic, "hbm_bytes_stale": net_stale},
        "dense_products": "one launch: float32 operands split into two half-precision parts (value rounded, 2^11 x residual), "
                          "three partial products per pair on v_mfma_f32_32x32x16_f16, float32 accumulation; layer by layer: "
                          + ("three bfloat16 parts, six partial products on v_mfma_f32_32x32x16_bf16"
                             if os.environ.get("KHAN_DENSE_MATRIX") != "f32" else "v_mfma_f32_32x32x2_f32"),
        "roofline": {"kernel": "the atomic networks, forward and data gradient (khan_atomic_networks_f32): float32-equivalent "
                               "flops of the whole step against the float32 matrix peak",
                     "bound": "mfma", "achieved": gemm_flops / (ms_per_step * 1e-3) / 1e12,
                     "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": gemm_flops / (ms_per_step * 1e-3) / 1e12 / FP32_PEAK_TFLOPS,
                     "traffic": net_traffic, "traffic_stale": net_stale},      # of the networks' one launch
    })


def grad_inverse_bench(args, batch, w, kind):
    """featurize_grad_inverse on the batch: one JSON line; algorithmic bytes are the forward's plus the
    three incoming vectors."""
    import torch
    from khan_amd import ops
    dev = torch.device("cuda:0")
    N, n_mols = batch.n_atoms, batch.n_mols
    tdt, tname = (torch.float32, "float") if w == 4 else (torch.float64, "double")
    X, Y, Z = (torch.from_numpy(v).to(dev).to(tdt) for v in (batch.X, batch.Y, batch.Z))
    A = torch.from_numpy(batch.A).to(dev)
    macs, mos = ops.mol_offsets(torch.from_numpy(batch.mol_idxs).to(dev), n_mols)
    sc, ga, ac = ops.ani_sort(A)
    acs = ac.cpu()
    gen = torch.Generator(device=dev)
    gen.manual_seed(7)
    v = [torch.randn(N, device=dev, generator=gen, dtype=tdt) for _ in range(3)]
    for _ in range(args.warmup):
        ops.featurize_grad_inverse(X, Y, Z, A, mos, macs, sc, acs, *v)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        out = ops.featurize_grad_inverse(X, Y, Z, A, mos, macs, sc, acs, *v)
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    launch_ms = e0.elapsed_time(e1) / args.steps
    nbytes = N * (384 * w + 6 * w + 8) + 8 * n_mols
    kernel = "aev_fwd_%s_kernel<%s, true>" % ("small" if kind == "organic" else "medium", tname)
    import bench_profiling as profiling
    traffic, stale, _ = profiling.measured_traffic(args.workload.replace("grad_inverse", "organic") if kind == "organic" and w == 4 else args.workload, "jvp")
    return ({
        "metric": "AEV grad-inverse (Jacobian-vector product) atoms/sec, fp%d, 1 MI355X" % (8 * w),
        "value": N / (ms_per_step * 1e-3), "unit": "atoms/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f%d" % (8 * w),
        "data": "synthetic",
        "config": {"workload": "%s: featurize_grad_inverse, %d molecules, %d atoms" % (args.workload, n_mols, N)},
        "roofline": {"kernel": kernel, "bound": "hbm", "achieved": nbytes / (launch_ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / (launch_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": traffic, "traffic_stale": stale, "launch_ms": launch_ms, "algorithmic_bytes": nbytes},
    })


def charges_bench(args, batch, w):
    """ani_charge + ani_charge_grad_xyz (energy, dE/dq, dE/dxyz) on a resident batch: one JSON line.  Contract figures:
    20 C flops for the energy, 45 C for energy + both gradients (C = unordered pairs), N 8w + M (w + 8) bytes."""
    import torch
    from khan_amd import datagen, ops
    dev = torch.device("cuda:0")
    tdt = torch.float32 if w == 4 else torch.float64
    N, n_mols = batch.n_atoms, batch.n_mols
    X, Y, Z = (torch.from_numpy(v).to(dev).to(tdt) for v in (batch.X, batch.Y, batch.Z))
    Q = torch.from_numpy(datagen.charges(N)).to(dev).to(tdt)
    macs, mos = ops.mol_offsets(torch.from_numpy(batch.mol_idxs).to(dev), n_mols)
    ones = torch.ones(n_mols, dtype=tdt, device=dev)
    C = batch.work_counts()["C"]
    for _ in range(args.warmup):
        ops.ani_charge(X, Y, Z, Q, mos, macs)
        ops.ani_charge_grad_xyz(X, Y, Z, Q, mos, macs, ones)
        ops.ani_charge_all(X, Y, Z, Q, mos, macs, ones)
    torch.cuda.synchronize()
    # the reference's two ops, one after the other (each a pass over the pairs) ...
    marks = []
    for _ in range(args.steps):
        m = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        m[0].record()
        e = ops.ani_charge(X, Y, Z, Q, mos, macs)
        m[1].record()
        g = ops.ani_charge_grad_xyz(X, Y, Z, Q, mos, macs, ones)
        m[2].record()
        marks.append(m)
    torch.cuda.synchronize()
    t_e = sum(m[0].elapsed_time(m[1]) for m in marks) / args.steps
    t_g = sum(m[1].elapsed_time(m[2]) for m in marks) / args.steps
    # ... and the step: energy and both gradients from one pass (khan_ani_charge_all)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        out = ops.ani_charge_all(X, Y, Z, Q, mos, macs, ones)
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    t_all = e0.elapsed_time(e1) / args.steps
    nbytes = N * 8 * w + n_mols * (w + 8)
    peak = FP32_PEAK_TFLOPS if w == 4 else FP64_PEAK_TFLOPS
    tflops = 45.0 * C / (t_all * 1e-3) / 1e12
    import bench_profiling as profiling
    traffic, stale, _ = profiling.measured_traffic(args.workload, "charges")
    return ({
        "metric": "ani_charge energy + gradients atoms/sec, fp%d, 1 MI355X" % (8 * w),
        "value": N / (ms_per_step * 1e-3), "unit": "atoms/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if w == 4 else "f64", "data": "synthetic",
        "config": {"workload": "%s: charge energy, dE/dq and dE/dxyz in one pass (khan_ani_charge_all), %d molecules, %d atoms, %d pairs" % (
            args.workload, n_mols, N, C)},
        "molecules_per_s": n_mols / (ms_per_step * 1e-3),
        # all pairs of a molecule from a few bytes per atom: the vector ALUs bound these kernels, not HBM
        "roofline": {"kernel": "charge kernels", "bound": "valu", "achieved": tflops, "peak": peak, "unit": "TFLOP/s",
                     "frac": tflops / peak, "traffic": traffic, "traffic_stale": stale, "launch_ms": t_all,
                     "energy_ms": t_e, "gradients_ms": t_g,       # ani_charge and ani_charge_grad_xyz as separate calls
                     "algorithmic_flops": 45.0 * C, "algorithmic_bytes": nbytes,
                     "hbm_frac": nbytes / (t_all * 1e-3) / 1e9 / HBM_PEAK_GBS},
    })


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="organic65536", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="with the default workload: leave out the shorter runs of the other configurations "
                         "(`configs` in the printed line)")
    ap.add_argument("--traffic-probe", choices=("fwd", "bwd", "jvp", "networks", "charges"), default=None,
                    help="counter-collection mode: launch that pass twice (fwd, bwd: the AEV passes; jvp: featurize_grad_inverse; networks: "
                         "khan_atomic_networks_f32 with its gradient on the workload's feature rows; charges: "
                         "khan_ani_charge_all), then a plain 64 MiB device copy of known traffic (scales FETCH_SIZE / "
                         "WRITE_SIZE), print nothing else and exit")
    ap.add_argument("--reproducible-gradients", action="store_true",
                    help="time (or probe) the backward pass with khan_set_reproducible_gradients(1): forces of molecules "
                         "of 33-256 atoms summed in a fixed order in LDS instead of by atomics")
    ap.add_argument("--phase2", choices=("vector", "matrix"), default="vector",
                    help="matrix: measure the variant of the small-molecule forward kernel that sums the angular "
                         "records on the matrix cores (loads the check build of the library, which alone holds it, "
                         "and sets KHAN_AEV_PHASE2 before its first launch)")
    args = ap.parse_args()
    if args.phase2 == "matrix":
        from khan_amd import build as _build
        os.environ["KHAN_AEV_LIBRARY"] = _build.CHECK_LIBRARY
        os.environ["KHAN_AEV_PHASE2"] = "matrix"
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; the path shards by molecule with no exchange, "
                 "but no multi-GPU launch is part of this run (got --gpus %d)" % args.gpus)

    import torch
    from khan_amd import datagen, _lib

    _lib.load()   # fails loudly if the HIP library is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    if args.reproducible_gradients:
        from khan_amd import ops as _ops
        _ops.set_reproducible_gradients(True)
    result = run_workload(args, args.workload, args.steps, args.warmup, cpu=not args.no_cpu_baseline)
    if result is None:
        return
    if args.workload == HEADLINE and not args.headline_only:
        # the other configurations, each a shorter run of its own step, summarised in the same line
        steps, warmup = max(10, args.steps // 3), max(5, args.warmup // 2)
        result["configs"] = {}
        for name in EXTRA_CONFIGS:
            torch.cuda.empty_cache()
            result["configs"][name] = summary(run_workload(args, name, steps, warmup, cpu=False), steps, warmup)
    print(json.dumps(result))


HEADLINE = "organic65536"
# the float64 + charges, dense-box and grad-inverse configurations, reported beside the headline configuration
EXTRA_CONFIGS = ("organic16384_f64", "boxes4096", "grad_inverse65536", "charges_boxes4096_f64")


def summary(r, steps, warmup):
    """The figures of one extra configuration that go into the headline line."""
    rf = r["roofline"]
    out = {"ms_per_step": r["ms_per_step"], "atoms_per_s": r["value"], "dtype": r["dtype"], "steps": steps, "warmup": warmup,
           "workload": r["config"]["workload"]}
    if "fwd" in rf:
        out.update({"fwd_ms": rf["fwd"]["ms"], "bwd_ms": rf["bwd"]["ms"],
                    "hbm_frac": {"fwd": rf["fwd"]["hbm_frac"], "bwd": rf["bwd"]["hbm_frac"]},
                    "valu_frac": {"fwd": rf["fwd"]["valu_frac"], "bwd": rf["bwd"]["valu_frac"]}})
        if "charges" in rf:
            out["charges"] = rf["charges"]
    elif rf["bound"] == "valu":
        out.update({"launch_ms": rf["launch_ms"], "energy_ms": rf["energy_ms"], "gradients_ms": rf["gradients_ms"],
                    "valu_frac": rf["frac"], "hbm_frac": rf["hbm_frac"]})
    else:
        out.update({"launch_ms": rf["launch_ms"], "hbm_frac": rf["frac"]})
    return out


def run_workload(args, workload, steps, warmup, cpu):
    """Times one workload; -> its result (the JSON object a run of that workload alone prints), or None in the
    counter-collection mode."""
    import numpy as np
    import torch
    from khan_amd import datagen, ops

    args = argparse.Namespace(**dict(vars(args), workload=workload, steps=steps, warmup=warmup, no_cpu_baseline=not cpu))
    dev = torch.device("cuda:0")
    kind, n_mols, w, with_charges = WORKLOADS[args.workload]
    tdt = torch.float32 if w == 4 else torch.float64
    batch = datagen.make_batch(kind, n_mols)
    if args.workload.startswith("inference"):
        return inference_bench(args, batch)
    if args.workload.startswith("grad_inverse"):
        return grad_inverse_bench(args, batch, w, kind)
    if args.workload.startswith("charges_") and not args.traffic_probe:
        return charges_bench(args, batch, w)
    N = batch.n_atoms
    counts = batch.work_counts()
    work = algorithmic_work(counts, N, n_mols, w)

    X, Y, Z = (torch.from_numpy(v).to(dev).to(tdt) for v in (batch.X, batch.Y, batch.Z))
    A = torch.from_numpy(batch.A).to(dev)
    mol_idxs = torch.from_numpy(batch.mol_idxs).to(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    upstream = torch.randn(N * 384, dtype=tdt, device=dev, generator=gen)   # dL/dAEV ~ N(0,1)
    Q = torch.from_numpy(datagen.charges(N)).to(dev).to(tdt) if with_charges else None
    ones_m = torch.ones(n_mols, dtype=tdt, device=dev) if with_charges else None
    torch.cuda.synchronize()

    if args.traffic_probe:
        macs, mos = ops.mol_offsets(mol_idxs, n_mols)
        sc, ga, ac = ops.ani_sort(A)
        acs = ac.cpu()
        grads, start = [], 0
        for c in acs.tolist():
            grads.append(upstream[start * 384:(start + c) * 384])
            start += c
        if args.traffic_probe == "networks":
            from khan_amd import model
            net = model.AniModel(model.DEFAULT_LAYERS, model.celu, torch.float32, dev, seed=1).near
            feats = ops.featurize(X, Y, Z, A, mos, macs, sc, acs)
            packed, biases, head_w, head_b = net.one_launch_operands()
        if args.traffic_probe == "charges":
            Qp = torch.from_numpy(datagen.charges(N)).to(dev).to(tdt)
            ones_p = torch.ones(n_mols, dtype=tdt, device=dev)
        for _ in range(2):
            if args.traffic_probe == "fwd":
                ops.featurize(X, Y, Z, A, mos, macs, sc, acs)
            elif args.traffic_probe == "bwd":
                ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *grads)
            elif args.traffic_probe == "jvp":
                ops.featurize_grad_inverse(X, Y, Z, A, mos, macs, sc, acs, *(upstream[k * N:(k + 1) * N] for k in range(3)))
            elif args.traffic_probe == "networks":
                ops.atomic_networks(feats, None, biases, head_w, head_b, want_grad=True, packed=packed)
            else:
                ops.ani_charge_all(X, Y, Z, Qp, mos, macs, ones_p)
        src = torch.empty(64 * 1024 * 1024 // 4, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        print("traffic probe: %s x2 on %s, then a 64 MiB device copy" % (args.traffic_probe, args.workload))
        return

    ev = {k: [] for k in ("sort", "fwd", "bwd", "charges")}

    def sort_alone_ms(reps=20):
        """mol_offsets + ani_sort + size_order (nine launches) on an otherwise idle GPU, per batch."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for k in range(3 + reps):
            if k == 3:
                torch.cuda.synchronize()
                e0.record()
            macs_, _ = ops.mol_offsets(mol_idxs, n_mols)
            ops.ani_sort(A)
            ops.size_order(macs_)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    sort_ms_alone = sort_alone_ms()

    # atom_counts is a host-memory input of featurize (the reference's op reads it on the host), so every batch
    # needs one 16-byte device-to-host copy between its sort and its forward pass.  As the reference's staging
    # queue does, the feeder side runs one batch ahead: a step enqueues the sort of the NEXT batch (same synthetic
    # data) and the asynchronous copy of its counts into pinned memory, then the forward and backward passes of the
    # current batch, whose counts arrived a step ago.  Every step does one sort, one forward and one backward.
    # [0:4] the atom counts of ani_sort, [4:8] the size-class counts behind the size order
    counts_pinned = [torch.empty(8, dtype=torch.int32, pin_memory=True) for _ in range(2)]
    main_stream = torch.cuda.current_stream()
    feed_stream = torch.cuda.Stream()          # default priority; the feeder side of the pipeline, as in khan_amd.batching

    def enqueue_sort(slot, timed):
        m0 = m1 = None
        with torch.cuda.stream(feed_stream):
            if timed:
                m0, m1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                m0.record()
            macs, mos = ops.mol_offsets(mol_idxs, n_mols)
            sc, ga, ac = ops.ani_sort(A)
            order = ops.size_order(macs)       # largest molecules first: once per batch, shared by both passes
            if timed:
                m1.record()
            counts_pinned[slot][0:4].copy_(ac, non_blocking=True)
            counts_pinned[slot][4:8].copy_(order[-4:], non_blocking=True)
            done = torch.cuda.Event()
            done.record()
        # macs, mos, sc and order are allocated on the feeder's stream and read by the passes on the main one: the
        # step keeps them alive until an event behind its passes has completed (`in_use` below).  Telling the
        # allocator instead (record_stream) costs an event packet per array on the main stream at every step boundary.
        return {"macs": macs, "mos": mos, "sc": sc, "order": order, "slot": slot, "done": done, "marks": (m0, m1)}

    state = {"cur": None, "n": 0}
    in_use = collections.deque()      # (event behind a step's passes, that step's arrays)

    def step(timed):
        if state["cur"] is None:
            state["cur"] = enqueue_sort(0, False)
        cur = state["cur"]
        state["n"] += 1
        nxt = enqueue_sort(state["n"] & 1, timed)           # the next batch's sort, ahead of this batch's passes
        # this batch's counts: copied a step ago.  The host has waited for the feeder's event, so everything enqueued on
        # the main stream from here on starts after it: no wait on the device is needed.
        cur["done"].synchronize()
        acs = counts_pinned[cur["slot"]][0:4].clone()
        classes = counts_pinned[cur["slot"]][4:8].clone()
        macs, mos, sc, order = cur["macs"], cur["mos"], cur["sc"], cur["order"]
        # events sit directly around each op, on the stream the kernels are launched on
        # (three per step: the end of the forward pass is the start of the backward pass; every event is a packet the
        # next kernel waits behind)
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(3)] if timed else None
        grads, start = [], 0
        for c in acs.tolist():
            grads.append(upstream[start * 384:(start + c) * 384])
            start += c
        if timed:
            marks[0].record()
        feats = ops.featurize(X, Y, Z, A, mos, macs, sc, acs, order=order, size_classes=classes)
        if timed:
            marks[1].record()
        gx, gy, gz = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *grads, order=order, size_classes=classes)
        if timed:
            marks[2].record()
        behind = marks[2] if timed else None
        if with_charges:     # energy, then its gradient with respect to charges and coordinates
            e, qg, cx, cy, cz = ops.ani_charge_all(X, Y, Z, Q, mos, macs, ones_m)
            behind = None
            if timed:
                marks.append(torch.cuda.Event(enable_timing=True))
                marks[3].record()
                behind = marks[3]
        if behind is None:
            behind = torch.cuda.Event()
            behind.record()
        in_use.append((behind, cur))
        while in_use and in_use[0][0].query():
            in_use.popleft()
        state["cur"] = nxt
        return (nxt["marks"], marks), (feats, gx, gy, gz)

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    all_marks = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        m, out = step(True)
        all_marks.append(m)
    host_enqueue_s = time.perf_counter() - t0
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    for sm, m in all_marks:
        ev["sort"].append(sm[0].elapsed_time(sm[1]))
        ev["fwd"].append(m[0].elapsed_time(m[1]))
        ev["bwd"].append(m[1].elapsed_time(m[2]))
        if with_charges:
            ev["charges"].append(m[2].elapsed_time(m[3]))
    ms = {k: float(np.mean(v)) for k, v in ev.items() if v}      # event intervals on the launch stream
    ms_per_step = elapsed / args.steps * 1e3

    # dominant kernel = the longer of forward / backward; both bound by HBM when the arithmetic is minimal
    dom = "bwd" if ms["bwd"] >= ms["fwd"] else "fwd"
    dom_bytes = work["bytes_" + dom]
    dom_flops = work["flops_" + dom]
    achieved = dom_bytes / (ms[dom] * 1e-3) / 1e9
    valu_peak = FP32_PEAK_TFLOPS if w == 4 else FP64_PEAK_TFLOPS
    import bench_profiling as profiling
    traffic, traffic_stale, traffic_entry = profiling.measured_traffic(args.workload, dom)
    roofline = {
        "kernel": "aev_bwd" if dom == "bwd" else "aev_fwd",
        "bound": "hbm",
        "achieved": achieved,
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS,
        "traffic": traffic,
        "traffic_stale": traffic_stale,
        "traffic_source": "profiles/hbm_traffic.json entry %s/%s (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a 64 MiB copy)"
                          % (args.workload, dom) if traffic_entry else None,
        "launch_ms": ms[dom],
        "algorithmic_bytes": dom_bytes,
        "valu_frac": dom_flops / (ms[dom] * 1e-3) / 1e12 / valu_peak,
        "valu_peak_tflops": valu_peak,
        "fwd": {"ms": ms["fwd"], "hbm_frac": work["bytes_fwd"] / (ms["fwd"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "valu_frac": work["flops_fwd"] / (ms["fwd"] * 1e-3) / 1e12 / valu_peak},
        "bwd": {"ms": ms["bwd"], "hbm_frac": work["bytes_bwd"] / (ms["bwd"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "valu_frac": work["flops_bwd"] / (ms["bwd"] * 1e-3) / 1e12 / valu_peak},
        # mol_offsets + ani_sort + size_order of one batch: the nine launches alone on an idle GPU, and the interval
        # they span in the timed loop, where they ride on the feeder stream beside the passes of the batch before
        # (both passes fill the GPU, so the small launches wait for free wave slots; the step does not wait for them)
        "sort_offsets_ms": sort_ms_alone,
        "sort_offsets_interval_beside_passes_ms": ms["sort"],
        "host_enqueue_ms_per_step": host_enqueue_s / args.steps * 1e3,
    }
    if with_charges:
        C = counts["C"]
        peak = FP32_PEAK_TFLOPS if w == 4 else FP64_PEAK_TFLOPS
        roofline["charges"] = {"ms": ms["charges"], "what": "khan_ani_charge_all: energy, dE/dq and dE/dxyz in one pass over the pairs",
                               "valu_frac": 45.0 * C / (ms["charges"] * 1e-3) / 1e12 / peak}

    result = {
        "metric": "AEV fwd+grad atoms/sec, fp%d, 1 MI355X" % (8 * w),
        "value": N / (ms_per_step * 1e-3),
        "unit": "atoms/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if w == 4 else "f64",
        "data": "synthetic",
        "config": {"workload": "%s: ani_sort + AEV forward + AEV backward%s, %d molecules, %d atoms" % (
            args.workload, " + ani_charge energy and gradients" if with_charges else "", n_mols, N), "n_mols": n_mols, "n_atoms": N, "work_counts": counts,
            "feeding": "each step enqueues the next batch's mol_offsets + ani_sort + size_order (and the copy of its 4 atom "
                       "counts and 4 size-class counts to the host) on a feeder stream, ahead of the current batch's "
                       "forward and backward on the main stream, which share that order and launch only the kernels "
                       "whose size class is present"},
        "molecules_per_s": n_mols / (ms_per_step * 1e-3),
        "roofline": roofline,
    }
    if args.reproducible_gradients:
        result["config"]["backward"] = "khan_set_reproducible_gradients(1): not the default kernel for molecules of 33-256 atoms"
    if args.phase2 != "vector":
        result["config"]["forward_phase2"] = args.phase2 + " cores (measurement variant, not the default kernel)"
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(batch, min(n_mols, 8192) if kind == "organic" else 32, min(n_mols, 4096) if kind == "organic" else 8, w)
    return result


if __name__ == "__main__":
    main()
