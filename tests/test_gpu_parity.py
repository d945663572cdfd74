"""Parity of the HIP path (through the C ABI of libkhan_aev.so) with the CPU oracle, on a real MI355X.

Tolerances (stated once, used everywhere below):
  integers (sort, offsets)        bit-exact
  float32 features                |gpu - ref| <= 1e-6 + 1e-5 |ref|, ref = float64 oracle
                                  (and, against the float32 oracle, the same bound widened by the float32
                                  oracle's own distance from the float64 one: the reference's float path
                                  takes acos of a float, which alone moves some entries by > 1e-5 relative)
  float64 features                |gpu - ref| <= 1e-15 + 1e-12 |ref|
  gradients                       |gpu - ref| <= atol + rtol * max(|ref|, S), S = largest |component| of the
                                  reference gradient in the same molecule (components are sums of terms of
                                  both signs, so a tolerance relative to each component alone is not
                                  meaningful); rtol = 1e-5, atol = 1e-6 in float32, rtol = 1e-12 in float64.
                                  float32 gradients are judged against the float64 oracle: the reference's
                                  own float functor is not finite everywhere (see test_oracle_featurize.py).
  charges                         rtol as above relative to max(|ref|, largest |value| in the molecule).
"""
import os
import sys

import numpy as np
import pytest

import helpers
from khan_amd import datagen
from oracle import binding as ob

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

F32_RTOL, F32_ATOL = 1e-5, 1e-6
F64_RTOL, F64_ATOL = 1e-12, 1e-15


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from khan_amd import ops as _ops
    from khan_amd import _lib
    _lib.load()      # fails loudly if the HIP library is missing
    return _ops


def dev(a, dtype=None):
    a = np.ascontiguousarray(a if dtype is None else np.asarray(a).astype(dtype))
    return torch.from_numpy(a).to("cuda:0")


def host(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def mol_scale(ref, MOs, MACs):
    """per-element scale S: largest |ref| inside the element's molecule (ref is [N] or [N,k])."""
    ref = np.asarray(ref, dtype=np.float64)
    flat = np.abs(ref.reshape(ref.shape[0], -1)).max(axis=1) if ref.shape[0] else np.zeros(0)
    S = np.zeros(ref.shape[0])
    for m in range(len(MOs)):
        s = slice(MOs[m], MOs[m] + MACs[m])
        if MACs[m] > 0:
            S[s] = flat[s].max()
    return S.reshape((-1,) + (1,) * (ref.ndim - 1))


def assert_close(name, got, ref, rtol, atol, scale=None, slack=None):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert np.all(np.isfinite(got)), name + ": non-finite output"
    mag = np.abs(ref) if scale is None else np.maximum(np.abs(ref), scale)
    bound = atol + rtol * mag
    if slack is not None:
        bound = bound + slack
    err = np.abs(got - ref)
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(bound > 0, err / bound, np.where(err == 0, 0.0, np.inf))   # bound 0: must be exact
    worst = float(ratio.max()) if err.size else 0.0
    say("   %-34s max|err| %.3e  worst err/bound %.3f" % (name, err.max() if err.size else 0.0, worst))
    assert worst <= 1.0, "%s: err/bound %.3f" % (name, worst)


class Case:
    """A batch on the device plus oracle results, built lazily."""

    def __init__(self, X, Y, Z, A, mol_idxs, n_mols):
        self.X, self.Y, self.Z = (np.asarray(v, dtype=np.float32) for v in (X, Y, Z))
        self.A = np.asarray(A, dtype=np.int32)
        self.mol_idxs = np.asarray(mol_idxs, dtype=np.int32)
        self.n_mols = n_mols
        self.N = self.A.size
        self.MACs, self.MOs = ob.mol_offsets(self.mol_idxs, n_mols)
        self.sc, self.ga, self.ac = ob.ani_sort(self.A)

    @classmethod
    def from_batch(cls, b):
        return cls(b.X, b.Y, b.Z, b.A, b.mol_idxs, b.n_mols)

    def oracle_feat(self, dtype):
        return ob.featurize(self.X, self.Y, self.Z, self.A, self.MOs, self.MACs, self.sc, self.ac, dtype=dtype)

    def upstream(self, seed=11):
        up = np.random.default_rng(seed).standard_normal((self.N, 384)).astype(np.float32).astype(np.float64)
        return ob.scatter_rows(up, self.A, self.sc, self.ac)

    def oracle_grad(self, upb):
        return np.stack(ob.featurize_grad(self.X, self.Y, self.Z, self.A, self.MOs, self.MACs, self.sc, self.ac,
                                          upb, dtype=np.float64), axis=1)



def sample_case(c, mol_ids):
    """The molecules `mol_ids` of case c as a case of their own, and the indices of their atoms in c."""
    mol_ids = np.asarray(mol_ids, dtype=np.int64)
    idx = np.concatenate([np.arange(c.MOs[m], c.MOs[m] + c.MACs[m]) for m in mol_ids]).astype(np.int64)
    mi = np.repeat(np.arange(len(mol_ids)), c.MACs[mol_ids]).astype(np.int32)
    return Case(c.X[idx], c.Y[idx], c.Z[idx], c.A[idx], mi, len(mol_ids)), idx


def strided_molecules(n_mols, count, block=1):
    """`count` molecule indices spread evenly over 0..n_mols-1, in runs of `block` consecutive molecules."""
    starts = np.linspace(0, n_mols - block, count // block).astype(np.int64)
    return np.unique((starts[:, None] + np.arange(block)[None, :]).reshape(-1))


def check_sample_against_oracle(name, c, mol_ids, rows, g, up, rtol, atol, grad_atol):
    """Rows (atom order) and gradients of a full-size launch against the float64 oracle on a sample of its molecules;
    `up` are the upstream rows of that launch in atom order."""
    sub, idx = sample_case(c, mol_ids)
    it = torch.from_numpy(idx).to("cuda:0")
    say("   %s: %d molecules, %d atoms against the float64 oracle" % (name, sub.n_mols, sub.N))
    ref64 = ob.gather_rows(sub.oracle_feat(np.float64), sub.ga)
    assert_close("rows, " + name, host(rows[it]), ref64, rtol, atol)
    upb = ob.scatter_rows(host(up[it]).astype(np.float64), sub.A, sub.sc, sub.ac)
    g64 = sub.oracle_grad(upb)
    assert_close("gradient, " + name, host(g[it]), g64, rtol, grad_atol, scale=mol_scale(g64, sub.MOs, sub.MACs))
    return sub, idx


def gpu_sort_offsets(ops, c):
    macs, mos = ops.mol_offsets(dev(c.mol_idxs), c.n_mols)
    sc, ga, ac = ops.ani_sort(dev(c.A))
    return macs, mos, sc, ga, ac


def check_forward_backward(ops, c, grad=True):
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    assert np.array_equal(host(macs), c.MACs) and np.array_equal(host(mos), c.MOs)
    assert np.array_equal(host(sc), c.sc) and np.array_equal(host(ga), c.ga) and np.array_equal(host(ac), c.ac)
    acs = ac.cpu()
    ref64 = np.concatenate(c.oracle_feat(np.float64))
    ref32 = np.concatenate(c.oracle_feat(np.float32)).astype(np.float64)
    upb = c.upstream() if grad else None
    g64 = c.oracle_grad(upb) if grad else None
    A = dev(c.A)
    for tdt, ndt in ((torch.float32, np.float32), (torch.float64, np.float64)):
        X, Y, Z = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
        f = ops.featurize(X, Y, Z, A, mos, macs, sc, acs)
        got = host(torch.cat(f))
        if ndt == np.float32:
            assert_close("features f32 vs f64 oracle", got, ref64, F32_RTOL, F32_ATOL)
            assert_close("features f32 vs f32 oracle", got, ref32, F32_RTOL, F32_ATOL, slack=np.abs(ref32 - ref64))
        else:
            assert_close("features f64 vs f64 oracle", got, ref64, F64_RTOL, F64_ATOL)
        if grad:
            gb = [dev(x, ndt) for x in upb]
            gx, gy, gz = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *gb)
            gg = host(torch.stack([gx, gy, gz], dim=1))
            S = mol_scale(g64, c.MOs, c.MACs)
            if ndt == np.float32:
                assert_close("gradient f32 vs f64 oracle", gg, g64, F32_RTOL, F32_ATOL, scale=S)
            else:
                assert_close("gradient f64 vs f64 oracle", gg, g64, F64_RTOL, 0.0, scale=S)


# ----------------------------------------------------------------------------- integers
def test_sort_reference_kat(ops):
    say("case: sort KAT, 11-atom fixture")
    _, _, _, a, mi = helpers.fixture11()
    sc, ga, ac = ops.ani_sort(dev(a))
    assert host(ac).tolist() == helpers.FIXTURE11_ATOM_COUNTS
    assert host(sc).tolist() == helpers.FIXTURE11_SCATTER
    assert host(ga).tolist() == helpers.FIXTURE11_GATHER
    macs, mos = ops.mol_offsets(dev(mi), 2)
    assert host(macs).tolist() == [8, 3] and host(mos).tolist() == [0, 8]


@pytest.mark.parametrize("n", [0, 1, 63, 64, 65, 255, 256, 257, 2047, 2048, 2049, 100003, 1 << 20])
def test_sort_bit_exact_random(ops, n):
    say("case: sort random n=%d" % n)
    rng = np.random.default_rng(n)
    a = rng.choice(4, size=n, p=[0.55, 0.3, 0.1, 0.05]).astype(np.int32)
    sc, ga, ac = ops.ani_sort(dev(a))
    osc, oga, oac = ob.ani_sort(a)
    assert np.array_equal(host(ac), oac)
    assert np.array_equal(host(sc), osc)
    assert np.array_equal(host(ga), oga)


def test_sort_single_type_and_out_of_range_types(ops):
    say("case: sort single type / folded types")
    a = np.full(5000, 1, dtype=np.int32)
    sc, ga, ac = ops.ani_sort(dev(a))
    assert host(ac).tolist() == [0, 5000, 0, 0] and np.array_equal(host(sc), np.arange(5000))
    # types outside 0..3 are treated as O, like the reference featurizer's else-branch
    a = np.array([0, 7, 3, -1, 1], dtype=np.int32)
    sc, ga, ac = ops.ani_sort(dev(a))
    osc, oga, oac = ob.ani_sort(np.array([0, 3, 3, 3, 1], dtype=np.int32))
    assert np.array_equal(host(sc), osc) and np.array_equal(host(ga), oga) and np.array_equal(host(ac), oac)


def test_mol_offsets_with_empty_molecules(ops):
    say("case: mol_offsets with empty molecules")
    rng = np.random.default_rng(2)
    counts = rng.integers(0, 30, size=3000)
    counts[[0, 5, 2999]] = 0
    idx = np.repeat(np.arange(3000), counts).astype(np.int32)
    macs, mos = ops.mol_offsets(dev(idx), 3000)
    omacs, omos = ob.mol_offsets(idx, 3000)
    assert np.array_equal(host(macs), omacs) and np.array_equal(host(mos), omos)
    macs, mos = ops.mol_offsets(dev(np.zeros(0, np.int32)), 4)
    assert host(macs).tolist() == [0] * 4 and host(mos).tolist() == [0] * 4


# ----------------------------------------------------------------------------- golden vectors
@pytest.mark.parametrize("prefix", ["fx11", "org8"])
def test_golden_vectors(ops, golden_dir, prefix):
    say("case: golden", prefix)
    g = np.load(os.path.join(golden_dir, "aev_golden.npz"))
    n_mols = int(g[prefix + "_macs"].size)
    c = Case(g[prefix + "_X"], g[prefix + "_Y"], g[prefix + "_Z"], g[prefix + "_A"], g[prefix + "_mol_idxs"], n_mols)
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    assert np.array_equal(host(sc), g[prefix + "_scatter"]) and np.array_equal(host(ga), g[prefix + "_gather"])
    acs = ac.cpu()
    A = dev(c.A)
    up = g[prefix + "_upstream"]
    for tdt, ndt, tag in ((torch.float32, np.float32, "f32"), (torch.float64, np.float64, "f64")):
        X, Y, Z = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
        f = ops.featurize(X, Y, Z, A, mos, macs, sc, acs)
        rows = host(torch.cat(f).view(-1, 384)[ga.long()])
        ref64 = g[prefix + "_feat_f64"]
        if ndt == np.float32:
            ref32 = g[prefix + "_feat_f32"].astype(np.float64)
            assert_close("features f32 vs reference f64", rows, ref64, F32_RTOL, F32_ATOL)
            assert_close("features f32 vs reference f32", rows, ref32, F32_RTOL, F32_ATOL, slack=np.abs(ref32 - ref64))
        else:
            assert_close("features f64 vs reference f64", rows, ref64, F64_RTOL, F64_ATOL)
        gb = [dev(x, ndt) for x in ob.scatter_rows(up, c.A, c.sc, c.ac)]
        gx, gy, gz = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *gb)
        gg = host(torch.stack([gx, gy, gz], dim=1))
        gref = g[prefix + "_grad_f64"]
        S = mol_scale(gref, c.MOs, c.MACs)
        if ndt == np.float32:
            assert_close("gradient f32 vs reference f64", gg, gref, F32_RTOL, F32_ATOL, scale=S)
        else:
            assert_close("gradient f64 vs reference f64", gg, gref, F64_RTOL, 0.0, scale=S)


# ----------------------------------------------------------------------------- seeded batches
def test_organic_batch(ops):
    say("case: organic 1024 molecules (the reference-CPU-sized configuration)")
    check_forward_backward(ops, Case.from_batch(datagen.make_batch("organic", 1024)))


def test_dense_boxes(ops):
    say("case: dense boxes, 6 boxes of 64-256 atoms")
    check_forward_backward(ops, Case.from_batch(datagen.make_batch("boxes", 6)))


def test_edge_shapes(ops):
    say("case: ragged edge shapes")
    rng = np.random.default_rng(9)
    mols = []
    # single atoms, a pair beyond every cutoff, a pair between the cutoffs, an empty molecule,
    # one with 65 atoms and one with 300 atoms (more than a wavefront / more than four wavefronts)
    mols.append((np.array([2]), np.zeros((1, 3))))
    mols.append((np.array([0, 3]), np.array([[0, 0, 0], [0, 0, 5.0]])))
    mols.append((np.array([1, 1]), np.array([[0, 0, 0], [0, 3.5, 0]])))
    mols.append((np.zeros(0, dtype=int), np.zeros((0, 3))))
    for n in (65, 300):
        side = (n / 0.1) ** (1 / 3)
        pts = []
        while len(pts) < n:
            p = rng.uniform(0, side, 3)
            if all(np.linalg.norm(p - q) >= 0.9 for q in pts):
                pts.append(p)
        mols.append((rng.integers(0, 4, n), np.array(pts)))
    mols.append((np.array([3]), np.ones((1, 3))))
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols])
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    check_forward_backward(ops, Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols)))


def _boundary_case():
    """One random box per atom count next to every limit the dispatch and the kernels know: scan shapes
    (16 / 17, 32 / 33), one wavefront (64 / 65), one workgroup (256 / 257), in mixed order."""
    rng = np.random.default_rng(21)
    mols = []
    for n in (33, 16, 257, 64, 17, 256, 32, 65, 1, 2):
        side = (n / 0.09) ** (1 / 3)
        pts = []
        while len(pts) < n:
            p = rng.uniform(0, side, 3)
            if all(np.linalg.norm(p - q) >= 0.9 for q in pts):
                pts.append(p)
        mols.append((rng.integers(0, 4, n), np.array(pts)))
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols]).astype(np.float32).astype(np.float64)
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    return Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))


def test_size_class_boundaries(ops):
    say("case: molecules of 16/17, 32/33, 64/65, 256/257 atoms: features, gradients, grad-inverse, charges")
    c = _boundary_case()
    check_forward_backward(ops, c)
    _check_grad_inverse(ops, c)
    _check_charges(ops, c)


def _check_charges(ops, c):
    """charge energies, dE/dq and dE/dxyz of a case in both precisions against the float64 oracle"""
    q = np.random.default_rng(3).normal(0.0, 0.3, c.N)
    gm = np.random.default_rng(4).standard_normal(c.n_mols)
    E64 = ob.ani_charge(c.X, c.Y, c.Z, q, c.MOs, c.MACs, dtype=np.float64)
    Eabs = ob.ani_charge(c.X, c.Y, c.Z, np.abs(q), c.MOs, c.MACs, dtype=np.float64)
    dq64 = ob.ani_charge_grad(c.X, c.Y, c.Z, q, c.MOs, c.MACs, gm, dtype=np.float64)
    dx64 = np.stack(ob.ani_charge_grad_xyz(c.X, c.Y, c.Z, q, c.MOs, c.MACs, gm, dtype=np.float64), axis=1)
    mos, macs = dev(c.MOs), dev(c.MACs)
    for ndt, rtol in ((np.float32, F32_RTOL), (np.float64, F64_RTOL)):
        X, Y, Z, Q, G = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt), dev(q, ndt), dev(gm, ndt)
        assert_close("charge energy %s" % ndt.__name__, host(ops.ani_charge(X, Y, Z, Q, mos, macs)), E64, rtol, 0.0,
                     scale=np.maximum(Eabs, 1e-300))
        qg, gx, gy, gz = ops.ani_charge_grad_xyz(X, Y, Z, Q, mos, macs, G)
        assert_close("charge dE/dq %s" % ndt.__name__, host(qg), dq64, rtol, 0.0, scale=mol_scale(dq64, c.MOs, c.MACs))
        assert_close("charge dE/dxyz %s" % ndt.__name__, host(torch.stack([gx, gy, gz], dim=1)), dx64, rtol, 0.0,
                     scale=mol_scale(dx64, c.MOs, c.MACs))


def test_mixed_sizes_in_one_ordered_batch(ops):
    say("case: 2,326 molecules of every size class in one batch, shuffled (the size order and the per-class counts are active)")
    rng = np.random.default_rng(5)
    org = datagen.make_batch("organic", 2300)
    box = datagen.make_batch("boxes", 24)
    mols = []
    for b in (org, box):
        for m in range(b.n_mols):
            sl = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
            mols.append((b.A[sl], np.stack([b.X[sl], b.Y[sl], b.Z[sl]], axis=1)))
    for n in (257, 300):                                  # beyond one workgroup
        side = (n / 0.08) ** (1 / 3)
        pts = []
        while len(pts) < n:
            p = rng.uniform(0, side, 3)
            if all(np.linalg.norm(p - q) >= 0.9 for q in pts):
                pts.append(p)
        mols.append((rng.integers(0, 4, n).astype(np.int32), np.array(pts, dtype=np.float32)))
    mols = [mols[i] for i in rng.permutation(len(mols))]
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols]).astype(np.float64)
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
    assert c.n_mols >= 2048                               # the dispatcher orders batches from 2,048 molecules on
    check_forward_backward(ops, c)
    _check_grad_inverse(ops, c)


def test_size_order_workspace_and_size_classes(ops):
    """khan_size_order: a permutation of the molecules by decreasing atom count, followed by the per-size counts and the
    four size-class totals; the *_ordered entry points with that order -- and with a host copy of the class totals,
    which lets them skip the kernels without work -- give what the plain entry points give."""
    say("case: caller-owned size order, size classes, ordered entry points")
    rng = np.random.default_rng(17)
    for label, parts in (("organic only", [("organic", 2200)]), ("organic + boxes", [("organic", 2100), ("boxes", 5)]),
                         ("boxes only", [("boxes", 7)])):
        mols = []
        for kind, k in parts:
            b = datagen.make_batch(kind, k)
            for m in range(b.n_mols):
                sl = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
                mols.append((b.A[sl], np.stack([b.X[sl], b.Y[sl], b.Z[sl]], axis=1)))
        if label == "organic + boxes":                   # one molecule for the general-shape kernel, and an empty one
            n = 270
            side = (n / 0.08) ** (1 / 3)
            pts = []
            while len(pts) < n:
                p = rng.uniform(0, side, 3)
                if all(np.linalg.norm(p - q) >= 0.9 for q in pts):
                    pts.append(p)
            mols.append((rng.integers(0, 4, n).astype(np.int32), np.array(pts, dtype=np.float32)))
            mols.append((np.zeros(0, dtype=np.int32), np.zeros((0, 3), dtype=np.float32)))
        mols = [mols[i] for i in rng.permutation(len(mols))]
        A = np.concatenate([m[0] for m in mols]).astype(np.int32)
        xyz = np.concatenate([m[1] for m in mols]).astype(np.float64)
        mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
        c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
        macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
        acs = ac.cpu()
        order = ops.size_order(macs)
        o = host(order)
        perm, classes = o[:c.n_mols], o[-4:]
        assert np.array_equal(np.sort(perm), np.arange(c.n_mols)), label
        sizes = c.MACs[perm]
        assert np.all(np.minimum(sizes[:-1], 257) >= np.minimum(sizes[1:], 257)), "largest first"
        want = [int((c.MACs <= 32).sum()), int(((c.MACs > 32) & (c.MACs <= 64)).sum()),
                int(((c.MACs > 64) & (c.MACs <= 256)).sum()), int((c.MACs > 256).sum())]
        assert classes.tolist() == want, (label, classes.tolist(), want)
        say("   %s: %d molecules, size classes %s" % (label, c.n_mols, want))
        Ad = dev(c.A)
        upb = c.upstream()
        for tdt, ndt in ((torch.float32, np.float32), (torch.float64, np.float64)):
            X, Y, Z = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
            gb = [dev(u, ndt) for u in upb]
            v = [dev(np.random.default_rng(k).standard_normal(c.N), ndt) for k in range(3)]
            f0 = torch.cat(ops.featurize(X, Y, Z, Ad, mos, macs, sc, acs))
            g0 = torch.stack(ops.featurize_grad(X, Y, Z, Ad, mos, macs, sc, acs, *gb))
            j0 = torch.cat(ops.featurize_grad_inverse(X, Y, Z, Ad, mos, macs, sc, acs, *v))
            for cls in (None, classes):
                f1 = torch.cat(ops.featurize(X, Y, Z, Ad, mos, macs, sc, acs, order=order, size_classes=cls))
                g1 = torch.stack(ops.featurize_grad(X, Y, Z, Ad, mos, macs, sc, acs, *gb, order=order, size_classes=cls))
                j1 = torch.cat(ops.featurize_grad_inverse(X, Y, Z, Ad, mos, macs, sc, acs, *v, order=order, size_classes=cls))
                assert torch.equal(f0, f1) and torch.equal(j0, j1), (label, ndt, cls is None)
                # molecules above one wavefront add their forces with atomics: equal up to the order of the additions
                assert torch.allclose(g0, g1, rtol=1e-5 if ndt == np.float32 else 1e-12, atol=1e-5 if ndt == np.float32 else 1e-12)
                one_wave = torch.from_numpy(c.MACs[c.mol_idxs] <= 32).to("cuda:0")
                assert torch.equal(g0[:, one_wave], g1[:, one_wave])


def test_empty_batch(ops):
    say("case: empty batch (0 atoms, 0 molecules)")
    e32 = torch.empty(0, dtype=torch.float32, device="cuda:0")
    ei = torch.empty(0, dtype=torch.int32, device="cuda:0")
    sc, ga, ac = ops.ani_sort(ei)
    assert host(ac).tolist() == [0, 0, 0, 0]
    f = ops.featurize(e32, e32, e32, ei, ei, ei, sc, ac.cpu())
    assert all(t.numel() == 0 for t in f)
    g = ops.featurize_grad(e32, e32, e32, ei, ei, ei, sc, ac.cpu(), *f)
    assert all(t.numel() == 0 for t in g)
    assert ops.ani_charge(e32, e32, e32, e32, ei, ei).numel() == 0


def _with_coincident_pair(b, mol, src, dst):
    """Copy of batch arrays in which atom `dst` of molecule `mol` sits exactly on atom `src`."""
    X, Y, Z = b.X.copy(), b.Y.copy(), b.Z.copy()
    o = b.MOs[mol]
    X[o + dst], Y[o + dst], Z[o + dst] = X[o + src], Y[o + src], Z[o + src]
    return X, Y, Z


@pytest.mark.parametrize("kind,n_mols,mol,generic", [("organic", 40, 7, False), ("boxes", 3, 1, False), ("boxes", 2, 0, True)])
def test_coincident_atoms_stay_inside_their_pair(ops, kind, n_mols, mol, generic):
    """Two atoms of one molecule at the same position.  Features: the reference's cosine is 0/0 there and its
    fmax/fmin clamp turns that into -1, the angle pi (kernel_cpu.cpp:514-517): finite rows, which the kernels
    reproduce.  Derivatives and charges: the reference divides by the distance (kernel_cpu.cpp:335,
    ani_charges.cpp:67) and returns NaN for every term that holds the pair.  Here such a pair has no direction: it
    is left out of every derivative, and its charge term is the limit 0.  Pinned: every output is finite; the
    features agree with the oracle everywhere; gradients and energies agree wherever the oracle (= the
    reference's arithmetic) is finite; the other molecules of the batch are untouched."""
    say("case: coincident atoms, %s, general kernel %s" % (kind, generic))
    b = datagen.make_batch(kind, n_mols, first_mol=2 if generic else 0)
    if generic:          # two boxes, 30 A apart, declared as ONE molecule of 500 atoms: the general-shape kernels
        assert b.n_atoms > 256
        b.X = b.X.copy()
        b.X[b.MOs[1]:] += np.float32(30.0)
        b.mol_idxs = np.zeros(b.n_atoms, dtype=np.int32)
        b.n_mols = 1
        b.MOs, b.MACs = np.array([0], dtype=np.int32), np.array([b.n_atoms], dtype=np.int32)
    X, Y, Z = _with_coincident_pair(b, mol, 0, 2)
    c = Case(X, Y, Z, b.A, b.mol_idxs, b.n_mols)
    clean = Case(b.X, b.Y, b.Z, b.A, b.mol_idxs, b.n_mols)
    pair = (c.MOs[mol] + 0, c.MOs[mol] + 2)
    with np.errstate(all="ignore"):
        ref = np.concatenate(c.oracle_feat(np.float64)).reshape(-1, 384)
        upb = c.upstream()
        gref = c.oracle_grad(upb)
    rows = c.ga            # row of atom g in the concatenated buckets
    assert np.all(np.isfinite(ref)), "the reference's features are finite for a coincident pair"
    assert not np.array_equal(ref[rows[pair[0]]], np.concatenate(clean.oracle_feat(np.float64)).reshape(-1, 384)[rows[pair[0]]])
    in_mol = (c.mol_idxs == mol)
    assert np.all(np.isfinite(gref[~in_mol])) and not np.all(np.isfinite(gref[in_mol]))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    A = dev(c.A)
    q = np.random.default_rng(5).normal(0.0, 0.3, c.N)
    with np.errstate(all="ignore"):
        E64 = ob.ani_charge(c.X, c.Y, c.Z, q, c.MOs, c.MACs, dtype=np.float64)
    assert not np.isfinite(E64[mol]) and np.all(np.isfinite(np.delete(E64, mol)))
    for tdt, ndt, rtol, atol in ((torch.float32, np.float32, F32_RTOL, F32_ATOL), (torch.float64, np.float64, F64_RTOL, F64_ATOL)):
        Xd, Yd, Zd = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
        got = host(torch.cat(ops.featurize(Xd, Yd, Zd, A, mos, macs, sc, acs))).reshape(-1, 384)
        assert np.all(np.isfinite(got)), "features must be finite"
        # The atoms that see the pair as two partners form an exactly collinear triple (angle 0): the reference takes
        # acos of a cosine that rounding left at 1 - 1e-16, i.e. an angle of 1.5e-8 instead of 0, and loses up to
        # 1e-7 relative there in float64 (the kernels take the sine from the cross product: exactly 0).  The rows
        # of the pair's molecule are therefore compared to 1e-6 in float64; all other rows to the usual bound.
        own = np.isin(np.arange(got.shape[0]), rows[in_mol])
        assert_close("features %s vs f64 oracle, other molecules" % ndt.__name__, got[~own], ref[~own], rtol, atol)
        assert_close("features %s vs f64 oracle, the pair's molecule" % ndt.__name__, got[own], ref[own],
                     max(rtol, 1e-6), atol)
        gx, gy, gz = ops.featurize_grad(Xd, Yd, Zd, A, mos, macs, sc, acs, *[dev(u, ndt) for u in upb])
        gg = host(torch.stack([gx, gy, gz], dim=1))
        assert np.all(np.isfinite(gg)), "gradients must be finite"
        okg = np.isfinite(gref).all(axis=1)
        S = mol_scale(np.where(np.isfinite(gref), gref, 0.0), c.MOs, c.MACs)
        assert_close("gradient %s where the oracle is finite" % ndt.__name__, gg[okg], gref[okg], rtol,
                     atol if ndt == np.float32 else 0.0, scale=S[okg])
        # the other molecules do not notice
        Xc, Yc, Zc = dev(clean.X, ndt), dev(clean.Y, ndt), dev(clean.Z, ndt)
        got_clean = host(torch.cat(ops.featurize(Xc, Yc, Zc, A, mos, macs, sc, acs))).reshape(-1, 384)
        others = rows[~in_mol]
        assert np.array_equal(got[others], got_clean[others])
        # Jacobian-vector product and charges: finite
        v = [dev(np.random.default_rng(k).standard_normal(c.N), ndt) for k in range(3)]
        jv = host(torch.cat(ops.featurize_grad_inverse(Xd, Yd, Zd, A, mos, macs, sc, acs, *v)))
        assert np.all(np.isfinite(jv)), "grad-inverse must be finite"
        Q = dev(q, ndt)
        e = host(ops.ani_charge(Xd, Yd, Zd, Q, mos, macs))
        qg, cx, cy, cz = ops.ani_charge_grad_xyz(Xd, Yd, Zd, Q, mos, macs, torch.ones(c.n_mols, dtype=tdt, device="cuda:0"))
        assert np.all(np.isfinite(e)) and all(np.all(np.isfinite(host(t))) for t in (qg, cx, cy, cz))
        keep = np.arange(c.n_mols) != mol
        Eabs = ob.ani_charge(c.X, c.Y, c.Z, np.abs(q), c.MOs, c.MACs, dtype=np.float64)
        assert_close("charge energy of the other molecules", e[keep], E64[keep], rtol, 0.0, scale=np.maximum(Eabs[keep], 1e-300))


def test_atoms_without_a_molecule_get_zeros(ops):
    """A batch with atoms and no molecule: the reference zero-fills its outputs before it looks at the molecules
    (functor_op_cpu.cpp:31-38, 68-72), so rows and gradients are zeros."""
    say("case: n_mols = 0 with 5 atoms")
    A = dev(np.array([0, 1, 1, 3, 2], dtype=np.int32))
    sc, ga, ac = ops.ani_sort(A)
    ei = torch.empty(0, dtype=torch.int32, device="cuda:0")
    for tdt in (torch.float32, torch.float64):
        x = torch.rand(5, dtype=tdt, device="cuda:0")
        f = ops.featurize(x, x, x, A, ei, ei, sc, ac.cpu())
        assert sum(t.numel() for t in f) == 5 * 384 and all(float(t.abs().sum()) == 0.0 for t in f)
        up = [torch.ones_like(t) for t in f]
        g = ops.featurize_grad(x, x, x, A, ei, ei, sc, ac.cpu(), *up)
        assert all(t.numel() == 5 and float(t.abs().sum()) == 0.0 for t in g)
        j = ops.featurize_grad_inverse(x, x, x, A, ei, ei, sc, ac.cpu(), x, x, x)
        assert all(float(t.abs().sum()) == 0.0 for t in j)


def test_out_of_range_type_goes_to_oxygen_bucket(ops):
    say("case: atom type outside 0..3 is treated as O")
    b = datagen.make_batch("organic", 4, first_mol=77)
    A_bad = b.A.copy()
    A_bad[b.A == 3] = 9
    c = Case(b.X, b.Y, b.Z, b.A, b.mol_idxs, b.n_mols)
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    X, Y, Z = dev(c.X), dev(c.Y), dev(c.Z)
    good = host(torch.cat(ops.featurize(X, Y, Z, dev(b.A), mos, macs, sc, ac.cpu())))
    bad = host(torch.cat(ops.featurize(X, Y, Z, dev(A_bad), mos, macs, sc, ac.cpu())))
    assert np.array_equal(good, bad)


# ----------------------------------------------------------------------------- charges
@pytest.mark.parametrize("kind,n_mols", [("organic", 512), ("boxes", 4)])
def test_charges(ops, kind, n_mols):
    say("case: charges", kind, n_mols)
    b = datagen.make_batch(kind, n_mols)
    q = datagen.charges(b.n_atoms).astype(np.float64)
    gm = np.random.default_rng(4).standard_normal(n_mols)
    E64 = ob.ani_charge(b.X, b.Y, b.Z, q, b.MOs, b.MACs, dtype=np.float64)
    dq64 = ob.ani_charge_grad(b.X, b.Y, b.Z, q, b.MOs, b.MACs, gm, dtype=np.float64)
    dx64 = np.stack(ob.ani_charge_grad_xyz(b.X, b.Y, b.Z, q, b.MOs, b.MACs, gm, dtype=np.float64), axis=1)
    # the energy is a sum of terms of both signs: scale = sum of |terms| per molecule = energy with |q|
    Eabs = ob.ani_charge(b.X, b.Y, b.Z, np.abs(q), b.MOs, b.MACs, dtype=np.float64)
    mos, macs = dev(b.MOs), dev(b.MACs)
    for tdt, ndt, rtol in ((torch.float32, np.float32, F32_RTOL), (torch.float64, np.float64, F64_RTOL)):
        X, Y, Z, Q, G = dev(b.X, ndt), dev(b.Y, ndt), dev(b.Z, ndt), dev(q, ndt), dev(gm, ndt)
        E = host(ops.ani_charge(X, Y, Z, Q, mos, macs))
        assert_close("charge energy %s" % ndt.__name__, E, E64, rtol, 0.0, scale=Eabs)
        dq = host(ops.ani_charge_grad(X, Y, Z, Q, mos, macs, G))
        assert_close("charge dE/dq %s" % ndt.__name__, dq, dq64, rtol, 0.0, scale=mol_scale(dq64, b.MOs, b.MACs))
        qg, gx, gy, gz = ops.ani_charge_grad_xyz(X, Y, Z, Q, mos, macs, G)
        assert np.array_equal(host(qg), dq)
        dxyz = host(torch.stack([gx, gy, gz], dim=1))
        assert_close("charge dE/dxyz %s" % ndt.__name__, dxyz, dx64, rtol, 0.0, scale=mol_scale(dx64, b.MOs, b.MACs))
        # energy and both gradients from one pass over the pairs: the same gradients bit for bit, the energy (summed
        # there as half the sum of q_i dE/dq_i) against the oracle
        ea, qa, xa, ya, za = ops.ani_charge_all(X, Y, Z, Q, mos, macs, G)
        assert_close("charge energy from the one-pass call %s" % ndt.__name__, host(ea), E64, rtol, 0.0, scale=Eabs)
        assert torch.equal(qa, qg) and torch.equal(xa, gx) and torch.equal(ya, gy) and torch.equal(za, gz)
        # Euler: E is bilinear in q, so E = 1/2 sum_i q_i dE/dq_i (with unit upstream gradient)
        ones = torch.ones(n_mols, dtype=tdt, device="cuda:0")
        dq1 = host(ops.ani_charge_grad(X, Y, Z, Q, mos, macs, ones)).astype(np.float64)
        euler = 0.5 * np.add.reduceat(np.asarray(q, ndt).astype(np.float64) * dq1, b.MOs)
        assert_close("Euler identity %s" % ndt.__name__, euler, E.astype(np.float64), 10 * rtol, 0.0, scale=Eabs)


def _coulomb_brute(X, Y, Z, q, MOs, MACs, k, g):
    """k sum_{i<j} q_i q_j / r_ij per molecule and its gradients, straight from the definition in float64."""
    E = np.zeros(len(MOs))
    dq = np.zeros(len(q))
    dx = np.zeros((len(q), 3))
    xyz = np.stack([X, Y, Z], axis=1).astype(np.float64)
    for m in range(len(MOs)):
        s = slice(MOs[m], MOs[m] + MACs[m])
        d = xyz[s, None, :] - xyz[None, s, :]
        r = np.linalg.norm(d, axis=-1)
        np.fill_diagonal(r, np.inf)
        qq = q[s, None] * q[None, s]
        E[m] = 0.5 * k * (qq / r).sum()
        dq[s] = g[m] * k * (q[None, s] / r).sum(axis=1)
        dx[s] = g[m] * k * (-(qq / r ** 3)[:, :, None] * d).sum(axis=1)
    return E, dq, dx


@pytest.mark.parametrize("kind,n_mols", [("organic", 300), ("boxes", 3)])
def test_plain_coulomb_sums(ops, kind, n_mols):
    """khan_coulomb_*: the charge kernels without damping, E = k sum q_i q_j / r_ij (the literal pairwise Coulomb
    energy), against the definition evaluated with numpy in float64; the damped kernel must differ from it."""
    say("case: plain Coulomb sums, %s" % kind)
    b = datagen.make_batch(kind, n_mols)
    q = datagen.charges(b.n_atoms).astype(np.float64)
    g = np.random.default_rng(8).standard_normal(b.n_mols)
    for k in (1.0, 14.399645):
        E, dq, dx = _coulomb_brute(b.X, b.Y, b.Z, q, b.MOs, b.MACs, k, g)
        Eabs, _, _ = _coulomb_brute(b.X, b.Y, b.Z, np.abs(q), b.MOs, b.MACs, k, g)
        mos, macs = dev(b.MOs), dev(b.MACs)
        for ndt, rtol in ((np.float32, F32_RTOL), (np.float64, F64_RTOL)):
            X, Y, Z, Q, G = dev(b.X, ndt), dev(b.Y, ndt), dev(b.Z, ndt), dev(q, ndt), dev(g, ndt)
            e = host(ops.coulomb(X, Y, Z, Q, mos, macs, k))
            assert_close("coulomb energy %s" % ndt.__name__, e, E, rtol, 0.0, scale=Eabs)
            qg, gx, gy, gz = ops.coulomb_grad(X, Y, Z, Q, mos, macs, G, k)
            assert_close("coulomb dE/dq %s" % ndt.__name__, host(qg), dq, rtol, 0.0, scale=mol_scale(dq, b.MOs, b.MACs))
            assert_close("coulomb dE/dxyz %s" % ndt.__name__, host(torch.stack([gx, gy, gz], dim=1)), dx, rtol, 0.0,
                         scale=mol_scale(dx, b.MOs, b.MACs))
    damped = host(ops.ani_charge(dev(b.X, np.float64), dev(b.Y, np.float64), dev(b.Z, np.float64), dev(q, np.float64), mos, macs))
    assert not np.allclose(damped, helpers.CHARGE_K * _coulomb_brute(b.X, b.Y, b.Z, q, b.MOs, b.MACs, 1.0, g)[0], rtol=1e-3)


def test_charge_reference_fixture_gradient_consistency(ops):
    # the reference's only check of charges: dE/dq from the op agrees with a numeric derivative of the
    # energy op (gpu_featurizer/test_kernel.py:403-459, delta 1e-3, tol 1e-11 in float64)
    say("case: charges on the 11-atom fixture, numeric dE/dq")
    x, y, z, a, mi = helpers.fixture11()
    q = helpers.FIXTURE11_QS
    X, Y, Z = dev(x), dev(y), dev(z)
    mos, macs = dev(np.array([0, 8], np.int32)), dev(np.array([8, 3], np.int32))
    ones = torch.ones(2, dtype=torch.float64, device="cuda:0")
    dq = host(ops.ani_charge_grad(X, Y, Z, dev(q), mos, macs, ones))
    delta = 1e-3
    for i in range(11):
        qp, qm = q.copy(), q.copy()
        qp[i] += delta
        qm[i] -= delta
        ep = host(ops.ani_charge(X, Y, Z, dev(qp), mos, macs)).sum()
        em = host(ops.ani_charge(X, Y, Z, dev(qm), mos, macs)).sum()
        assert abs((ep - em) / (2 * delta) - dq[i]) < 1e-11
    xyz = np.stack([x, y, z], axis=1)
    for m, s in enumerate((slice(0, 8), slice(8, 11))):
        e = host(ops.ani_charge(X, Y, Z, dev(q), mos, macs))[m]
        assert e == pytest.approx(helpers.brute_force_charge_energy(xyz[s], q[s]), rel=1e-12)


# ----------------------------------------------------------------------------- crowded centres
def _packed_ball(rng, n, radius, min_dist):
    pts = []
    while len(pts) < n:
        p = rng.uniform(-radius, radius, 3)
        if np.linalg.norm(p) <= radius and all(np.linalg.norm(p - q) >= min_dist for q in pts):
            pts.append(p)
    return np.array(pts)


def test_crowded_centres_take_the_fallback(ops):
    # molecules of at most 64 atoms in which centres have more than 32 partners inside the 3.1 A angular
    # cutoff: the one-wavefront-per-molecule kernels keep 32 per centre and must redo such a centre with
    # the general per-centre routine.  Mixed with ordinary molecules in the same workgroup.
    say("case: centres with more than 32 angular partners")
    rng = np.random.default_rng(31)
    mols = []
    small = datagen.make_batch("organic", 3, first_mol=5)
    for m in range(3):
        s = slice(small.MOs[m], small.MOs[m] + small.MACs[m])
        mols.append((small.A[s], np.stack([small.X[s], small.Y[s], small.Z[s]], axis=1)))
    mols.insert(1, (rng.integers(0, 4, 60), _packed_ball(rng, 60, 2.3, 0.85)))       # every centre crowded
    # a dumbbell: a crowded ball joined to a sparse tail, so only some centres overflow
    ball = _packed_ball(rng, 40, 2.0, 0.85)
    # (jittered: exactly collinear triples have no derivative, the oracle returns NaN for them)
    tail = np.array([[2.5 + 1.1 * k, 0.2 * (-1) ** k, 0.0] for k in range(12)]) + rng.uniform(-0.05, 0.05, (12, 3))
    mols.append((rng.integers(0, 4, 52), np.concatenate([ball, tail])))
    mols.append((np.full(45, 1), _packed_ball(rng, 45, 2.1, 0.85)))                   # one type only
    # the same for the one-workgroup-per-molecule kernels (65..256 atoms): more than 32 angular and more
    # than 64 radial partners around the inner atoms
    mols.append((rng.integers(0, 4, 110), _packed_ball(rng, 110, 3.0, 0.85)))
    mols.append((rng.integers(0, 4, 200), _packed_ball(rng, 200, 3.9, 0.85)))
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols])
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
    # the premise of the test: some centre really has more than 32 angular partners
    worst = 0
    for m in range(len(mols)):
        p = mols[m][1]
        dm = np.linalg.norm(p[:, None] - p[None], axis=2)
        worst = max(worst, int(((dm < 3.1) & (dm > 0)).sum(axis=1).max()))
    assert worst > 32, worst
    check_forward_backward(ops, c)



def test_reproducible_gradients_setting(ops):
    """khan_set_reproducible_gradients(1): the workgroup-per-molecule backward kernel sums a molecule's forces in LDS in
    a fixed order instead of with hardware atomics.  Dense boxes (65..256 atoms), boxes of 40 and 60 atoms
    (that kernel's in float32), small organic molecules and a ball with more than 64 angular partners per centre (its fallback inside the
    kernel), in both precisions: against the float64 oracle at the usual tolerances, identical bits on repeated runs
    (the outputs are fresh, uninitialised arrays every time: this form stores every gradient once and never reads
    them), and, since the setting changes the order of the sums only, close to what the default gives."""
    say("case: reproducible gradients (forces summed in LDS)")
    rng = np.random.default_rng(77)
    box = datagen.make_batch("boxes", 10, first_mol=100)
    org = datagen.make_batch("organic", 400, first_mol=3000)
    mols = []
    for b in (box, org):
        for m in range(b.n_mols):
            sl = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
            mols.append((b.A[sl], np.stack([b.X[sl], b.Y[sl], b.Z[sl]], axis=1)))
    mols.insert(3, (rng.integers(0, 4, 200), _packed_ball(rng, 200, 3.9, 0.85)))
    for n_small in (40, 60):
        mols.insert(5, (rng.integers(0, 4, n_small), _sparse_box(rng, n_small, 0.1, 0.9)))
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols])
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
    assert int((c.MACs > 64).sum()) >= 11 and int(((c.MACs > 32) & (c.MACs <= 64)).sum()) == 2, np.sort(c.MACs)[-20:]
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    upb = c.upstream()
    g64 = c.oracle_grad(upb)
    S = mol_scale(g64, c.MOs, c.MACs)
    Ad = dev(c.A)
    previous = ops.set_reproducible_gradients(True)
    try:
        assert previous is False
        for ndt, rtol, atol in ((np.float32, F32_RTOL, F32_ATOL), (np.float64, F64_RTOL, 0.0)):
            X, Y, Z = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
            gb = [dev(u, ndt) for u in upb]
            runs = []
            for k in range(3):
                g = torch.stack(ops.featurize_grad(X, Y, Z, Ad, mos, macs, sc, acs, *gb), dim=1)
                runs.append(g)
                torch.zeros(1 << 22, device="cuda:0").sum()          # other work in between
            assert_close("reproducible gradient %s vs f64 oracle" % ndt.__name__, host(runs[0]), g64, rtol, atol, scale=S)
            assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2]), "gradients differ between runs"
            assert ops.set_reproducible_gradients(False) is True
            g_default = torch.stack(ops.featurize_grad(X, Y, Z, Ad, mos, macs, sc, acs, *gb), dim=1)
            assert ops.set_reproducible_gradients(True) is False
            assert_close("default gradient %s vs f64 oracle" % ndt.__name__, host(g_default), g64, rtol, atol, scale=S)
            assert_close("reproducible vs default %s" % ndt.__name__, host(runs[0]), host(g_default).astype(np.float64), 4 * rtol, 4 * atol, scale=S)
    finally:
        ops.set_reproducible_gradients(False)

def _sparse_box(rng, n, density, min_dist):
    """n points in a cube at the given number density, no two closer than min_dist (cell by cell, so that thousands
    of points take a moment and not minutes)."""
    side = (n / density) ** (1 / 3)
    pts = np.empty((0, 3))
    while len(pts) < n:
        cand = rng.uniform(0, side, (n, 3))
        for p in cand:
            if len(pts) == 0 or np.min(np.linalg.norm(pts - p, axis=1)) >= min_dist:
                pts = np.vstack([pts, p])
                if len(pts) == n:
                    break
    return pts


def test_molecules_of_more_than_256_atoms(ops):
    # above 256 atoms several workgroups share a molecule and read its atoms, sorted by type, from device memory:
    # boxes of 257 to 1,500 atoms at the density of the dense-box workload, a crowded ball whose inner centres
    # overflow the partner lists (more than 64 radial, more than 32 angular forward, more than 64 angular backward),
    # a single-type box, ordinary molecules in between; features, gradients and the Jacobian-vector product
    say("case: molecules of 257..1,500 atoms, one of them crowded")
    rng = np.random.default_rng(41)
    mols = []
    small = datagen.make_batch("organic", 4, first_mol=11)
    for m in range(4):
        sl = slice(small.MOs[m], small.MOs[m] + small.MACs[m])
        mols.append((small.A[sl], np.stack([small.X[sl], small.Y[sl], small.Z[sl]], axis=1)))
    for n in (257, 700, 1500):
        mols.append((rng.choice(4, n, p=[0.5, 0.3, 0.1, 0.1]), _sparse_box(rng, n, 0.1, 0.9)))
    mols.append((rng.integers(0, 4, 420), _packed_ball(rng, 420, 5.0, 0.85)))
    mols.append((np.full(300, 2), _sparse_box(rng, 300, 0.1, 0.9)))
    # denser: most centres have more than 64 radial partners (their lists are worked off in pieces), few more than 32 angular
    dense = _sparse_box(rng, 500, 0.17, 0.9)
    dd = np.linalg.norm(dense[:, None] - dense[None], axis=2)
    crowd_r, crowd_a = ((dd < 4.6) & (dd > 0)).sum(axis=1), ((dd < 3.1) & (dd > 0)).sum(axis=1)
    assert int(((crowd_r > 64) & (crowd_a <= 32)).sum()) >= 20, (np.sort(crowd_r)[-30:], np.sort(crowd_a)[-30:])
    mols.append((rng.choice(4, 500, p=[0.5, 0.3, 0.1, 0.1]), dense))
    box = datagen.make_batch("boxes", 1)
    mols.append((box.A, np.stack([box.X, box.Y, box.Z], axis=1)))
    mols = [mols[i] for i in rng.permutation(len(mols))]
    p = max(mols, key=lambda m: len(m[0]) if len(m[0]) == 420 else 0)[1]
    dm = np.linalg.norm(p[:, None] - p[None], axis=2)
    assert int(((dm < 3.1) & (dm > 0)).sum(axis=1).max()) > 64 and int(((dm < 4.6) & (dm > 0)).sum(axis=1).max()) > 64
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols]).astype(np.float32).astype(np.float64)
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
    check_forward_backward(ops, c)
    _check_grad_inverse(ops, c)
    _check_charges(ops, c)


def _jittered_lattice(rng, n, spacing, jitter, shape=None):
    """n points on a cubic lattice (or one of the given shape), each moved by up to `jitter` along every axis"""
    if shape is None:
        k = int(np.ceil(n ** (1 / 3)))
        shape = (k, k, k)
    grid = np.stack(np.meshgrid(*[np.arange(d) for d in shape], indexing="ij"), axis=-1).reshape(-1, 3).astype(np.float64)
    pick = rng.permutation(len(grid))[:n]
    return grid[pick] * spacing + rng.uniform(-jitter, jitter, (n, 3))


def test_large_molecules_in_every_regime_of_their_sort(ops):
    # The kernel that sorts the atoms of a molecule of more than 256 atoms takes 4, 8 or 16 cells per dimension by the
    # molecule's size and ranks the atoms of a step in one of two ways; a chunk of 64 sorted atoms may be full, nearly
    # empty, or span two types.  Shapes: 9,000 atoms (16 cells, few atoms share a bin within a step), 1,025 (8 cells), 320
    # (five full chunks) and 321, a flat sheet and a chain (no extent along one or two axes), in input orders that are
    # not spatial.  Features, gradients, Jacobian-vector product and charges against the oracle.
    say("case: large molecules: 9,000 / 1,025 / 320 / 321 atoms, a sheet, a chain")
    rng = np.random.default_rng(57)
    types = lambda n: rng.choice(4, n, p=[0.5, 0.3, 0.1, 0.1])
    mols = [(types(9000), _jittered_lattice(rng, 9000, 2.15, 0.5)),
            (types(1025), _jittered_lattice(rng, 1025, 2.15, 0.5)),
            (types(320), _jittered_lattice(rng, 320, 2.15, 0.5)),
            (np.full(321, 1), _jittered_lattice(rng, 321, 2.15, 0.5)),
            (types(400), _jittered_lattice(rng, 400, 1.6, 0.3, shape=(20, 20, 1))),
            (types(300), _jittered_lattice(rng, 300, 1.3, 0.25, shape=(300, 1, 1)))]
    small = datagen.make_batch("organic", 2, first_mol=21)
    for m in range(2):
        sl = slice(small.MOs[m], small.MOs[m] + small.MACs[m])
        mols.insert(2 * m + 1, (small.A[sl], np.stack([small.X[sl], small.Y[sl], small.Z[sl]], axis=1)))
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols]).astype(np.float32).astype(np.float64)
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
    check_forward_backward(ops, c)
    _check_grad_inverse(ops, c)
    _check_charges(ops, c)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_large_molecules(ops, seed):
    # batches of one to four molecules of up to 3,000 atoms, most of them above 256: cubes, slabs and rods at densities
    # of 0.02 to 0.16 atoms per cubic Angstrom, even or skewed type mixes, in an input order that is not spatial
    say("case: random large molecules, seed %d" % seed)
    rng = np.random.default_rng(seed)
    for _ in range(4):
        mols = []
        for _m in range(int(rng.integers(1, 5))):
            n = int(rng.choice([rng.integers(257, 400), rng.integers(400, 1100), rng.integers(1100, 3000), rng.integers(1, 200)]))
            side = (n / float(rng.uniform(0.02, 0.16))) ** (1 / 3)
            ext = np.array({"cube": (side, side, side), "slab": (2 * side, 2 * side, side / 4),
                            "rod": (4 * side, side / 2, side / 2)}[str(rng.choice(["cube", "slab", "rod"]))])
            k = np.maximum(np.ceil(ext / 1.9).astype(int), 1)
            while np.prod(k) < n:
                k += 1
            cell = ext / k
            grid = np.stack(np.meshgrid(*[np.arange(d) for d in k], indexing="ij"), -1).reshape(-1, 3)
            pos = grid[rng.permutation(len(grid))[:n]] * cell + rng.uniform(-0.4, 0.4, (n, 3)) * np.minimum(cell, 1.9) / 1.9
            mols.append((rng.choice(4, n, p=rng.dirichlet(np.ones(4) * rng.choice([0.3, 3.0]))), pos))
        A = np.concatenate([m[0] for m in mols]).astype(np.int32)
        xyz = np.concatenate([m[1] for m in mols]).astype(np.float32).astype(np.float64)
        mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
        say("   sizes %s" % [len(m[0]) for m in mols])
        check_forward_backward(ops, Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols)))


def test_radial_lists_at_their_fullest(ops):
    # The one-wavefront forward kernel gives every partner type a place of its own in a centre's radial list, each
    # rounded up to a whole trip of the walk.  Fullest lists: molecules of exactly 16, 32 and 64 atoms (the three scan
    # shapes) with an odd number of atoms of every type, packed so that every atom is inside every other atom's
    # radial cutoff; beside them single-type molecules and one with a type that no atom has.
    say("case: radial lists at their fullest (16 / 32 / 64 atoms, odd type counts, everything inside the cutoff)")
    rng = np.random.default_rng(77)
    mols = []
    for counts in ((5, 5, 3, 3), (9, 9, 7, 7), (17, 17, 15, 15), (1, 1, 1, 13), (16, 0, 0, 0), (0, 31, 1, 0), (3, 0, 5, 7)):
        n = sum(counts)
        types = rng.permutation(np.repeat(np.arange(4), counts))
        if n < 64:
            mols.append((types, _packed_ball(rng, n, 2.25, 0.8)))
        else:
            # 64 atoms on a sphere of 4.58 A diameter: 63 radial partners each, and no more than 32 inside the
            # angular cutoff, so that the lists are used and not the fallback for crowded centres
            pts = []
            while len(pts) < n:
                v = rng.standard_normal(3)
                v *= 2.29 / np.linalg.norm(v)
                if all(np.linalg.norm(v - q) >= 0.8 for q in pts):
                    pts.append(v)
            pts = np.array(pts)
            dm = np.linalg.norm(pts[:, None] - pts[None], axis=2)
            assert ((dm < 3.1) & (dm > 0)).sum(axis=1).max() <= 32
            mols.append((types, pts))
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols])
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    for types, p in mols:
        dm = np.linalg.norm(p[:, None] - p[None], axis=2)
        assert dm.max() < 4.6                       # the premise: every pair is a radial pair
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
    check_forward_backward(ops, c)
    _check_grad_inverse(ops, c)


# ----------------------------------------------------------------------------- full-size batch
def test_full_size_batch_properties(ops):
    # 65,536 molecules (the benchmark batch) in float32: properties that need no oracle at full size, plus
    # the oracle on the first and last 256 molecules.
    say("case: organic 65536, full-size properties")
    M = 65536
    b = datagen.make_batch("organic", M)
    c = Case.from_batch(b)
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    assert np.array_equal(host(sc), c.sc) and np.array_equal(host(ga), c.ga) and np.array_equal(host(ac), c.ac)
    assert np.array_equal(host(macs), c.MACs) and np.array_equal(host(mos), c.MOs)
    # ga is the inverse of the bucket placement: sorted-by-type rows gathered back give atom order
    acs = ac.cpu()
    X, Y, Z, A = dev(c.X), dev(c.Y), dev(c.Z), dev(c.A)
    f = ops.featurize(X, Y, Z, A, mos, macs, sc, acs)
    rows = torch.cat(f).view(-1, 384)[ga.long()]          # [N, 384] in atom order
    assert bool(torch.isfinite(rows).all())
    assert float(rows.min()) >= 0.0                        # every term of every feature is non-negative
    up = torch.from_numpy(datagen.normal(c.N * 384)).to("cuda:0").view(-1, 384)
    inv = torch.empty_like(ga.long())
    inv[ga.long()] = torch.arange(c.N, device="cuda:0")
    upb_all = up[inv]                                      # upstream rows in bucket order
    gb, start = [], 0
    for k in acs.tolist():
        gb.append(upb_all[start:start + k].reshape(-1))
        start += k
    gx, gy, gz = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *gb)
    g = torch.stack([gx, gy, gz], dim=1)
    assert bool(torch.isfinite(g).all())
    # translation invariance: the gradient components of a molecule add up to zero
    seg = torch.from_numpy(c.mol_idxs.astype(np.int64)).to("cuda:0")
    net = torch.zeros(M, 3, device="cuda:0", dtype=torch.float64).index_add_(0, seg, g.double())
    mag = torch.zeros(M, 3, device="cuda:0", dtype=torch.float64).index_add_(0, seg, g.double().abs())
    rel = (net.abs() / (mag + 1e-30)).max().item()
    say("   net force / sum |force| per molecule, worst %.3e" % rel)
    assert rel < 2e-5
    # batch independence: a molecule's rows do not depend on what else is in the batch -- bit for bit
    for first, cnt in ((0, 256), (M - 256, 256), (30000, 64)):
        sb = datagen.make_batch("organic", cnt, first_mol=first)
        sc_ = Case.from_batch(sb)
        a0 = int(c.MOs[first])
        assert np.array_equal(sb.X, c.X[a0:a0 + sb.n_atoms])
        m2, o2, s2, g2, c2 = gpu_sort_offsets(ops, sc_)
        f2 = ops.featurize(dev(sb.X), dev(sb.Y), dev(sb.Z), dev(sb.A), o2, m2, s2, c2.cpu())
        rows2 = torch.cat(f2).view(-1, 384)[g2.long()]
        assert torch.equal(rows2, rows[a0:a0 + sb.n_atoms])
        ref64 = ob.gather_rows(sc_.oracle_feat(np.float64), sc_.ga)
        assert_close("rows of molecules %d.. vs f64 oracle" % first, host(rows2), ref64, F32_RTOL, F32_ATOL)
        upb = ob.scatter_rows(host(up[a0:a0 + sb.n_atoms]).astype(np.float64), sb.A, sc_.sc, sc_.ac)
        g64 = sc_.oracle_grad(upb)
        assert_close("gradient of molecules %d.. vs f64 oracle" % first, host(g[a0:a0 + sb.n_atoms]), g64,
                     F32_RTOL, F32_ATOL, scale=mol_scale(g64, sc_.MOs, sc_.MACs))
    # the oracle on a sample taken at a stride through the whole batch (2,048 molecules in runs of 8), and on the
    # 64 molecules with the most atoms
    check_sample_against_oracle("2048 molecules at a stride", c, strided_molecules(M, 2048, block=8), rows, g, up,
                                F32_RTOL, F32_ATOL, F32_ATOL)
    largest = np.argsort(-c.MACs.astype(np.int64), kind="stable")[:64]
    say("   the 64 largest molecules have %d..%d atoms" % (c.MACs[largest].min(), c.MACs[largest].max()))
    check_sample_against_oracle("the 64 largest molecules", c, np.sort(largest), rows, g, up, F32_RTOL, F32_ATOL, F32_ATOL)


# ----------------------------------------------------------------------------- autograd wiring
def test_autograd_wiring(ops):
    say("case: torch.autograd wiring of featurize and ani_charge")
    from khan_amd import autograd as kag
    b = datagen.make_batch("organic", 16, first_mol=100)
    c = Case.from_batch(b)
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    A = dev(c.A)
    X, Y, Z = (dev(v, np.float64).requires_grad_(True) for v in (c.X, c.Y, c.Z))
    w = torch.from_numpy(np.random.default_rng(3).standard_normal(c.N * 384)).to("cuda:0")
    feats = kag.featurize(X, Y, Z, A, mos, macs, sc, acs)
    loss = (torch.cat(feats) * w).sum()
    loss.backward()
    wb, start = [], 0
    for k in acs.tolist():
        wb.append(w[start * 384:(start + k) * 384])
        start += k
    gx, gy, gz = ops.featurize_grad(X.detach(), Y.detach(), Z.detach(), A, mos, macs, sc, acs, *wb)
    # (the float64 kernels add forces with atomics, so two runs differ in the last bits)
    same = lambda a, b: torch.allclose(a, b, rtol=1e-11, atol=1e-11)
    assert same(X.grad, gx) and same(Y.grad, gy) and same(Z.grad, gz)
    # central difference of the loss along one random direction, float64
    rng = np.random.default_rng(5)
    d = [dev(rng.standard_normal(c.N)) for _ in range(3)]
    h = 1e-5

    def L(s):
        f = ops.featurize(X.detach() + s * d[0], Y.detach() + s * d[1], Z.detach() + s * d[2], A, mos, macs, sc, acs)
        return float((torch.cat(f) * w).sum())
    num = (L(h) - L(-h)) / (2 * h)
    ana = float((gx * d[0]).sum() + (gy * d[1]).sum() + (gz * d[2]).sum())
    say("   directional derivative: numeric %.10e analytic %.10e" % (num, ana))
    assert abs(num - ana) <= 1e-6 * max(1.0, abs(ana))

    q = dev(datagen.charges(c.N).astype(np.float64)).requires_grad_(True)
    X2, Y2, Z2 = (dev(v, np.float64).requires_grad_(True) for v in (c.X, c.Y, c.Z))
    gm = dev(np.random.default_rng(6).standard_normal(c.n_mols))
    (kag.ani_charge(X2, Y2, Z2, q, mos, macs) * gm).sum().backward()
    qg, cx, cy, cz = ops.ani_charge_grad_xyz(X2.detach(), Y2.detach(), Z2.detach(), q.detach(), mos, macs, gm)
    assert same(q.grad, qg) and same(X2.grad, cx) and same(Y2.grad, cy) and same(Z2.grad, cz)
    # only the charges need a gradient: the reference's own wiring
    q3 = q.detach().clone().requires_grad_(True)
    (kag.ani_charge(X2.detach(), Y2.detach(), Z2.detach(), q3, mos, macs) * gm).sum().backward()
    assert same(q3.grad, qg)


# ----------------------------------------------------------------------------- grad-inverse (Jacobian . v)
def _check_grad_inverse(ops, c, seed=23):
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    v = np.random.default_rng(seed).standard_normal((c.N, 3)).astype(np.float32).astype(np.float64)
    ref = ob.gather_rows(ob.featurize_grad_inverse(c.X, c.Y, c.Z, c.A, c.MOs, c.MACs, c.sc, c.ac,
                                                    v[:, 0], v[:, 1], v[:, 2]), c.ga)
    S = mol_scale(ref, c.MOs, c.MACs)
    A = dev(c.A)
    for ndt, rtol, atol in ((np.float32, F32_RTOL, F32_ATOL), (np.float64, F64_RTOL, 0.0)):
        X, Y, Z = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
        out = ops.featurize_grad_inverse(X, Y, Z, A, mos, macs, sc, acs, dev(v[:, 0], ndt), dev(v[:, 1], ndt), dev(v[:, 2], ndt))
        rows = host(torch.cat(out).view(-1, 384)[ga.long()])
        assert_close("grad-inverse %s vs f64 oracle" % ndt.__name__, rows, ref, rtol, atol, scale=S)
    return X, Y, Z, A, mos, macs, sc, acs


def test_grad_inverse_organic_and_boxes(ops):
    say("case: featurize_grad_inverse, organic 256 molecules / 2 boxes / fixture")
    _check_grad_inverse(ops, Case.from_batch(datagen.make_batch("organic", 256)))
    _check_grad_inverse(ops, Case.from_batch(datagen.make_batch("boxes", 2)))
    x, y, z, a, mi = helpers.fixture11()
    _check_grad_inverse(ops, Case(x, y, z, a, mi, 2))


@pytest.mark.parametrize("kind,n_mols,first", [("organic", 512, 2000), ("boxes", 3, 40)])
def test_grad_inverse_adjoint_identity_and_uniform_vector(ops, kind, n_mols, first):
    # on the device, in float64: <u, J v> = <J^T u, v> with J^T u from featurize_grad, and J applied to a
    # uniform vector (the reference's only test input, test_kernel.py:363-400) is zero; the boxes go through the
    # workgroup-per-molecule kernels on both sides
    say("case: featurize_grad_inverse adjoint identity, %d %s molecules" % (n_mols, kind))
    c = Case.from_batch(datagen.make_batch(kind, n_mols, first_mol=first))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    X, Y, Z, A = dev(c.X, np.float64), dev(c.Y, np.float64), dev(c.Z, np.float64), dev(c.A)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(5)
    v = [torch.randn(c.N, dtype=torch.float64, device="cuda:0", generator=gen) for _ in range(3)]
    u = torch.randn(c.N * 384, dtype=torch.float64, device="cuda:0", generator=gen)
    ub, start = [], 0
    for k in acs.tolist():
        ub.append(u[start * 384:(start + k) * 384])
        start += k
    Jv = torch.cat(ops.featurize_grad_inverse(X, Y, Z, A, mos, macs, sc, acs, *v))
    JTu = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *ub)
    lhs = float((u * Jv).sum())
    rhs = float(sum((a * b).sum() for a, b in zip(JTu, v)))
    say("   <u,Jv> = %.12e   <J^T u,v> = %.12e" % (lhs, rhs))
    assert abs(lhs - rhs) <= 1e-10 * max(abs(lhs), abs(rhs))
    one, zero = torch.ones(c.N, dtype=torch.float64, device="cuda:0"), torch.zeros(c.N, dtype=torch.float64, device="cuda:0")
    J1 = torch.cat(ops.featurize_grad_inverse(X, Y, Z, A, mos, macs, sc, acs, one, zero, zero))
    assert float(J1.abs().max()) < 1e-11


def test_autograd_second_order_wiring(ops):
    # gradient of a function of the coordinate gradient with respect to the upstream weights goes
    # through featurize_grad_inverse (trainer_multi_tower.py:64-91)
    say("case: torch.autograd double backward through featurize")
    from khan_amd import autograd as kag
    c = Case.from_batch(datagen.make_batch("organic", 8, first_mol=300))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    A = dev(c.A)
    X, Y, Z = (dev(t, np.float64).requires_grad_(True) for t in (c.X, c.Y, c.Z))
    w = torch.from_numpy(np.random.default_rng(3).standard_normal(c.N * 384)).to("cuda:0").requires_grad_(True)
    energy = (torch.cat(kag.featurize(X, Y, Z, A, mos, macs, sc, acs)) * w).sum()
    fx, fy, fz = torch.autograd.grad(energy, (X, Y, Z), create_graph=True)
    a = [dev(np.random.default_rng(k).standard_normal(c.N)) for k in (7, 8, 9)]
    force_loss = (fx * a[0]).sum() + (fy * a[1]).sum() + (fz * a[2]).sum()
    (dw,) = torch.autograd.grad(force_loss, (w,))
    want = torch.cat(ops.featurize_grad_inverse(X.detach(), Y.detach(), Z.detach(), A, mos, macs, sc, acs, *a))
    assert torch.allclose(dw, want, rtol=1e-11, atol=1e-11)


# ----------------------------------------------------------------------------- the other full-size configurations
def _property_checks(ops, c, ndt, grad_rtol):
    """forward + backward of a whole batch on the device; returns rows (atom order) and gradients."""
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    assert np.array_equal(host(sc), c.sc) and np.array_equal(host(ga), c.ga) and np.array_equal(host(ac), c.ac)
    acs = ac.cpu()
    tdt = torch.float32 if ndt == np.float32 else torch.float64
    X, Y, Z, A = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt), dev(c.A)
    f = ops.featurize(X, Y, Z, A, mos, macs, sc, acs)
    rows = torch.cat(f).view(-1, 384)[ga.long()]
    assert bool(torch.isfinite(rows).all()) and float(rows.min()) >= 0.0
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(77)
    up = torch.randn(c.N, 384, dtype=tdt, device="cuda:0", generator=gen)
    inv = torch.empty_like(ga.long())
    inv[ga.long()] = torch.arange(c.N, device="cuda:0")
    upb_all = up[inv]
    gb, start = [], 0
    for k in acs.tolist():
        gb.append(upb_all[start:start + k].reshape(-1))
        start += k
    gx, gy, gz = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *gb)
    g = torch.stack([gx, gy, gz], dim=1)
    assert bool(torch.isfinite(g).all())
    seg = torch.from_numpy(c.mol_idxs.astype(np.int64)).to("cuda:0")
    net = torch.zeros(c.n_mols, 3, device="cuda:0", dtype=torch.float64).index_add_(0, seg, g.double())
    mag = torch.zeros(c.n_mols, 3, device="cuda:0", dtype=torch.float64).index_add_(0, seg, g.double().abs())
    rel = (net.abs() / (mag + 1e-30)).max().item()
    say("   net force / sum |force| per molecule, worst %.3e" % rel)
    assert rel < grad_rtol
    # radial symmetry: sum over centres of type a of their [partner type b] block = the same with a, b swapped
    # (every unordered pair is counted once from each side), per molecule-independent global sums
    types = torch.from_numpy(np.minimum(c.A, 3).astype(np.int64)).to("cuda:0")
    rad = rows[:, :64].double().view(-1, 4, 16)
    S = torch.zeros(4, 4, 16, dtype=torch.float64, device="cuda:0").index_add_(0, types, rad)
    sym = float((S - S.transpose(0, 1)).abs().max() / S.abs().max())
    say("   radial block symmetry, relative %.3e" % sym)
    assert sym < (1e-5 if ndt == np.float32 else 1e-12)
    return rows, g, up


def test_full_size_double_precision_configuration(ops):
    # 16,384 molecules in float64 with the charge kernels: properties at full size, the oracle on both ends
    say("case: organic 16384 float64 + charges, full size")
    M = 16384
    b = datagen.make_batch("organic", M)
    c = Case.from_batch(b)
    rows, g, up = _property_checks(ops, c, np.float64, 1e-11)
    for first, cnt in ((0, 128), (M - 128, 128)):
        sb = datagen.make_batch("organic", cnt, first_mol=first)
        sc_ = Case.from_batch(sb)
        a0 = int(c.MOs[first])
        ref64 = ob.gather_rows(sc_.oracle_feat(np.float64), sc_.ga)
        assert_close("rows of molecules %d.. f64" % first, host(rows[a0:a0 + sb.n_atoms]), ref64, F64_RTOL, F64_ATOL)
        upb = ob.scatter_rows(host(up[a0:a0 + sb.n_atoms]), sb.A, sc_.sc, sc_.ac)
        g64 = sc_.oracle_grad(upb)
        assert_close("gradient of molecules %d.. f64" % first, host(g[a0:a0 + sb.n_atoms]), g64, F64_RTOL, 0.0,
                     scale=mol_scale(g64, sc_.MOs, sc_.MACs))
    # charges at full size: Euler identity and zero net force per molecule, oracle on the first 256 molecules
    q = datagen.charges(b.n_atoms).astype(np.float64)
    X, Y, Z, Q = dev(b.X, np.float64), dev(b.Y, np.float64), dev(b.Z, np.float64), dev(q)
    mos, macs = dev(b.MOs), dev(b.MACs)
    ones = torch.ones(M, dtype=torch.float64, device="cuda:0")
    E = ops.ani_charge(X, Y, Z, Q, mos, macs)
    qg, cx, cy, cz = ops.ani_charge_grad_xyz(X, Y, Z, Q, mos, macs, ones)
    seg = torch.from_numpy(b.mol_idxs.astype(np.int64)).to("cuda:0")
    euler = 0.5 * torch.zeros(M, dtype=torch.float64, device="cuda:0").index_add_(0, seg, Q * qg)
    Eabs = ops.ani_charge(X, Y, Z, Q.abs(), mos, macs)
    assert float(((euler - E).abs() / (Eabs + 1e-300)).max()) < 1e-11
    net = torch.zeros(M, 3, dtype=torch.float64, device="cuda:0").index_add_(0, seg, torch.stack([cx, cy, cz], 1))
    mag = torch.zeros(M, 3, dtype=torch.float64, device="cuda:0").index_add_(0, seg, torch.stack([cx, cy, cz], 1).abs())
    assert float((net.abs() / (mag + 1e-300)).max()) < 1e-10
    n256 = int(b.MOs[256])
    E64 = ob.ani_charge(b.X[:n256], b.Y[:n256], b.Z[:n256], q[:n256], b.MOs[:256], b.MACs[:256], dtype=np.float64)
    Ea = host(Eabs)[:256]
    assert_close("charge energy, first 256 molecules", host(E)[:256], E64, F64_RTOL, 0.0, scale=Ea)
    # the oracle on 1,024 molecules taken at a stride through the batch: features, gradients, and the charge
    # energy with its derivatives by charge and by coordinate
    ids = strided_molecules(M, 1024, block=4)
    sub, idx = check_sample_against_oracle("1024 molecules at a stride, f64", c, ids, rows, g, up, F64_RTOL, F64_ATOL, 0.0)
    qs = q[idx]
    ones_s = np.ones(sub.n_mols)
    E_ref = ob.ani_charge(sub.X, sub.Y, sub.Z, qs, sub.MOs, sub.MACs, dtype=np.float64)
    dq_ref = ob.ani_charge_grad(sub.X, sub.Y, sub.Z, qs, sub.MOs, sub.MACs, ones_s, dtype=np.float64)
    dxyz_ref = np.stack(ob.ani_charge_grad_xyz(sub.X, sub.Y, sub.Z, qs, sub.MOs, sub.MACs, ones_s, dtype=np.float64), axis=1)
    # sums of terms of both signs, scaled as in test_charges: the energy by the same sum over |q|, the derivatives by
    # their largest component in the molecule
    Ea_s = ob.ani_charge(sub.X, sub.Y, sub.Z, np.abs(qs), sub.MOs, sub.MACs, dtype=np.float64)
    it = torch.from_numpy(idx).to("cuda:0")
    assert_close("charge energy, 1024 molecules at a stride", host(E)[ids], E_ref, F64_RTOL, 0.0, scale=Ea_s)
    assert_close("dE/dq, 1024 molecules at a stride", host(qg[it]), dq_ref, F64_RTOL, 0.0, scale=mol_scale(dq_ref, sub.MOs, sub.MACs))
    got_xyz = host(torch.stack([cx, cy, cz], 1)[it])
    assert_close("dE/dxyz, 1024 molecules at a stride", got_xyz, dxyz_ref, F64_RTOL, 0.0, scale=mol_scale(dxyz_ref, sub.MOs, sub.MACs))


def test_full_size_dense_boxes_configuration(ops):
    # 4,096 boxes of 64..256 atoms in float32: properties at full size, the oracle on the first and last boxes
    say("case: boxes 4096 float32, full size")
    M = 4096
    b = datagen.make_batch("boxes", M)
    c = Case.from_batch(b)
    rows, g, up = _property_checks(ops, c, np.float32, 2e-5)
    for first, cnt in ((0, 3), (M - 3, 3)):
        sb = datagen.make_batch("boxes", cnt, first_mol=first)
        sc_ = Case.from_batch(sb)
        a0 = int(c.MOs[first])
        assert np.array_equal(sb.X, c.X[a0:a0 + sb.n_atoms])
        ref64 = ob.gather_rows(sc_.oracle_feat(np.float64), sc_.ga)
        assert_close("rows of boxes %d.. vs f64 oracle" % first, host(rows[a0:a0 + sb.n_atoms]), ref64, F32_RTOL, F32_ATOL)
        upb = ob.scatter_rows(host(up[a0:a0 + sb.n_atoms]).astype(np.float64), sb.A, sc_.sc, sc_.ac)
        g64 = sc_.oracle_grad(upb)
        assert_close("gradient of boxes %d.. vs f64 oracle" % first, host(g[a0:a0 + sb.n_atoms]), g64,
                     F32_RTOL, F32_ATOL, scale=mol_scale(g64, sc_.MOs, sc_.MACs))
    # the oracle on 128 boxes taken at a stride through the batch (float32 launch above), and 32 of them through the
    # float64 kernels as a batch of their own
    ids = strided_molecules(M, 128)
    check_sample_against_oracle("128 boxes at a stride", c, ids, rows, g, up, F32_RTOL, F32_ATOL, F32_ATOL)
    sub, _ = sample_case(c, ids[::4])
    say("   32 boxes in float64: %d atoms" % sub.N)
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, sub)
    acs = ac.cpu()
    Xd, Yd, Zd = dev(sub.X, np.float64), dev(sub.Y, np.float64), dev(sub.Z, np.float64)
    f = ops.featurize(Xd, Yd, Zd, dev(sub.A), mos, macs, sc, acs)
    assert_close("features f64, 32 boxes", host(torch.cat(f)), np.concatenate(sub.oracle_feat(np.float64)), F64_RTOL, F64_ATOL)
    upb = sub.upstream()
    gx, gy, gz = ops.featurize_grad(Xd, Yd, Zd, dev(sub.A), mos, macs, sc, acs, *[dev(u) for u in upb])
    g64 = sub.oracle_grad(upb)
    assert_close("gradient f64, 32 boxes", host(torch.stack([gx, gy, gz], 1)), g64, F64_RTOL, 0.0,
                 scale=mol_scale(g64, sub.MOs, sub.MACs))


def test_gradient_against_central_differences_on_64_molecules(ops):
    # the backward pass against a central difference of the float64 forward pass, h = 1e-4 A, on 64 molecules:
    # directional derivatives along 8 random directions
    say("case: central differences of the float64 forward, 64 molecules")
    c = Case.from_batch(datagen.make_batch("organic", 64, first_mol=500))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    A = dev(c.A)
    X, Y, Z = dev(c.X, np.float64), dev(c.Y, np.float64), dev(c.Z, np.float64)
    rng = np.random.default_rng(8)
    w = dev(rng.standard_normal(c.N * 384))
    wb, start = [], 0
    for k in acs.tolist():
        wb.append(w[start * 384:(start + k) * 384])
        start += k
    g64 = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *wb)
    g32 = ops.featurize_grad(X.float(), Y.float(), Z.float(), A, mos, macs, sc, acs, *[t.float() for t in wb])
    h = 1e-4
    for trial in range(8):
        d = [dev(rng.standard_normal(c.N)) for _ in range(3)]
        Lp = float((torch.cat(ops.featurize(X + h * d[0], Y + h * d[1], Z + h * d[2], A, mos, macs, sc, acs)) * w).sum())
        Lm = float((torch.cat(ops.featurize(X - h * d[0], Y - h * d[1], Z - h * d[2], A, mos, macs, sc, acs)) * w).sum())
        num = (Lp - Lm) / (2 * h)
        ana64 = float(sum((a * b_).sum() for a, b_ in zip(g64, d)))
        ana32 = float(sum((a.double() * b_).sum() for a, b_ in zip(g32, d)))
        scale = float(sum((a.abs() * b_.abs()).sum() for a, b_ in zip(g64, d)))
        say("   direction %d: numeric %.9e  f64 %.9e  f32 %.9e" % (trial, num, ana64, ana32))
        assert abs(num - ana64) <= 1e-6 * scale      # truncation of the difference quotient, O(h^2)
        assert abs(ana32 - ana64) <= 1e-5 * scale



def test_radial_gradient_at_every_distance(ops):
    """The float32 backward kernels sum the radial shells nearest to the pair's distance only (nine of sixteen): pairs
    at 240 distances from 0.04 A to beyond the cutoff, alone (one-wavefront kernel) and inside a 70-atom molecule
    whose other atoms are out of reach (workgroup-per-molecule kernel), against the float64 oracle, which sums all
    sixteen.  Also a third atom at an angle, so that the window edges are met together with angular terms."""
    say("case: pair distances 0.04 .. 4.7 A, float32 radial window against the oracle's full sum")
    rng = np.random.default_rng(21)
    dists = np.concatenate([np.linspace(0.04, 4.7, 200), 0.5 + 0.25625 * (np.arange(16) + 0.5), 0.5 + 0.25625 * np.arange(16),
                            [4.5999, 4.6, 4.6001, 3.0999, 3.1, 3.1001, 1e-3, 2e-2]])
    mols = []
    for k, d in enumerate(dists):
        u = rng.standard_normal(3)
        u /= np.linalg.norm(u)
        t = rng.integers(0, 4, 3)
        v = np.cross(u, rng.standard_normal(3))
        v /= np.linalg.norm(v)
        third = 0.8 * d * (0.3 * u + 0.95 * v) + 1e-3
        mols.append((t.astype(np.int32), np.stack([np.zeros(3), d * u, third])))            # 3 atoms
        if k % 4 == 0:                                                                       # the same pair in a large molecule
            far = np.stack([np.array([20.0 + 12.0 * (i % 8), 12.0 * (i // 8), 40.0]) for i in range(67)])
            mols.append((np.concatenate([t, rng.integers(0, 4, 67)]).astype(np.int32),
                         np.concatenate([np.stack([np.zeros(3), d * u, third]), far])))
    A = np.concatenate([m[0] for m in mols])
    xyz = np.concatenate([m[1] for m in mols])
    mol_idxs = np.concatenate([np.full(len(m[0]), i, dtype=np.int32) for i, m in enumerate(mols)])
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mol_idxs, len(mols))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    upb = c.upstream(seed=22)
    g64 = c.oracle_grad(upb)
    assert np.all(np.isfinite(g64))
    S = mol_scale(g64, c.MOs, c.MACs)
    Ad = dev(c.A)
    for tdt, ndt, rtol, atol in ((torch.float32, np.float32, F32_RTOL, F32_ATOL), (torch.float64, np.float64, F64_RTOL, 0.0)):
        X, Y, Z = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
        gx, gy, gz = ops.featurize_grad(X, Y, Z, Ad, mos, macs, sc, acs, *[dev(x, ndt) for x in upb])
        gg = host(torch.stack([gx, gy, gz], dim=1))
        assert_close("gradient %s, %d molecules" % (np.dtype(ndt).name, len(mols)), gg, g64, rtol, atol, scale=S)
        # the forces of a molecule add up to nothing (sum over a molecule of mixed-sign components: on its scale)
        for m in range(0, len(mols), 37):
            s_ = slice(c.MOs[m], c.MOs[m] + c.MACs[m])
            assert np.abs(gg[s_].sum(axis=0)).max() <= (2e-5 if ndt == np.float32 else 1e-11) * max(float(S[c.MOs[m]].max()), 1e-30)


def _ratio_quantiles(name, got, ref, rtol, atol):
    """Per-element |got - ref| / (atol + rtol |ref|) -- the tolerance taken component by component, every component on
    its own -- as quantiles; non-finite entries of `got` are left out and counted."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    ok = np.isfinite(got)
    ratio = np.abs(got[ok] - ref[ok]) / (atol + rtol * np.abs(ref[ok]))
    qs = [float(np.quantile(ratio, q)) for q in (0.5, 0.9, 0.99, 0.999)] + [float(ratio.max())]
    say("   %-46s non-finite %5d   err/(atol+rtol|ref|): median %.3g  90%% %.3g  99%% %.3g  99.9%% %.3g  max %.3g"
        % (name, int((~np.isfinite(got)).sum()), *qs))
    return qs


def test_gradient_error_per_element_beside_the_references_own_functor(ops):
    """How much the per-molecule scale in the gradient tolerance relaxes a per-element reading of the same tolerance
    (float32 1e-5 relative / 1e-6 absolute; float64 1e-12 relative), measured: the per-element error ratio of
    the HIP gradients against the float64 oracle, beside the same ratio for the reference's own functor
    (gpu_featurizer/kernel_cpu.cpp:217-366 compiled in place, float32 and float64, finite entries only).  A
    gradient component is a sum of terms of both signs, so its error is set by the size of the terms, not of
    the sum; the bar here is that the HIP kernels are at least as close to the float64 oracle as the reference's
    functor of the same precision, quantile by quantile, and that the worst per-element ratios stay where they
    were measured (stated in the assertions)."""
    say("case: per-element gradient error, HIP vs the reference's own functor, 256 organic molecules")
    c = Case.from_batch(datagen.make_batch("organic", 256))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu()
    upb = c.upstream()
    g64 = c.oracle_grad(upb)
    have_ref = ob.ref_lib(False) is not None
    impl = "ref" if have_ref else "oracle"
    say("   comparison functor: %s" % ("the reference's kernel_cpu.cpp compiled in place" if have_ref else
                                      "the oracle's restatement (oracle/_ref is not built)"))
    with np.errstate(all="ignore"):
        r32 = np.stack(ob.featurize_grad(c.X, c.Y, c.Z, c.A, c.MOs, c.MACs, c.sc, c.ac, upb, dtype=np.float32, impl=impl), axis=1)
        r64 = np.stack(ob.featurize_grad(c.X, c.Y, c.Z, c.A, c.MOs, c.MACs, c.sc, c.ac, upb, dtype=np.float64, impl=impl), axis=1)
    A = dev(c.A)
    out = {}
    for tdt, ndt in ((torch.float32, np.float32), (torch.float64, np.float64)):
        X, Y, Z = dev(c.X, ndt), dev(c.Y, ndt), dev(c.Z, ndt)
        gx, gy, gz = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *[dev(u, ndt) for u in upb])
        out[ndt] = host(torch.stack([gx, gy, gz], dim=1))
    q_hip32 = _ratio_quantiles("HIP float32 vs float64 oracle", out[np.float32], g64, F32_RTOL, F32_ATOL)
    q_ref32 = _ratio_quantiles("reference float32 functor vs float64 oracle", r32, g64, F32_RTOL, F32_ATOL)
    q_hip64 = _ratio_quantiles("HIP float64 vs float64 oracle", out[np.float64], g64, F64_RTOL, F64_ATOL)
    q_ref64 = _ratio_quantiles("reference float64 functor vs float64 oracle", r64, g64, F64_RTOL, F64_ATOL)
    assert np.all(np.isfinite(out[np.float32])) and np.all(np.isfinite(out[np.float64]))
    # the same comparison on the scale the other tests use (largest component of the molecule)
    S = mol_scale(g64, c.MOs, c.MACs) + np.zeros_like(g64)
    for name, got, rtol, atol in (("HIP float32", out[np.float32], F32_RTOL, F32_ATOL), ("reference float32", r32, F32_RTOL, F32_ATOL),
                                  ("HIP float64", out[np.float64], F64_RTOL, 0.0), ("reference float64", r64, F64_RTOL, 0.0)):
        ok = np.isfinite(got)
        worst = (np.abs(got - g64)[ok] / (atol + rtol * np.maximum(np.abs(g64), S))[ok]).max()
        say("   %-46s worst err/bound on the molecule's scale: %.3g" % (name, worst))
    # at least as close to the float64 oracle as the reference's functor of the same precision, at the median, the
    # 90th, 99th and 99.9th percentile and at the worst element
    for k in range(5):
        assert q_hip32[k] <= q_ref32[k], ("float32 quantile", k, q_hip32, q_ref32)
        assert q_hip64[k] <= q_ref64[k], ("float64 quantile", k, q_hip64, q_ref64)
    # worst per-element ratios: 1.5 times what was measured (13.1 in float32, 2.4 in float64 on 1,024 molecules; 10.8 and
    # 1.2 on these 256: cancelling components); a regression
    # in the kernels moves these
    assert q_hip32[4] <= 20.0 and q_hip64[4] <= 4.0, (q_hip32, q_hip64)


# ----------------------------------------------------------------------------- HIP graph capture
def test_forward_backward_replay_from_a_hip_graph(ops):
    # featurize + featurize_grad launch only kernels on the caller's stream (no allocation, no memset node,
    # no host synchronisation), so they can be captured once and replayed; every replay is checked against
    # the eager result, with eager work and synchronisations in between
    say("case: HIP graph capture and replay of forward + backward")
    # enough molecules for the eager calls to take the size order (which they allocate, so they go without it under
    # capture); the captured calls are given a caller-owned order and must produce the same rows
    b = datagen.make_batch("organic", 2100, first_mol=900)
    big = datagen.make_batch("boxes", 2)               # brings the medium-molecule kernels into the graph
    X = np.concatenate([b.X, big.X]); Y = np.concatenate([b.Y, big.Y]); Z = np.concatenate([b.Z, big.Z])
    A = np.concatenate([b.A, big.A])
    mi = np.concatenate([b.mol_idxs, big.mol_idxs + b.n_mols]).astype(np.int32)
    c = Case(X, Y, Z, A, mi, b.n_mols + big.n_mols)
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu().tolist()
    Xd, Yd, Zd, Ad = dev(c.X), dev(c.Y), dev(c.Z), dev(c.A)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(3)
    up = torch.randn(c.N * 384, device="cuda:0", generator=gen)
    gb, start = [], 0
    for k in acs:
        gb.append(up[start * 384:(start + k) * 384])
        start += k
    feats = torch.cat(ops.featurize(Xd, Yd, Zd, Ad, mos, macs, sc, acs)).clone()
    grads = torch.stack(ops.featurize_grad(Xd, Yd, Zd, Ad, mos, macs, sc, acs, *gb)).clone()
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up on the capture stream
        ops.featurize(Xd, Yd, Zd, Ad, mos, macs, sc, acs)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        # with a caller-owned size order the captured launches walk the molecules largest first, as eager calls do;
        # the order itself is part of the graph (kernels only: its counts are cleared by a kernel, not a memset node)
        order = ops.size_order(macs)
        f_out = ops.featurize(Xd, Yd, Zd, Ad, mos, macs, sc, acs, order=order)
        g_out = ops.featurize_grad(Xd, Yd, Zd, Ad, mos, macs, sc, acs, *gb, order=order)
    f_cat = lambda: torch.cat(f_out)
    for replay in range(4):
        order.zero_()                                  # a stale order would send every workgroup to molecule 0
        for t in f_out:
            t.fill_(-1.0)                              # eager work between replays
        for t in g_out:
            t.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(f_cat(), feats), "replay %d: features differ" % replay
        got = torch.stack(list(g_out))
        # molecules above 64 atoms add forces with atomics: the last bits depend on the order
        assert torch.allclose(got, grads, rtol=1e-5, atol=1e-5), "replay %d: gradients differ" % replay
        small = torch.from_numpy(c.mol_idxs < b.n_mols).to("cuda:0")
        assert torch.equal(got[:, small], grads[:, small])


def test_upstream_buckets_without_16_byte_alignment(ops):
    # the fast backward kernels read upstream rows in 16-byte pieces; buckets at an odd float offset must
    # still give the same gradients (they are routed to the general kernel)
    say("case: upstream gradient buckets at a 4-byte-aligned address")
    c = Case.from_batch(datagen.make_batch("organic", 64, first_mol=1200))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu().tolist()
    X, Y, Z, A = dev(c.X), dev(c.Y), dev(c.Z), dev(c.A)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(9)
    up = torch.randn(c.N * 384, device="cuda:0", generator=gen)
    aligned, shifted, start = [], [], 0
    store = torch.empty(c.N * 384 + 8, device="cuda:0")
    for k in acs:
        seg = up[start * 384:(start + k) * 384]
        aligned.append(seg)
        off = start * 384 + 1                       # one float off a 16-byte boundary
        store[off:off + k * 384] = seg
        shifted.append(store[off:off + k * 384])
        start += k
    assert any(t.data_ptr() % 16 != 0 for t in shifted if t.numel())
    ga_ = torch.stack(ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *aligned))
    gs_ = torch.stack(ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *shifted))
    scale = float(ga_.abs().max())
    assert float((ga_ - gs_).abs().max()) <= 2e-5 * scale


def test_linear_molecules_give_finite_gradients(ops):
    # exactly collinear triples: the angle has a cusp there and the reference's derivative is 0/0.  The
    # kernels return finite gradients: zero across the axis (by symmetry) and the derivative of the smooth
    # dependence along the axis, checked against central differences of the forward pass
    say("case: exactly linear molecules, both precisions, every kernel (one wavefront, one workgroup, general)")
    mols = [
        (np.array([3, 1, 3]), np.array([[0, 0, -1.16], [0, 0, 0.0], [0, 0, 1.16]])),            # CO2 on the z axis
        (np.array([0, 1, 2]), np.array([[0, 0, 0.0], [0, 0, 1.06], [0, 0, 2.21]])),             # HCN
        (np.array([0, 1, 1, 0]), np.array([[-1.66, 0, 0], [-0.6, 0, 0], [0.6, 0, 0], [1.66, 0, 0]])),   # acetylene on x
    ]
    # straight chains on the y axis, unevenly spaced: 40 atoms (one workgroup in float32), 100 (one workgroup in
    # both precisions) and 300 (the general-shape kernel)
    crng = np.random.default_rng(31)
    for n_chain in (40, 100, 300):
        pos = np.cumsum(crng.uniform(0.95, 1.4, n_chain))
        mols.append((crng.integers(0, 4, n_chain), np.stack([np.zeros(n_chain), pos, np.zeros(n_chain)], axis=1)))
    A = np.concatenate([m[0] for m in mols]).astype(np.int32)
    xyz = np.concatenate([m[1] for m in mols]).astype(np.float64)
    mi = np.concatenate([np.full(len(m[0]), k) for k, m in enumerate(mols)]).astype(np.int32)
    c = Case(xyz[:, 0], xyz[:, 1], xyz[:, 2], A, mi, len(mols))
    macs, mos, sc, ga, ac = gpu_sort_offsets(ops, c)
    acs = ac.cpu().tolist()
    rng = np.random.default_rng(12)
    w = dev(rng.standard_normal(c.N * 384))
    wb, start = [], 0
    for k in acs:
        wb.append(w[start * 384:(start + k) * 384])
        start += k
    Ad = dev(c.A)
    axis = np.array([2, 2, 2, 2, 2, 2, 0, 0, 0, 0] + [1] * 440)     # the molecule's axis per atom
    for ndt, tol in ((np.float64, 1e-7), (np.float32, 2e-3)):
        X, Y, Z = dev(xyz[:, 0], ndt), dev(xyz[:, 1], ndt), dev(xyz[:, 2], ndt)
        wl = [t.to(X.dtype) for t in wb]
        g = torch.stack(ops.featurize_grad(X, Y, Z, Ad, mos, macs, sc, acs, *wl), dim=1).double().cpu().numpy()
        assert np.all(np.isfinite(g))
        scale = np.abs(g).max()
        for a in range(c.N):
            perp = [k for k in range(3) if k != axis[a]]
            assert np.abs(g[a, perp]).max() <= 1e-6 * scale, (a, g[a])
        if ndt == np.float64:
            # along the axis: central differences of the float64 forward
            h = 1e-5
            coords = [X, Y, Z]
            for a in range(c.N):
                k = int(axis[a])
                plus = [t.clone() for t in coords]
                minus = [t.clone() for t in coords]
                plus[k][a] += h
                minus[k][a] -= h
                Lp = float((torch.cat(ops.featurize(*plus, Ad, mos, macs, sc, acs)) * w).sum())
                Lm = float((torch.cat(ops.featurize(*minus, Ad, mos, macs, sc, acs)) * w).sum())
                assert abs((Lp - Lm) / (2 * h) - g[a, k]) <= tol * scale, (a, (Lp - Lm) / (2 * h), g[a, k])
