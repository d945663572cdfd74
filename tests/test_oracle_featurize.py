"""Pins the forward and backward AEV oracle without a GPU.

  * committed golden vectors written from the compiled reference (tests/golden/make_golden.py)
  * the compiled reference itself (oracle/_ref), bit for bit, where it is built
  * an independent brute-force closed form (the construction of the reference's own python check,
    gpu_featurizer/test_kernel.py:147-255) at the reference's tolerance, decimal=6
  * what the mathematics fixes: hand values for a diatomic and a right-angle triatomic, rotation /
    translation / permutation invariance, central finite differences of the forward for the gradient
    (the reference checks d(features)/dx numerically with delta=1e-6, tol 1e-9 in double,
    test_kernel.py:473-535), zero net force and torque.
"""
import math
import os

import numpy as np
import pytest

import helpers
from khan_amd import datagen
from oracle import binding as ob


@pytest.fixture(scope="module")
def golden(golden_dir):
    return np.load(os.path.join(golden_dir, "aev_golden.npz"))


def _run_case(g, prefix, dtype, impl="oracle"):
    X, Y, Z = g[prefix + "_X"], g[prefix + "_Y"], g[prefix + "_Z"]
    A, sc, ga, ac = g[prefix + "_A"], g[prefix + "_scatter"], g[prefix + "_gather"], g[prefix + "_counts"]
    macs, mos = g[prefix + "_macs"], g[prefix + "_mos"]
    f = ob.featurize(X, Y, Z, A, mos, macs, sc, ac, dtype=dtype, impl=impl)
    return ob.gather_rows(f, ga)


@pytest.mark.parametrize("prefix", ["fx11", "org8"])
def test_forward_matches_golden_bitwise(golden, prefix):
    # the oracle follows the reference's arithmetic operation by operation, so it reproduces the
    # compiled reference's output exactly, in both precisions
    for dtype, tag in ((np.float32, "f32"), (np.float64, "f64")):
        got = _run_case(golden, prefix, dtype)
        assert np.array_equal(got, golden[prefix + "_feat_" + tag])


@pytest.mark.skipif(not ob.have_ref(), reason="oracle/_ref not built (needs /root/reference)")
def test_forward_matches_compiled_reference_bitwise():
    b = datagen.make_batch("organic", 256)
    sc, ga, ac = ob.ani_sort(b.A)
    for dtype in (np.float32, np.float64):
        mine = ob.featurize(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, dtype=dtype)
        ref = ob.featurize(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, dtype=dtype, impl="ref")
        for m, r in zip(mine, ref):
            assert np.array_equal(m, r)


def test_forward_matches_brute_force_closed_form(golden):
    # reference tolerance: assert_almost_equal(decimal=6), test_kernel.py:340-347
    x, y, z, a, mi = helpers.fixture11()
    got = _run_case(golden, "fx11", np.float64)
    xyz = np.stack([x, y, z], axis=1)
    exp = np.concatenate([helpers.brute_force_aev(a[:8], xyz[:8]), helpers.brute_force_aev(a[8:], xyz[8:])])
    np.testing.assert_almost_equal(got, exp, decimal=6)
    assert np.abs(exp).max() > 0.5 and (exp[:, 64:] > 1e-3).sum() > 50    # both blocks are exercised
    # and on generator molecules, which contain O atoms (the fixture has none)
    b = datagen.make_batch("organic", 6)
    sc, ga, ac = ob.ani_sort(b.A)
    rows = ob.gather_rows(ob.featurize(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, dtype=np.float64), ga)
    xyz = np.stack([b.X, b.Y, b.Z], axis=1).astype(np.float64)
    for m in range(6):
        s = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
        np.testing.assert_almost_equal(rows[s], helpers.brute_force_aev(b.A[s], xyz[s]), decimal=6)


def _one_mol(types, xyz, dtype=np.float64):
    types = np.asarray(types, dtype=np.int32)
    xyz = np.asarray(xyz, dtype=np.float64)
    sc, ga, ac = ob.ani_sort(types)
    n = types.size
    f = ob.featurize(xyz[:, 0], xyz[:, 1], xyz[:, 2], types, np.array([0], np.int32), np.array([n], np.int32),
                     sc, ac, dtype=dtype)
    return ob.gather_rows(f, ga)


def test_single_atom_and_diatomic_hand_values():
    assert np.all(_one_mol([1], [[0.3, 0.2, 0.1]]) == 0)
    r = 1.1
    rows = _one_mol([1, 3], [[0, 0, 0], [0, 0, r]])
    fc = 0.5 * math.cos(math.pi * r / float(np.float32(4.6))) + 0.5
    # parameters are float-typed in the reference (parameters.h:66-114): use the rounded values
    exp = np.array([math.exp(-16.0 * (r - float(np.float32(rs))) ** 2) * fc for rs in helpers.R_RS])
    assert np.allclose(rows[0, 3 * 16:4 * 16], exp, rtol=1e-12, atol=0)      # C sees an O
    assert np.allclose(rows[1, 1 * 16:2 * 16], exp, rtol=1e-12, atol=0)      # O sees a C
    assert np.count_nonzero(rows[0]) == 16 and np.count_nonzero(rows[1]) == 16
    # beyond the radial cutoff nothing is produced; the cutoff is strict
    assert np.all(_one_mol([0, 0], [[0, 0, 0], [0, 0, 4.7]]) == 0)


def test_right_angle_triatomic_hand_value():
    # centre C at the origin, H on x and N on y at 1.0 and 1.2 A: theta = pi/2 exactly
    rows = _one_mol([1, 0, 2], [[0, 0, 0], [1.0, 0, 0], [0, 1.2, 0]])
    rc = float(np.float32(3.1))
    fc = lambda r: 0.5 * math.cos(math.pi * r / rc) + 0.5
    block = 64 + 32 * helpers.pair_block(0, 2)
    for t, th in enumerate(helpers.A_THETAS):
        for s, rs in enumerate(helpers.A_RS):
            th32, rs32 = float(np.float32(th)), float(np.float32(rs))
            exp = 2.0 ** -7 * (1 + math.cos(math.pi / 2 - th32)) ** 8 * math.exp(-6.0 * (1.1 - rs32) ** 2) * fc(1.0) * fc(1.2)
            assert rows[0, block + 4 * t + s] == pytest.approx(exp, rel=1e-12)
    others = np.delete(rows[0, 64:], np.arange(block - 64, block - 64 + 32))
    assert np.all(others == 0)


def test_rigid_motion_and_permutation_invariance():
    rng = np.random.default_rng(3)
    b = datagen.make_batch("organic", 4, first_mol=100)
    s = slice(b.MOs[2], b.MOs[2] + b.MACs[2])
    types, xyz = b.A[s], np.stack([b.X[s], b.Y[s], b.Z[s]], axis=1).astype(np.float64)
    base = _one_mol(types, xyz)
    moved = xyz @ helpers.random_rotation(rng).T + rng.standard_normal(3)
    assert np.allclose(_one_mol(types, moved), base, rtol=1e-9, atol=1e-12)
    perm = rng.permutation(len(types))
    assert np.allclose(_one_mol(types[perm], xyz[perm]), base[perm], rtol=1e-12, atol=1e-14)


def test_linearize_table():
    # kernel_cpu.cpp:9-23: HH0 HC1 HN2 HO3 CC4 CN5 CO6 NN7 NO8 OO9, symmetric in its arguments
    lib = ob.oracle_lib()
    for a in range(4):
        for c in range(4):
            assert lib.khan_oracle_pair_block(a, c) == helpers.pair_block(a, c)


# ------------------------------------------------------------------------------------ backward
def _grad_case(g, prefix, dtype, impl="oracle"):
    X, Y, Z = g[prefix + "_X"], g[prefix + "_Y"], g[prefix + "_Z"]
    A, sc, ac = g[prefix + "_A"], g[prefix + "_scatter"], g[prefix + "_counts"]
    up = ob.scatter_rows(g[prefix + "_upstream"].astype(dtype), A, sc, ac)
    gx, gy, gz = ob.featurize_grad(X, Y, Z, A, g[prefix + "_mos"], g[prefix + "_macs"], sc, ac, up, dtype=dtype, impl=impl)
    return np.stack([gx, gy, gz], axis=1)


@pytest.mark.parametrize("prefix", ["fx11", "org8"])
def test_backward_matches_golden_f64(golden, prefix):
    # reduced-form derivative vs the reference's expanded sympy expressions: agreement to rounding
    got = _grad_case(golden, prefix, np.float64)
    ref = golden[prefix + "_grad_f64"]
    scale = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-12 * scale


def test_reference_float_gradient_is_not_finite_everywhere(golden):
    # documents why float32 gradients are judged against the float64 oracle: the reference's float
    # functor divides 0 by 0 for theta_t - theta near +-pi (kernel_cpu.cpp:335)
    ref32 = golden["org8_grad_f32"]
    assert np.count_nonzero(~np.isfinite(ref32)) > 0
    got = _grad_case(golden, "org8", np.float32)
    assert np.all(np.isfinite(got))
    ok = np.isfinite(ref32)
    ref64 = golden["org8_grad_f64"]
    assert np.abs(got - ref64).max() <= 1e-4 * np.abs(ref64).max()
    assert np.abs(ref32[ok] - ref64[ok]).max() <= 1e-3 * np.abs(ref64).max()


def test_backward_central_differences_and_invariants():
    b = datagen.make_batch("organic", 3, first_mol=40)
    sc, ga, ac = ob.ani_sort(b.A)
    n = b.n_atoms
    up = np.random.default_rng(5).standard_normal((n, 384))
    g = ob.scatter_rows(up, b.A, sc, ac)
    xyz = [b.X.astype(np.float64), b.Y.astype(np.float64), b.Z.astype(np.float64)]
    grad = np.stack(ob.featurize_grad(*xyz, b.A, b.MOs, b.MACs, sc, ac, g, dtype=np.float64), axis=1)

    def loss(c):
        f = ob.featurize(c[0], c[1], c[2], b.A, b.MOs, b.MACs, sc, ac, dtype=np.float64)
        return float((ob.gather_rows(f, ga) * up).sum())

    h = 1e-4
    scale = np.abs(grad).max()
    for a in range(0, n, 3):
        for ax in range(3):
            cp = [v.copy() for v in xyz]
            cm = [v.copy() for v in xyz]
            cp[ax][a] += h
            cm[ax][a] -= h
            fd = (loss(cp) - loss(cm)) / (2 * h)
            assert abs(fd - grad[a, ax]) <= 2e-6 * scale, (a, ax, fd, grad[a, ax])
    # translation invariance -> zero net force; rotation invariance -> zero net torque, per molecule
    pos = np.stack(xyz, axis=1)
    for m in range(b.n_mols):
        s = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
        assert np.abs(grad[s].sum(axis=0)).max() <= 1e-11 * scale
        assert np.abs(np.cross(pos[s], grad[s]).sum(axis=0)).max() <= 1e-10 * scale


@pytest.mark.skipif(not ob.have_ref(), reason="oracle/_ref not built (needs /root/reference)")
def test_backward_matches_compiled_reference_f64():
    b = datagen.make_batch("organic", 24, first_mol=500)
    sc, ga, ac = ob.ani_sort(b.A)
    up = np.random.default_rng(6).standard_normal((b.n_atoms, 384))
    g = ob.scatter_rows(up, b.A, sc, ac)
    mine = np.stack(ob.featurize_grad(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, g, dtype=np.float64), axis=1)
    ref = np.stack(ob.featurize_grad(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, g, dtype=np.float64, impl="ref"), axis=1)
    assert np.abs(mine - ref).max() <= 1e-11 * np.abs(ref).max()


# ----------------------------------------------------------------------------- grad-inverse (Jacobian . v)
def _jvp_case(n_mols=12, first_mol=40):
    b = datagen.make_batch("organic", n_mols, first_mol=first_mol)
    sc, ga, ac = ob.ani_sort(b.A)
    rng = np.random.default_rng(17)
    v = rng.standard_normal((b.n_atoms, 3))
    return b, sc, ga, ac, v


def test_grad_inverse_is_the_adjoint_of_the_gradient():
    # <u, J v> = <J^T u, v>: J^T u is featurize_grad (pinned against the compiled reference above), so
    # this identity pins J v for arbitrary v; a wrong index, sign or dropped term breaks it
    b, sc, ga, ac, v = _jvp_case()
    rng = np.random.default_rng(3)
    u_rows = rng.standard_normal((b.n_atoms, 384))
    u = ob.scatter_rows(u_rows, b.A, sc, ac)
    Jv = ob.featurize_grad_inverse(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, v[:, 0], v[:, 1], v[:, 2])
    JTu = ob.featurize_grad(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, u)
    lhs = sum(float(np.dot(a.reshape(-1), c.reshape(-1))) for a, c in zip(u, Jv))
    rhs = float(np.dot(JTu[0], v[:, 0]) + np.dot(JTu[1], v[:, 1]) + np.dot(JTu[2], v[:, 2]))
    assert abs(lhs - rhs) <= 1e-11 * max(abs(lhs), abs(rhs), 1.0)
    # one molecule at a time as well, so that errors cannot cancel between molecules
    Jv_rows = ob.gather_rows(Jv, ga)
    for m in range(b.n_mols):
        s = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
        lhs = float((u_rows[s] * Jv_rows[s]).sum())
        rhs = float(sum(np.dot(JTu[k][s], v[s, k]) for k in range(3)))
        assert abs(lhs - rhs) <= 1e-11 * max(abs(lhs), abs(rhs), 1.0)


def test_grad_inverse_matches_central_differences_of_the_forward():
    b, sc, ga, ac, v = _jvp_case(n_mols=6)
    h = 1e-6
    X, Y, Z = (np.asarray(t, dtype=np.float64) for t in (b.X, b.Y, b.Z))
    fp = ob.featurize(X + h * v[:, 0], Y + h * v[:, 1], Z + h * v[:, 2], b.A, b.MOs, b.MACs, sc, ac, dtype=np.float64)
    fm = ob.featurize(X - h * v[:, 0], Y - h * v[:, 1], Z - h * v[:, 2], b.A, b.MOs, b.MACs, sc, ac, dtype=np.float64)
    num = [(p - m) / (2 * h) for p, m in zip(fp, fm)]
    Jv = ob.featurize_grad_inverse(X, Y, Z, b.A, b.MOs, b.MACs, sc, ac, v[:, 0], v[:, 1], v[:, 2])
    for a, n_ in zip(Jv, num):
        if a.size:
            assert np.max(np.abs(a - n_)) <= 2e-8 * max(1.0, float(np.max(np.abs(n_))))


def test_grad_inverse_uniform_vector_gives_zero_like_the_reference_test():
    # the reference's only check feeds dL/dx = 1, dL/dy = dL/dz = 0 for every atom (test_kernel.py:
    # 363-400): features are translation invariant, so the result is zero up to rounding
    b, sc, ga, ac, v = _jvp_case()
    one, zero = np.ones(b.n_atoms), np.zeros(b.n_atoms)
    Jv = ob.featurize_grad_inverse(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, one, zero, zero)
    assert max(float(np.max(np.abs(a))) for a in Jv if a.size) < 1e-12
    if ob.have_ref():
        ref = ob.featurize_grad_inverse(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, one, zero, zero, impl="ref")
        assert max(float(np.max(np.abs(a))) for a in ref if a.size) < 1e-9
        # and the reference returns (numerically) zero for ANY input, because it reads the vectors
        # by atomic number of the centre for all three atoms of a term (kernel_cpu.cpp:111-169)
        ref2 = ob.featurize_grad_inverse(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, v[:, 0], v[:, 1], v[:, 2], impl="ref")
        assert max(float(np.max(np.abs(a))) for a in ref2 if a.size) < 1e-9


def test_grad_inverse_float32_oracle_close_to_float64():
    b, sc, ga, ac, v = _jvp_case()
    a64 = ob.featurize_grad_inverse(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, v[:, 0], v[:, 1], v[:, 2])
    a32 = ob.featurize_grad_inverse(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, v[:, 0], v[:, 1], v[:, 2], dtype=np.float32)
    for p, q in zip(a32, a64):
        if p.size:
            assert np.max(np.abs(p - q)) <= 2e-5 * max(1.0, float(np.max(np.abs(q))))
