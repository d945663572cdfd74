"""Pins the charge oracle without a GPU.

The reference holds no expected VALUES for charges (gpu_featurizer/test_charges.py prints and asserts
nothing); its only check is that dE/dq agrees with a numeric derivative (test_kernel.py:403-459,
delta 1e-3, tol 1e-11 in float64).  So values are pinned by the two-line closed form
(ani_charges.cpp:58-71) evaluated by brute force in long double, by the textbook limit K q_i q_j / r
beyond the cutoff, by Euler's identity for a bilinear form, and by finite differences.
The coordinate gradient has no reference counterpart at all: finite differences and zero net force.
"""
import numpy as np
import pytest

import helpers
from khan_amd import datagen
from oracle import binding as ob

K32 = float(np.float32(helpers.CHARGE_K))


def _fixture():
    x, y, z, a, mi = helpers.fixture11()
    return x, y, z, helpers.FIXTURE11_QS, np.array([0, 8], np.int32), np.array([8, 3], np.int32)


def test_energy_brute_force_long_double():
    x, y, z, q, mos, macs = _fixture()
    e = ob.ani_charge(x, y, z, q, mos, macs, dtype=np.float64)
    xyz = np.stack([x, y, z], axis=1)
    assert e[0] == pytest.approx(helpers.brute_force_charge_energy(xyz[:8], q[:8]), rel=1e-13)
    assert e[1] == pytest.approx(helpers.brute_force_charge_energy(xyz[8:], q[8:]), rel=1e-13)
    e32 = ob.ani_charge(x, y, z, q, mos, macs, dtype=np.float32)
    assert np.allclose(e32, e, rtol=1e-5)


def test_beyond_cutoff_is_plain_coulomb_and_inside_is_damped():
    one = np.array([0], np.int32), np.array([2], np.int32)
    for r in (4.7, 9.0):
        e = ob.ani_charge([0, 0], [0, 0], [0, r], [0.7, -1.3], *one, dtype=np.float64)[0]
        assert e == pytest.approx(K32 * 0.7 * -1.3 / r, rel=1e-14)
    r = 1.5
    e = ob.ani_charge([0, 0], [0, 0], [0, r], [0.7, -1.3], *one, dtype=np.float64)[0]
    fc = 0.5 * np.cos(np.pi * r / float(np.float32(4.6))) + 0.5
    assert e == pytest.approx(K32 * 0.7 * -1.3 * (1 - fc) / r, rel=1e-14)
    assert abs(e) < abs(K32 * 0.7 * -1.3 / r)


def test_dq_numeric_like_reference_and_euler():
    x, y, z, q, mos, macs = _fixture()
    dq = ob.ani_charge_grad(x, y, z, q, mos, macs, np.ones(2), dtype=np.float64)
    delta = 1e-3
    for i in range(11):
        qp, qm = q.copy(), q.copy()
        qp[i] += delta
        qm[i] -= delta
        num = (ob.ani_charge(x, y, z, qp, mos, macs).sum() - ob.ani_charge(x, y, z, qm, mos, macs).sum()) / (2 * delta)
        assert abs(num - dq[i]) < 1e-11
    e = ob.ani_charge(x, y, z, q, mos, macs)
    assert 0.5 * (q[:8] * dq[:8]).sum() == pytest.approx(e[0], rel=1e-13)
    assert 0.5 * (q[8:] * dq[8:]).sum() == pytest.approx(e[1], rel=1e-13)
    # the upstream gradient scales each molecule's block
    dq2 = ob.ani_charge_grad(x, y, z, q, mos, macs, np.array([2.0, -3.0]), dtype=np.float64)
    assert np.allclose(dq2[:8], 2.0 * dq[:8], rtol=1e-15) and np.allclose(dq2[8:], -3.0 * dq[8:], rtol=1e-15)


def test_dxyz_finite_differences_and_net_force():
    b = datagen.make_batch("organic", 5, first_mol=9)
    q = datagen.charges(b.n_atoms).astype(np.float64)
    gm = np.array([1.0, -2.0, 0.5, 3.0, 1.5])
    xyz = [b.X.astype(np.float64), b.Y.astype(np.float64), b.Z.astype(np.float64)]
    g = np.stack(ob.ani_charge_grad_xyz(*xyz, q, b.MOs, b.MACs, gm, dtype=np.float64), axis=1)
    h = 1e-5
    scale = np.abs(g).max()
    for a in range(0, b.n_atoms, 4):
        for ax in range(3):
            cp = [v.copy() for v in xyz]
            cm = [v.copy() for v in xyz]
            cp[ax][a] += h
            cm[ax][a] -= h
            num = ((ob.ani_charge(*cp, q, b.MOs, b.MACs) - ob.ani_charge(*cm, q, b.MOs, b.MACs)) * gm).sum() / (2 * h)
            assert abs(num - g[a, ax]) <= 1e-8 * scale
    for m in range(5):
        s = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
        assert np.abs(g[s].sum(axis=0)).max() <= 1e-13 * scale
