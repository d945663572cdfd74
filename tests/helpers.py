"""Shared test data and independent closed forms.

FIXTURE11 is the 11-atom / 2-molecule case the reference's own op test uses
(gpu_featurizer/test_kernel.py:269-287; the same atoms appear in README.md:118-134 and
gpu_featurizer/test_charges.py:46-61), with the expected sort outputs the reference asserts
(test_kernel.py:310-312) and its charge vector (test_kernel.py:426-438).
"""
import math

import numpy as np

FIXTURE11_ATOMS = np.array([
    [0, 1.0, 2.0, 3.0],     # H
    [2, 2.0, 1.0, 4.0],     # N
    [0, 0.5, 1.2, 2.3],     # H
    [1, 0.3, 1.7, 3.2],     # C
    [2, 0.6, 1.2, 1.1],     # N
    [0, 14.0, 23.0, 15.0],  # H
    [0, 2.0, 0.5, 0.3],     # H
    [0, 2.3, 0.2, 0.4],     # H
    [0, 2.3, 0.2, 0.4],     # H
    [1, 0.3, 1.7, 3.2],     # C
    [2, 0.6, 1.2, 1.1],     # N
], dtype=np.float64)
FIXTURE11_MOL_IDXS = np.array([0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1], dtype=np.int32)
FIXTURE11_ATOM_COUNTS = [6, 2, 3, 0]
FIXTURE11_SCATTER = [0, 0, 1, 0, 1, 2, 3, 4, 5, 1, 2]
FIXTURE11_GATHER = [0, 8, 1, 6, 9, 2, 3, 4, 5, 7, 10]
FIXTURE11_QS = np.array([0.3, 4.5, 2.2, 3.4, -5.6, 3.4, 1.1, 3.2, 1.0, 0.3, 2.4], dtype=np.float64)


def fixture11():
    a = FIXTURE11_ATOMS
    return (a[:, 1].copy(), a[:, 2].copy(), a[:, 3].copy(), a[:, 0].astype(np.int32),
            FIXTURE11_MOL_IDXS.copy())


# ---- parameters as the reference's python test writes them (test_kernel.py:149-189) ----
R_RS = [0.5 + 0.25625 * i for i in range(16)]
R_RC, R_ETA = 4.6, 16.0
A_THETAS = [0.0, 7.8539816e-01, 1.5707963e+00, 2.3561945e+00, 3.1415927e+00, 3.9269908e+00,
            4.7123890e+00, 5.4977871e+00]
A_RS = [0.5, 1.15, 1.8, 2.45]
A_RC, A_ETA, A_ZETA = 3.1, 6.0, 8.0
CHARGE_K = 0.529176917


def pair_block(a, b):
    """Index of the unordered type pair in HH HC HN HO CC CN CO NN NO OO order."""
    order = [(0, 0), (0, 1), (0, 2), (0, 3), (1, 1), (1, 2), (1, 3), (2, 2), (2, 3), (3, 3)]
    return order.index((min(a, b), max(a, b)))


def f_c(r, rc):
    return 0.5 * math.cos(math.pi * r / rc) + 0.5 if r <= rc else 0.0


def brute_force_aev(types, xyz):
    """[n,384] features of ONE molecule from the defining sums, in double.

    Independent of the oracle's loop structure: every centre sums over all ordered partners (radial)
    and all unordered partner pairs (angular), using the angle from arccos of the normalised dot
    product -- the construction of the reference's own python check (test_kernel.py:147-255).
    """
    n = len(types)
    xyz = np.asarray(xyz, dtype=np.float64)
    out = np.zeros((n, 384))
    for i in range(n):
        for j in range(n):
            if j == i:
                continue
            rij = float(np.linalg.norm(xyz[i] - xyz[j]))
            if rij < R_RC:
                for r, rs in enumerate(R_RS):
                    out[i, types[j] * 16 + r] += math.exp(-R_ETA * (rij - rs) ** 2) * f_c(rij, R_RC)
            for k in range(j + 1, n):
                if k == i:
                    continue
                rik = float(np.linalg.norm(xyz[i] - xyz[k]))
                if not (rij < A_RC and rik < A_RC):
                    continue
                vij, vik = xyz[i] - xyz[j], xyz[i] - xyz[k]
                cosang = float(np.dot(vij, vik) / (rij * rik))
                theta = math.acos(max(-1.0, min(1.0, cosang)))
                base = 64 + 32 * pair_block(types[j], types[k])
                for t, th in enumerate(A_THETAS):
                    for s, rs in enumerate(A_RS):
                        out[i, base + 4 * t + s] += (2.0 ** (1 - A_ZETA) * (1 + math.cos(theta - th)) ** A_ZETA *
                                                     math.exp(-A_ETA * ((rij + rik) / 2 - rs) ** 2) *
                                                     f_c(rij, A_RC) * f_c(rik, A_RC))
    return out


def brute_force_charge_energy(xyz, q):
    """sum_{i<j} K q_i q_j (1 - f_C(r, R_Rc)) / r for one molecule, accumulated in long double.
    K and R_Rc are the float-rounded values the reference compiles in (parameters.h:10,72)."""
    xyz = np.asarray(xyz, dtype=np.float64)
    k32, rc32 = float(np.float32(CHARGE_K)), float(np.float32(R_RC))
    e = np.longdouble(0)
    for i in range(len(q)):
        for j in range(i + 1, len(q)):
            r = float(np.linalg.norm(xyz[i] - xyz[j]))
            e += np.longdouble(k32 * q[i] * q[j] * (1 - f_c(r, rc32)) / r)
    return float(e)


def within(a, b, rtol, atol):
    """Elementwise |a-b| <= atol + rtol*|b| ; returns (ok, worst ratio, index)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    ratio = np.abs(a - b) / (atol + rtol * np.abs(b))
    if ratio.size == 0:
        return True, 0.0, -1
    worst = int(np.nanargmax(ratio)) if not np.all(np.isnan(ratio)) else 0
    return bool(np.all(ratio <= 1.0)), float(ratio.reshape(-1)[worst]), worst


def random_rotation(rng):
    q, r = np.linalg.qr(rng.standard_normal((3, 3)))
    q = q * np.sign(np.diag(r))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return q
