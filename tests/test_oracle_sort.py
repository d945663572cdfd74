"""Pins the integer part of the oracle (ani_sort, mol_offsets) without a GPU.

Checks: the reference's own KATs (gpu_featurizer/test_kernel.py:310-312; khan/model/test_nn.py:95 and
test_ani.py:46 hold the same gather_idxs as inv(argsort(types))), the definition by brute-force rank
counting, and numpy's stable argsort.
"""
import numpy as np
import pytest

import helpers
from oracle import binding as ob


def test_sort_reference_kat():
    _, _, _, a, _ = helpers.fixture11()
    sc, ga, ac = ob.ani_sort(a)
    assert ac.tolist() == helpers.FIXTURE11_ATOM_COUNTS
    assert sc.tolist() == helpers.FIXTURE11_SCATTER
    assert ga.tolist() == helpers.FIXTURE11_GATHER


def test_gather_is_inverse_of_stable_argsort():
    # khan/model/test_nn.py:95: gather_idxs == inv(argsort(types)) with a stable sort
    rng = np.random.default_rng(0)
    for n in (0, 1, 2, 63, 64, 65, 1000, 5000):
        a = rng.integers(0, 4, size=n).astype(np.int32)
        sc, ga, ac = ob.ani_sort(a)
        perm = np.argsort(a, kind="stable")
        inv = np.empty(n, dtype=np.int64)
        inv[perm] = np.arange(n)
        assert np.array_equal(ga, inv)
        assert ac.tolist() == np.bincount(a, minlength=4).tolist()


def test_scatter_brute_force_rank():
    rng = np.random.default_rng(1)
    a = rng.choice(4, size=300, p=[0.6, 0.25, 0.1, 0.05]).astype(np.int32)
    sc, ga, ac = ob.ani_sort(a)
    for g in range(a.size):
        assert sc[g] == int(np.sum(a[:g] == a[g]))
        assert ga[g] == int(np.sum(a < a[g])) + sc[g]


def test_sort_single_type_and_missing_types():
    a = np.full(130, 2, dtype=np.int32)
    sc, ga, ac = ob.ani_sort(a)
    assert ac.tolist() == [0, 0, 130, 0]
    assert np.array_equal(sc, np.arange(130)) and np.array_equal(ga, np.arange(130))


def test_sort_rejects_out_of_range_types():
    with pytest.raises(ValueError):
        ob.ani_sort(np.array([0, 4, 1], dtype=np.int32))


def test_mol_offsets_fixture_and_numpy():
    macs, mos = ob.mol_offsets(helpers.FIXTURE11_MOL_IDXS, 2)
    assert macs.tolist() == [8, 3] and mos.tolist() == [0, 8]
    rng = np.random.default_rng(2)
    counts = rng.integers(0, 30, size=200)           # includes empty molecules
    idx = np.repeat(np.arange(200), counts).astype(np.int32)
    macs, mos = ob.mol_offsets(idx, 200)
    assert np.array_equal(macs, counts)
    assert np.array_equal(mos, np.concatenate([[0], np.cumsum(counts)[:-1]]))


def test_mol_offsets_empty_batch():
    macs, mos = ob.mol_offsets(np.zeros(0, dtype=np.int32), 0)
    assert macs.size == 0 and mos.size == 0
    macs, mos = ob.mol_offsets(np.zeros(0, dtype=np.int32), 3)
    assert macs.tolist() == [0, 0, 0] and mos.tolist() == [0, 0, 0]
