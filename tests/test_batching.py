"""Host batch assembly (khan_amd.batching) against the reference's semantics, khan/data/dataset.py:118-183."""
import numpy as np
import pytest

from khan_amd import batching, datagen


def _molecules(n_mols=23, seed=5):
    b = datagen.make_batch("organic", n_mols, first_mol=seed)
    mols = []
    for m in range(n_mols):
        s = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
        mols.append(np.stack([b.A[s].astype(np.float64), b.X[s], b.Y[s], b.Z[s]], axis=1))
    return mols


def test_iterate_matches_reference_semantics():
    mols = _molecules()
    ys = [float(k) for k in range(len(mols))]
    grads = [np.full((len(m), 3), k, dtype=np.float64) for k, m in enumerate(mols)]
    ds = batching.RawDataset(mols, ys, grads)
    assert ds.num_mols() == 23 and ds.num_batches(5) == 5
    seen = 0
    for bi, (X, ids, yts, g) in enumerate(ds.iterate(5, shuffle=False)):
        k = 5 if bi < 4 else 3                      # the last batch is not padded
        assert len(yts) == k and yts == ys[seen:seen + k]
        want = np.concatenate(mols[seen:seen + k], axis=0)
        assert np.array_equal(X, want)
        assert np.array_equal(ids, np.repeat(np.arange(k), [len(m) for m in mols[seen:seen + k]]))
        assert g.shape == (X.shape[0], 3) and np.array_equal(g[:, 0], np.repeat(np.arange(seen, seen + k), [len(m) for m in mols[seen:seen + k]]))
        seen += k
    assert seen == 23


def test_shuffle_is_a_permutation_and_fuzz_is_bounded():
    mols = _molecules()
    ds = batching.RawDataset(mols, [float(k) for k in range(len(mols))])
    labels = []
    for X, ids, yts, g in ds.iterate(4, shuffle=True, rng=np.random.default_rng(1)):
        labels += yts
        assert g is None
    assert sorted(labels) == [float(k) for k in range(23)] and labels != sorted(labels)
    plain = next(iter(ds.iterate(23, shuffle=False)))[0]
    fuzzed = next(iter(ds.iterate(23, shuffle=False, fuzz=0.01, rng=np.random.default_rng(2))))[0]
    assert np.array_equal(plain[:, 0], fuzzed[:, 0])                       # types untouched
    d = np.abs(fuzzed[:, 1:] - plain[:, 1:])
    assert d.max() <= 0.01 and d.max() > 0.0
    assert np.array_equal(mols[0], ds.all_Xs[0])                           # the dataset itself is not modified


def test_split_columns():
    mols = _molecules(3)
    X, ids, _, _ = next(iter(batching.RawDataset(mols).iterate(3, False)))
    xs, ys, zs, types, mids = batching.split_columns(X, ids, np.float32)
    assert xs.dtype == np.float32 and types.dtype == np.int32 and mids.dtype == np.int32
    assert all(a.flags.c_contiguous for a in (xs, ys, zs, types, mids))
    assert np.array_equal(types, X[:, 0].astype(np.int32)) and np.allclose(ys, X[:, 2])


@pytest.mark.gpu
def test_device_feeder_feeds_the_featurizer():
    torch = pytest.importorskip("torch")
    from khan_amd import ops
    from oracle import binding as ob
    mols = _molecules(41, seed=60)
    ds = batching.RawDataset(mols, [0.0] * len(mols))
    feeder = batching.DeviceFeeder(ds, batch_size=16, dtype=np.float32)
    seen = 0
    for batch in feeder:
        batch.wait()
        k = batch.n_mols
        want = np.concatenate(mols[seen:seen + k], axis=0)
        assert np.array_equal(batch.xs.cpu().numpy(), want[:, 1].astype(np.float32))
        assert np.array_equal(batch.atom_types.cpu().numpy(), want[:, 0].astype(np.int32))
        A = want[:, 0].astype(np.int32)
        macs = np.array([len(m) for m in mols[seen:seen + k]], dtype=np.int32)
        mos = np.concatenate([[0], np.cumsum(macs)[:-1]]).astype(np.int32)
        sc, ga, ac = ob.ani_sort(A)
        assert np.array_equal(batch.scatter_idxs.cpu().numpy(), sc) and np.array_equal(batch.mol_offsets.cpu().numpy(), mos)
        acs = batch.atom_counts.cpu()
        f = ops.featurize(batch.xs, batch.ys, batch.zs, batch.atom_types, batch.mol_offsets, batch.mol_atom_counts,
                          batch.scatter_idxs, acs)
        ref = np.concatenate(ob.featurize(want[:, 1], want[:, 2], want[:, 3], A, mos, macs, sc, ac, dtype=np.float64))
        got = torch.cat(f).cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - ref) <= 1e-6 + 1e-5 * np.abs(ref))
        seen += k
    assert seen == 41


@pytest.mark.gpu
def test_device_feeder_keeps_trailing_molecules_without_atoms():
    """A batch whose last molecules have no atoms still has one molecule per label (the molecule ids of the atoms
    alone would end at the last non-empty one)."""
    pytest.importorskip("torch")
    mols = _molecules(5, seed=61) + [np.zeros((0, 4)), np.zeros((0, 4))]
    ds = batching.RawDataset(mols, [float(k) for k in range(len(mols))])
    batches = list(batching.DeviceFeeder(ds, batch_size=7, dtype=np.float32))
    assert len(batches) == 1
    b = batches[0].wait()
    assert b.n_mols == 7 and len(b.labels) == 7
    assert b.mol_atom_counts.cpu().tolist() == [len(m) for m in mols]
    assert b.mol_offsets.cpu().tolist()[-2:] == [sum(len(m) for m in mols)] * 2


# ------------------------------------------------------------------------------- packed data set (native gather)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_packed_dataset_yields_what_the_raw_one_yields(dtype):
    mols = _molecules(29, seed=11)
    ys = [float(3 * k) for k in range(len(mols))]
    grads = [np.random.default_rng(k).normal(size=(len(m), 3)) for k, m in enumerate(mols)]
    raw = batching.RawDataset(mols, ys, grads)
    packed = batching.PackedDataset.from_raw(raw, dtype=dtype, n_threads=3)
    assert packed.num_mols() == 29 and packed.num_batches(8) == 4
    for shuffle in (False, True):
        a = list(raw.iterate(8, shuffle, rng=np.random.default_rng(5)))
        b = list(packed.iterate(8, shuffle, rng=np.random.default_rng(5)))
        assert len(a) == len(b) == 4
        for (Xa, ia, ya, ga), (Xb, ib, yb, gb) in zip(a, b):
            # coordinates pass through the data set's precision (the generator's are float32 values)
            assert Xb.dtype == np.float64 and np.array_equal(Xa.astype(dtype), Xb.astype(dtype))
            assert ib.dtype == np.int32 and np.array_equal(ia, ib)
            assert ya == yb and np.array_equal(ga, gb)


def test_packed_dataset_gather_edge_cases():
    mols = _molecules(7, seed=2)
    packed = batching.PackedDataset(mols, dtype=np.float64)
    xs, ys, zs, types, ids = packed.gather([6, 0, 0, 3])               # any order, repeats allowed
    want = np.concatenate([mols[6], mols[0], mols[0], mols[3]], axis=0)
    assert np.array_equal(xs, want[:, 1]) and np.array_equal(zs, want[:, 3]) and np.array_equal(types, want[:, 0].astype(np.int32))
    assert np.array_equal(ids, np.repeat(np.arange(4), [len(mols[6]), len(mols[0]), len(mols[0]), len(mols[3])]))
    assert packed.gather([])[0].size == 0
    with pytest.raises(IndexError):
        packed.gather([7])
    with pytest.raises(IndexError):
        packed.gather([-1])
    sel, off, n = packed.batch_atoms([1, 2])
    small = np.empty(n - 1, dtype=np.float64)
    with pytest.raises(ValueError):
        packed.gather_into(sel, off, small, small, small, np.empty(n, np.int32), np.empty(n, np.int32))
    assert batching.PackedDataset([]).num_mols() == 0 and list(batching.PackedDataset([]).iterate(4, False)) == []
    fuzzed = next(iter(packed.iterate(7, False, fuzz=0.02, rng=np.random.default_rng(1))))[0]
    plain = next(iter(packed.iterate(7, False)))[0]
    d = np.abs(fuzzed[:, 1:] - plain[:, 1:])
    assert np.array_equal(fuzzed[:, 0], plain[:, 0]) and 0.0 < d.max() <= 0.02


@pytest.mark.gpu
def test_device_feeder_from_a_packed_dataset_matches_the_raw_one():
    torch = pytest.importorskip("torch")
    mols = _molecules(53, seed=80)
    labels = [float(k) for k in range(len(mols))]
    grads = [np.full((len(m), 3), k, dtype=np.float64) for k, m in enumerate(mols)]
    raw = batching.RawDataset(mols, labels, grads)
    packed = batching.PackedDataset.from_raw(raw, dtype=np.float32)
    for shuffle in (False, True):
        fa = batching.DeviceFeeder(raw, 20, shuffle=shuffle, rng=np.random.default_rng(9))
        fb = batching.DeviceFeeder(packed, 20, shuffle=shuffle, rng=np.random.default_rng(9))
        n_batches = 0
        for a, b in zip(fa, fb):
            a.wait()
            b.wait()
            for name in ("xs", "ys", "zs", "atom_types", "mol_idxs", "mol_atom_counts", "mol_offsets", "scatter_idxs",
                         "gather_idxs", "atom_counts", "grads"):
                assert torch.equal(getattr(a, name), getattr(b, name)), name
            assert a.n_mols == b.n_mols and a.labels == list(b.labels)
            n_batches += 1
        assert n_batches == 3
    with pytest.raises(TypeError):
        list(batching.DeviceFeeder(packed, 20, dtype=np.float64))
