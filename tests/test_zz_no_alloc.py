"""khan_featurize_f32_noalloc (the entry point that allocates nothing) against khan_featurize_f32, through the
C ABI, on two calls in a row, the second with a smaller input: both run the same kernels and differ only in
where the size order of the molecules lives, so the outputs must be identical bit for bit.  The first batch
is also checked against the CPU oracle.  Collected last (file name): a failure here hides nothing else."""
import ctypes
import sys

import numpy as np
import pytest

from khan_amd import datagen
from oracle import binding as ob

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _call(lib, name, t, acs, out):
    p = lambda x: ctypes.c_void_p(x.data_ptr() if x.numel() else None)
    bounds = np.concatenate([[0], np.cumsum(acs)]) * 384
    buckets = [out[bounds[k]:bounds[k + 1]] for k in range(4)]
    acs_c = (ctypes.c_int32 * 4)(*[int(v) for v in acs])
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return getattr(lib, name)(p(t["X"]), p(t["Y"]), p(t["Z"]), p(t["A"]), p(t["mos"]), p(t["macs"]),
                              t["macs"].numel(), p(t["sc"]), p(buckets[0]), p(buckets[1]), p(buckets[2]),
                              p(buckets[3]), acs_c, stream)


def _batch(kind, n_mols, first_mol):
    b = datagen.make_batch(kind, n_mols, first_mol=first_mol)
    sc, _, ac = ob.ani_sort(b.A)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    t = {"X": d(b.X), "Y": d(b.Y), "Z": d(b.Z), "A": d(b.A), "mos": d(b.MOs), "macs": d(b.MACs), "sc": d(sc)}
    return b, sc, ac, t


def test_no_alloc_entry_point_matches_featurize_on_two_calls_in_a_row():
    assert torch.cuda.is_available()
    from khan_amd import _lib
    lib = _lib.load()
    # 4,096 then 2,500 molecules (both large enough for the size order to be used), then a batch below that
    # threshold; the boxes put molecules into the kernels for larger sizes, which read the class counts
    for kind, n_mols, first in (("organic", 4096, 0), ("organic", 2500, 5000), ("boxes", 40, 0), ("organic", 64, 9000)):
        b, sc, ac, t = _batch(kind, n_mols, first)
        say("   no-alloc entry point: %s, %d molecules, %d atoms" % (kind, n_mols, b.n_atoms))
        ref_out = torch.full((b.n_atoms * 384,), -1.0, dtype=torch.float32, device="cuda:0")
        new_out = torch.full((b.n_atoms * 384,), -2.0, dtype=torch.float32, device="cuda:0")
        assert _call(lib, "khan_featurize_f32", t, ac, ref_out) == 0
        assert _call(lib, "khan_featurize_f32_noalloc", t, ac, new_out) == 0
        torch.cuda.synchronize()
        assert torch.equal(ref_out, new_out), "the two entry points differ"
        if first == 0 and kind == "organic":
            ref = np.concatenate(ob.featurize(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, sc, ac, dtype=np.float64))
            got = new_out.cpu().numpy().astype(np.float64)
            assert np.all(np.abs(got - ref) <= 1e-6 + 1e-5 * np.abs(ref)), "no-alloc entry point vs the oracle"


def test_no_alloc_entry_point_replays_from_a_hip_graph():
    """What sets the entry point apart: it can run where nothing may be allocated.  After one eager call (which looks
    the scratch array's address up) it is captured into a HIP graph -- a capture fails on any allocation or memset on
    the capturing stream -- and replayed on poisoned outputs, with eager work and synchronisations between the replays;
    every replay must reproduce the eager result bit for bit.  4,096 molecules and two boxes: the size order (cleared by
    a kernel of the graph, not by a memset node) and the kernels of the larger size classes are part of the graph."""
    from khan_amd import _lib
    lib = _lib.load()
    b, sc, ac, t = _batch("organic", 4096, 20000)
    big = datagen.make_batch("boxes", 2)
    A = np.concatenate([b.A, big.A])
    sc, _, ac = ob.ani_sort(A)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    macs = np.concatenate([b.MACs, big.MACs]).astype(np.int32)
    mos = np.concatenate([[0], np.cumsum(macs)[:-1]]).astype(np.int32)
    t = {"X": d(np.concatenate([b.X, big.X])), "Y": d(np.concatenate([b.Y, big.Y])), "Z": d(np.concatenate([b.Z, big.Z])),
         "A": d(A), "mos": d(mos), "macs": d(macs), "sc": d(sc)}
    n = len(A)
    say("   no-alloc entry point under graph capture: %d molecules, %d atoms" % (len(macs), n))
    eager = torch.full((n * 384,), -1.0, dtype=torch.float32, device="cuda:0")
    assert _call(lib, "khan_featurize_f32_noalloc", t, ac, eager) == 0
    torch.cuda.synchronize()
    out = torch.full((n * 384,), -2.0, dtype=torch.float32, device="cuda:0")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        status = _call(lib, "khan_featurize_f32_noalloc", t, ac, out)     # on the capturing stream (the current one here)
    assert status == 0
    for replay in range(3):
        out.fill_(-3.0 - replay)
        scratch_user = torch.full((n * 384,), -1.0, dtype=torch.float32, device="cuda:0")
        if replay == 1:     # an eager call on a smaller batch in between leaves other contents in the shared scratch
            b2, sc2, ac2, t2 = _batch("organic", 2300, 100)
            o2 = torch.empty(b2.n_atoms * 384, dtype=torch.float32, device="cuda:0")
            assert _call(lib, "khan_featurize_f32_noalloc", t2, ac2, o2) == 0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), "replay %d differs from the eager call" % replay
        del scratch_user


def test_no_alloc_entry_point_with_a_molecule_of_more_than_256_atoms():
    # above 256 atoms khan_featurize_f32 works on a sorted copy of the atoms in scratch memory; the entry point that
    # allocates nothing keeps to the kernels without scratch: the same features to float32 rounding, both checked
    # against the oracle
    from khan_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(9)
    small = datagen.make_batch("organic", 3, first_mol=77)
    n_big = 300
    side = (n_big / 0.1) ** (1 / 3)
    pts = np.empty((0, 3))
    while len(pts) < n_big:
        q = rng.uniform(0, side, 3)
        if len(pts) == 0 or np.min(np.linalg.norm(pts - q, axis=1)) >= 0.9:
            pts = np.vstack([pts, q])
    X = np.concatenate([small.X, pts[:, 0]]).astype(np.float32)
    Y = np.concatenate([small.Y, pts[:, 1]]).astype(np.float32)
    Z = np.concatenate([small.Z, pts[:, 2]]).astype(np.float32)
    A = np.concatenate([small.A, rng.integers(0, 4, n_big)]).astype(np.int32)
    macs = np.concatenate([small.MACs, [n_big]]).astype(np.int32)
    mos = np.concatenate([[0], np.cumsum(macs)[:-1]]).astype(np.int32)
    sc, _, ac = ob.ani_sort(A)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    t = {"X": d(X), "Y": d(Y), "Z": d(Z), "A": d(A), "mos": d(mos), "macs": d(macs), "sc": d(sc)}
    n = len(A)
    say("   no-alloc entry point: 3 small molecules and one of %d atoms" % n_big)
    ref_out = torch.full((n * 384,), -1.0, dtype=torch.float32, device="cuda:0")
    new_out = torch.full((n * 384,), -2.0, dtype=torch.float32, device="cuda:0")
    assert _call(lib, "khan_featurize_f32", t, ac, ref_out) == 0
    assert _call(lib, "khan_featurize_f32_noalloc", t, ac, new_out) == 0
    torch.cuda.synchronize()
    ref = np.concatenate(ob.featurize(X, Y, Z, A, mos, macs, sc, ac, dtype=np.float64))
    for name, got in (("khan_featurize_f32", ref_out), ("khan_featurize_f32_noalloc", new_out)):
        g = got.cpu().numpy().astype(np.float64)
        assert np.all(np.abs(g - ref) <= 1e-6 + 1e-5 * np.abs(ref)), name + " vs the oracle"


def test_no_alloc_entry_point_rejects_what_its_scratch_cannot_hold():
    from khan_amd import _lib
    lib = _lib.load()
    acs = (ctypes.c_int32 * 4)(1, 0, 0, 0)
    one = ctypes.c_void_p(16)      # never dereferenced: the size check comes before any launch
    too_many = (1 << 20) + 1
    st = lib.khan_featurize_f32_noalloc(one, one, one, one, one, one, too_many, one, one, one, one, one, acs, None)
    assert st == 3 and b"scratch" in lib.khan_last_hip_error()
    acs0 = (ctypes.c_int32 * 4)(0, 0, 0, 0)
    assert lib.khan_featurize_f32_noalloc(None, None, None, None, None, None, 0, None, None, None, None, None, acs0, None) == 0
