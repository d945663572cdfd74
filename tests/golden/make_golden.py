"""Writes tests/golden/aev_golden.npz from the COMPILED REFERENCE (oracle/_ref/libkhan_ref.so, i.e.
/root/reference/gpu_featurizer/kernel_cpu.cpp built in place by `make -C oracle _ref`).

Run once in the build container:   python tests/golden/make_golden.py
The GPU box has no reference tree; tests there read only the committed .npz.

Cases
  fx11   the reference's 11-atom / 2-molecule test fixture (gpu_featurizer/test_kernel.py:269-287)
  org8   the first 8 molecules of the seeded organic generator (khan_amd.datagen, default seed)
For each case: inputs (X, Y, Z as float64 values exactly representable in float32, A, mol_idxs), the
sort outputs, feature rows in atom order from featurize_cpu<float> and <double>, an upstream gradient
drawn from numpy default_rng(7), and coordinate gradients from featurize_grad_cpu<double> and <float>
(the float functor produces non-finite entries for some triples; they are stored as they come).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import binding as ob  # noqa: E402
from khan_amd import datagen  # noqa: E402
import helpers  # noqa: E402


def case(prefix, X, Y, Z, A, mol_idxs, n_mols, out):
    X32, Y32, Z32 = (np.asarray(v, dtype=np.float32) for v in (X, Y, Z))
    sc, ga, ac = ob.ani_sort(A)
    macs, mos = ob.mol_offsets(mol_idxs, n_mols)
    n = A.size
    up = np.random.default_rng(7).standard_normal((n, 384))
    out[prefix + "_X"] = X32.astype(np.float64)
    out[prefix + "_Y"] = Y32.astype(np.float64)
    out[prefix + "_Z"] = Z32.astype(np.float64)
    out[prefix + "_A"] = A
    out[prefix + "_mol_idxs"] = mol_idxs
    out[prefix + "_scatter"] = sc
    out[prefix + "_gather"] = ga
    out[prefix + "_counts"] = ac
    out[prefix + "_macs"] = macs
    out[prefix + "_mos"] = mos
    out[prefix + "_upstream"] = up
    for dt, tag in ((np.float32, "f32"), (np.float64, "f64")):
        f = ob.featurize(X32, Y32, Z32, A, mos, macs, sc, ac, dtype=dt, impl="ref")
        out[prefix + "_feat_" + tag] = ob.gather_rows(f, ga)
        g = ob.scatter_rows(up.astype(dt), A, sc, ac)
        gx, gy, gz = ob.featurize_grad(X32, Y32, Z32, A, mos, macs, sc, ac, g, dtype=dt, impl="ref")
        out[prefix + "_grad_" + tag] = np.stack([gx, gy, gz], axis=1)


def main():
    if not ob.have_ref():
        raise SystemExit("oracle/_ref/libkhan_ref.so missing: run `make -C oracle _ref` where /root/reference exists")
    out = {}
    x, y, z, a, mi = helpers.fixture11()
    case("fx11", x, y, z, a, mi, 2, out)
    b = datagen.make_batch("organic", 8)
    case("org8", b.X, b.Y, b.Z, b.A, b.mol_idxs, 8, out)
    path = os.path.join(ROOT, "tests", "golden", "aev_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes;",
          {k: v.shape for k, v in out.items() if k.endswith("feat_f64")})


if __name__ == "__main__":
    main()
