"""The measurement variant of the small-molecule forward kernel that sums the angular records on the matrix cores
(KHAN_AEV_PHASE2=matrix, read once per process by the check build of libkhan_aev.so, which alone holds that kernel and
that switch: khan_amd/build.py, build_check_variant) gives the same features as the default kernel:
checked against the float64 oracle at the float32 tolerance of test_gpu_parity.py.  The variable is read when the
first forward pass is launched, so the variant runs in a child process."""
import os
import subprocess
import sys

import numpy as np
import pytest

from khan_amd import datagen
from oracle import binding as ob

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
import numpy as np, torch
sys.path.insert(0, sys.argv[1])
from khan_amd import datagen, ops
b = datagen.make_batch("organic", int(sys.argv[3]))
d = "cuda:0"
X, Y, Z = (torch.from_numpy(v).to(d) for v in (b.X, b.Y, b.Z))
A = torch.from_numpy(b.A).to(d)
macs, mos = ops.mol_offsets(torch.from_numpy(b.mol_idxs).to(d), b.n_mols)
sc, ga, ac = ops.ani_sort(A)
f = ops.featurize(X, Y, Z, A, mos, macs, sc, ac.cpu())
torch.cuda.synchronize()
np.save(sys.argv[2], torch.cat(f).cpu().numpy())
"""


def run_child(tmp_path, name, n_mols, variant):
    out = str(tmp_path / (name + ".npy"))
    env = dict(os.environ)
    env.pop("KHAN_AEV_PHASE2", None)
    env.pop("KHAN_AEV_LIBRARY", None)
    if variant:
        from khan_amd import build
        assert os.path.exists(build.CHECK_LIBRARY), "the check build is missing: python -m khan_amd.build"
        env["KHAN_AEV_LIBRARY"] = build.CHECK_LIBRARY
        env["KHAN_AEV_PHASE2"] = variant
    print("child: KHAN_AEV_PHASE2=%s, organic %d molecules" % (variant, n_mols), flush=True)
    subprocess.run([sys.executable, "-c", CHILD, ROOT, out, str(n_mols)], env=env, check=True, timeout=300)
    return np.load(out).astype(np.float64)


def test_matrix_core_phase2_matches_the_oracle(tmp_path):
    n_mols = 1024
    b = datagen.make_batch("organic", n_mols)
    MACs, MOs = ob.mol_offsets(b.mol_idxs, b.n_mols)
    sc, ga, ac = ob.ani_sort(b.A)
    ref = np.concatenate(ob.featurize(b.X, b.Y, b.Z, b.A, MOs, MACs, sc, ac, dtype=np.float64))
    got = run_child(tmp_path, "matrix", n_mols, "matrix")
    base = run_child(tmp_path, "default", n_mols, None)
    for name, v in (("matrix-core phase 2", got), ("default", base)):
        assert v.shape == ref.shape and np.all(np.isfinite(v))
        ratio = np.abs(v - ref) / (1e-6 + 1e-5 * np.abs(ref))
        print("   %-22s max|err| %.3e  worst err/bound %.3f" % (name, np.abs(v - ref).max(), ratio.max()), flush=True)
        assert ratio.max() <= 1.0, name
    # the two kernels differ in the order of the sums only, and somewhere: identical outputs would mean the
    # variable did not select the variant
    assert np.abs(got - base).max() > 0.0
    assert np.abs(got - base).max() <= 2e-6 + 2e-5 * np.abs(ref).max()
