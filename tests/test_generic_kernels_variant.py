"""The check build of libkhan_aev.so (khan_amd/build.py: build_check_variant; the default library reads no environment
variable) offers two switches.  KHAN_AEV_FORCE_GENERIC=1 (read once per process) routes every molecule through the general-shape
kernels (workgroup per molecule, wavefront per centre), which otherwise only see the centres whose lists overflow and,
when no scratch memory may be taken, molecules of more than 256 atoms.  KHAN_AEV_LARGE_SCRATCH=0 withholds that scratch
memory, as a stream under graph capture or a failed allocation would: molecules of more than 256 atoms then go to the
general-shape kernels while the others keep to theirs.  Features, gradients and the Jacobian-vector product from both
variants are checked against the float64 oracle at the tolerances of test_gpu_parity.py; the variables are read at the
first launch, so each run is a child process."""
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
from types import SimpleNamespace
from khan_amd import ops
inp, out = np.load(sys.argv[2]), sys.argv[3]
b = SimpleNamespace(X=inp["X"], Y=inp["Y"], Z=inp["Z"], A=inp["A"], mol_idxs=inp["mol_idxs"], n_mols=int(inp["n_mols"]),
                    n_atoms=len(inp["A"]))
d = "cuda:0"
res = {}
A = torch.from_numpy(b.A).to(d)
macs, mos = ops.mol_offsets(torch.from_numpy(b.mol_idxs).to(d), b.n_mols)
sc, ga, ac = ops.ani_sort(A)
acs = ac.cpu()
up = np.random.default_rng(11).standard_normal((b.n_atoms, 384))
v = np.random.default_rng(12).standard_normal((3, b.n_atoms))
counts = [int(c) for c in acs.tolist()]
for name, dt in (("f32", np.float32), ("f64", np.float64)):
    X, Y, Z = (torch.from_numpy(a.astype(dt)).to(d) for a in (b.X, b.Y, b.Z))
    f = ops.featurize(X, Y, Z, A, mos, macs, sc, acs)
    res["feat_" + name] = torch.cat(f).cpu().numpy()
    # upstream rows in bucket order: row of atom g is bucket row gather_idxs[g]
    bucket = torch.empty((b.n_atoms, 384), dtype=X.dtype, device=d)
    bucket[ga.long()] = torch.from_numpy(up.astype(dt)).to(d)
    gb = [t.reshape(-1) for t in bucket.split(counts)]
    g = ops.featurize_grad(X, Y, Z, A, mos, macs, sc, acs, *gb)
    res["grad_" + name] = torch.stack(g, 1).cpu().numpy()
    j = ops.featurize_grad_inverse(X, Y, Z, A, mos, macs, sc, acs, *[torch.from_numpy(v[c].astype(dt)).to(d) for c in range(3)])
    res["jvp_" + name] = torch.cat(j).cpu().numpy()
torch.cuda.synchronize()
np.savez(out, **res)
"""


def _with_large_molecules():
    """three organic molecules, a dense box, and boxes of 300 and 520 atoms at 0.1 atoms per cubic Angstrom"""
    from types import SimpleNamespace
    rng = np.random.default_rng(23)
    parts = []
    for kind, n in (("organic", 3), ("boxes", 1)):
        s = datagen.make_batch(kind, n)
        for m in range(n):
            sl = slice(s.MOs[m], s.MOs[m] + s.MACs[m])
            parts.append((s.A[sl], np.stack([s.X[sl], s.Y[sl], s.Z[sl]], 1)))
    for n in (300, 520):
        side = (n / 0.1) ** (1 / 3)
        pts = np.empty((0, 3))
        while len(pts) < n:
            q = rng.uniform(0, side, 3)
            if len(pts) == 0 or np.min(np.linalg.norm(pts - q, axis=1)) >= 0.9:
                pts = np.vstack([pts, q])
        parts.insert(1, (rng.integers(0, 4, n), pts))
    A = np.concatenate([p[0] for p in parts]).astype(np.int32)
    xyz = np.concatenate([p[1] for p in parts]).astype(np.float32)
    mi = np.concatenate([np.full(len(p[0]), k) for k, p in enumerate(parts)]).astype(np.int32)
    return SimpleNamespace(X=xyz[:, 0].copy(), Y=xyz[:, 1].copy(), Z=xyz[:, 2].copy(), A=A, mol_idxs=mi, n_mols=len(parts),
                           n_atoms=len(A))


@pytest.mark.parametrize("kind,n_mols,variable", [("organic", 96, "KHAN_AEV_FORCE_GENERIC=1"), ("boxes", 2, "KHAN_AEV_FORCE_GENERIC=1"),
                                                  ("large", 6, "KHAN_AEV_LARGE_SCRATCH=0")])
def test_general_shape_kernels_match_the_oracle(tmp_path, kind, n_mols, variable):
    b = _with_large_molecules() if kind == "large" else datagen.make_batch(kind, n_mols)
    MACs, MOs = ob.mol_offsets(b.mol_idxs, b.n_mols)
    sc, ga, ac = ob.ani_sort(b.A)
    up = np.random.default_rng(11).standard_normal((b.n_atoms, 384))
    v = np.random.default_rng(12).standard_normal((3, b.n_atoms))
    feat = np.concatenate(ob.featurize(b.X, b.Y, b.Z, b.A, MOs, MACs, sc, ac, dtype=np.float64))
    upb = ob.scatter_rows(up, b.A, sc, ac)
    grad = np.stack(ob.featurize_grad(b.X, b.Y, b.Z, b.A, MOs, MACs, sc, ac, upb, dtype=np.float64), 1)
    jvp = np.concatenate(ob.featurize_grad_inverse(b.X, b.Y, b.Z, b.A, MOs, MACs, sc, ac, v[0], v[1], v[2], dtype=np.float64))
    out, inp = str(tmp_path / "generic.npz"), str(tmp_path / "inputs.npz")
    np.savez(inp, X=b.X, Y=b.Y, Z=b.Z, A=b.A, mol_idxs=b.mol_idxs, n_mols=b.n_mols)
    from khan_amd import build
    assert os.path.exists(build.CHECK_LIBRARY), "the check build is missing: python -m khan_amd.build"
    env = dict(os.environ)
    env["KHAN_AEV_LIBRARY"] = build.CHECK_LIBRARY
    name, value = variable.split("=")
    env[name] = value
    print("child: %s, %s, %d molecules, %d atoms" % (variable, kind, b.n_mols, b.n_atoms), flush=True)
    subprocess.run([sys.executable, "-c", CHILD, ROOT, inp, out], env=env, check=True, timeout=300)
    got = np.load(out)
    gscale = np.zeros_like(grad)
    for m in range(b.n_mols):
        s = slice(MOs[m], MOs[m] + MACs[m])
        gscale[s] = np.abs(grad[s]).max()
    jscale = np.abs(jvp).max()
    for name, rtol, atol in (("f32", 1e-5, 1e-6), ("f64", 1e-12, 1e-15)):
        f = got["feat_" + name].astype(np.float64).reshape(-1)
        assert np.all(np.abs(f - feat.reshape(-1)) <= atol + rtol * np.abs(feat.reshape(-1))), ("features", name)
        g = got["grad_" + name].astype(np.float64)
        assert np.all(np.abs(g - grad) <= atol + rtol * np.maximum(np.abs(grad), gscale)), ("gradient", name)
        j = got["jvp_" + name].astype(np.float64).reshape(-1)
        assert np.all(np.abs(j - jvp.reshape(-1)) <= atol + rtol * np.maximum(np.abs(jvp.reshape(-1)), jscale)), ("jvp", name)
