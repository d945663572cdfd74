"""TEST INFRASTRUCTURE ONLY: numpy/ctypes access to the CPU checker.

Loads oracle/libkhan_oracle.so (own C restatement) and, when present, oracle/_ref/libkhan_ref.so (the
reference's kernel_cpu.cpp compiled in place).  Only tests/, the smoke check and the cpu_baseline leg of
bench.py may import this module; the product package never does.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
FEATS = 384

_vp = ctypes.c_void_p
_i32 = ctypes.c_int32


def _p(a):
    return _vp(a.ctypes.data) if a is not None else _vp(None)


def _load(path):
    if not os.path.exists(path):
        return None
    return ctypes.CDLL(path)


_oracle = {}
_ref = {}


def oracle_lib(fast=False):
    key = "fast" if fast else "strict"
    if key not in _oracle:
        name = "libkhan_oracle_fast.so" if fast else "libkhan_oracle.so"
        lib = _load(os.path.join(_HERE, name))
        if lib is None:
            raise RuntimeError("oracle/%s missing: run `make -C oracle`" % name)
        _oracle[key] = lib
    return _oracle[key]


def ref_lib(fast=False):
    """The compiled reference, or None where oracle/_ref was not built."""
    key = "fast" if fast else "strict"
    if key not in _ref:
        name = "libkhan_ref_fast.so" if fast else "libkhan_ref.so"
        _ref[key] = _load(os.path.join(_HERE, "_ref", name))
    return _ref[key]


def have_ref():
    return ref_lib() is not None


def _suffix(dtype):
    return {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}[np.dtype(dtype)]


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def ani_sort(A):
    A = _c(A, np.int32)
    sc = np.empty_like(A)
    ga = np.empty_like(A)
    counts = np.zeros(4, dtype=np.int32)
    rc = oracle_lib().khan_oracle_ani_sort(_p(A), ctypes.c_int64(A.size), _p(sc), _p(ga), _p(counts))
    if rc != 0:
        raise ValueError("atom types must be 0..3")
    return sc, ga, counts


def mol_offsets(mol_idxs, n_mols):
    m = _c(mol_idxs, np.int32)
    macs = np.zeros(n_mols, dtype=np.int32)
    mos = np.zeros(n_mols, dtype=np.int32)
    rc = oracle_lib().khan_oracle_mol_offsets(_p(m), ctypes.c_int64(m.size), _i32(n_mols), _p(macs), _p(mos))
    if rc != 0:
        raise ValueError("mol_idxs must be sorted and within [0, n_mols)")
    return macs, mos


def _split(acs, dtype):
    return [np.zeros(int(c) * FEATS, dtype=dtype) for c in acs]


def featurize(X, Y, Z, A, MOs, MACs, SIs, acs, dtype=np.float32, impl="oracle", fast=False,
              mol_range=None, out=None):
    """-> [h, c, n, o] flat arrays. impl: "oracle" (own restatement) or "ref" (compiled reference).

    mol_range=(lo, hi) restricts the work to molecules lo..hi-1 and accumulates into `out` without
    zeroing (used to shard the CPU baseline over threads)."""
    X, Y, Z = _c(X, dtype), _c(Y, dtype), _c(Z, dtype)
    A, MOs, MACs, SIs = _c(A, np.int32), _c(MOs, np.int32), _c(MACs, np.int32), _c(SIs, np.int32)
    acs = _c(acs, np.int32)
    outs = out if out is not None else _split(acs, dtype)
    lo, hi = mol_range if mol_range is not None else (0, MOs.size)
    mos_v, macs_v = MOs[lo:hi], MACs[lo:hi]
    sfx = _suffix(dtype)
    if impl == "ref":
        lib = ref_lib(fast)
        if lib is None:
            raise RuntimeError("oracle/_ref not built")
        if mol_range is not None:
            raise ValueError("the compiled reference entry zeroes its outputs; no mol_range")
        fn = getattr(lib, "ref_featurize_" + sfx)
        fn(_p(X), _p(Y), _p(Z), _p(A), _p(mos_v), _p(macs_v), _i32(hi - lo), _p(SIs),
           _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), _p(acs))
    else:
        fn = getattr(oracle_lib(fast), "khan_oracle_featurize_" + sfx)
        fn(_p(X), _p(Y), _p(Z), _p(A), _p(mos_v), _p(macs_v), _i32(hi - lo), _p(SIs),
           _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), _p(acs) if mol_range is None else _vp(None))
    return outs


def featurize_grad(X, Y, Z, A, MOs, MACs, SIs, acs, grads, dtype=np.float64, impl="oracle", fast=False):
    """grads = [gh, gc, gn, go] flat arrays -> (gx, gy, gz)."""
    X, Y, Z = _c(X, dtype), _c(Y, dtype), _c(Z, dtype)
    A, MOs, MACs, SIs = _c(A, np.int32), _c(MOs, np.int32), _c(MACs, np.int32), _c(SIs, np.int32)
    acs = _c(acs, np.int32)
    g = [_c(x, dtype).reshape(-1) for x in grads]
    n = X.size
    gx, gy, gz = (np.zeros(n, dtype=dtype) for _ in range(3))
    sfx = _suffix(dtype)
    if impl == "ref":
        lib = ref_lib(fast)
        if lib is None:
            raise RuntimeError("oracle/_ref not built")
        fn = getattr(lib, "ref_featurize_grad_" + sfx)
    else:
        fn = getattr(oracle_lib(fast), "khan_oracle_featurize_grad_" + sfx)
    fn(_p(X), _p(Y), _p(Z), _p(A), _p(MOs), _p(MACs), _i32(MOs.size), _p(SIs),
       _p(g[0]), _p(g[1]), _p(g[2]), _p(g[3]), _p(gx), _p(gy), _p(gz), _p(acs))
    return gx, gy, gz


def featurize_grad_inverse(X, Y, Z, A, MOs, MACs, SIs, acs, vX, vY, vZ, dtype=np.float64, impl="oracle", fast=False):
    """Jacobian applied to per-atom vectors v -> [h, c, n, o] flat buckets.  impl="ref" runs the
    reference's own routine (which reads v by atom type, not by atom)."""
    X, Y, Z = _c(X, dtype), _c(Y, dtype), _c(Z, dtype)
    vX, vY, vZ = _c(vX, dtype), _c(vY, dtype), _c(vZ, dtype)
    A, MOs, MACs, SIs = _c(A, np.int32), _c(MOs, np.int32), _c(MACs, np.int32), _c(SIs, np.int32)
    acs = _c(acs, np.int32)
    outs = [np.zeros(int(c) * FEATS, dtype=dtype) for c in acs]
    sfx = _suffix(dtype)
    if impl == "ref":
        lib = ref_lib(fast)
        if lib is None:
            raise RuntimeError("oracle/_ref not built")
        fn = getattr(lib, "ref_featurize_grad_inverse_" + sfx)
        fn(_p(X), _p(Y), _p(Z), _p(A), _p(MOs), _p(MACs), _i32(MOs.size), _p(SIs), _p(vX), _p(vY), _p(vZ),
           _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), _p(acs))
    else:
        fn = getattr(oracle_lib(fast), "khan_oracle_featurize_grad_inverse_" + sfx)
        fn(_p(X), _p(Y), _p(Z), _p(A), _p(MOs), _p(MACs), _i32(MOs.size), _p(SIs), _p(vX), _p(vY), _p(vZ),
           _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), _p(acs))
    return outs


def ani_charge(X, Y, Z, Q, MOs, MACs, dtype=np.float64):
    X, Y, Z, Q = _c(X, dtype), _c(Y, dtype), _c(Z, dtype), _c(Q, dtype)
    MOs, MACs = _c(MOs, np.int32), _c(MACs, np.int32)
    E = np.zeros(MOs.size, dtype=dtype)
    fn = getattr(oracle_lib(), "khan_oracle_ani_charge_" + _suffix(dtype))
    fn(_p(X), _p(Y), _p(Z), _p(Q), _p(MOs), _p(MACs), _i32(MOs.size), _p(E))
    return E


def ani_charge_grad(X, Y, Z, Q, MOs, MACs, grads, dtype=np.float64):
    X, Y, Z, Q = _c(X, dtype), _c(Y, dtype), _c(Z, dtype), _c(Q, dtype)
    MOs, MACs, grads = _c(MOs, np.int32), _c(MACs, np.int32), _c(grads, dtype)
    qg = np.zeros(X.size, dtype=dtype)
    fn = getattr(oracle_lib(), "khan_oracle_ani_charge_grad_" + _suffix(dtype))
    fn(_p(X), _p(Y), _p(Z), _p(Q), _p(MOs), _p(MACs), _i32(MOs.size), _p(grads), ctypes.c_int64(X.size), _p(qg))
    return qg


def ani_charge_grad_xyz(X, Y, Z, Q, MOs, MACs, grads, dtype=np.float64):
    X, Y, Z, Q = _c(X, dtype), _c(Y, dtype), _c(Z, dtype), _c(Q, dtype)
    MOs, MACs, grads = _c(MOs, np.int32), _c(MACs, np.int32), _c(grads, dtype)
    gx, gy, gz = (np.zeros(X.size, dtype=dtype) for _ in range(3))
    fn = getattr(oracle_lib(), "khan_oracle_ani_charge_grad_xyz_" + _suffix(dtype))
    fn(_p(X), _p(Y), _p(Z), _p(Q), _p(MOs), _p(MACs), _i32(MOs.size), _p(grads), _p(gx), _p(gy), _p(gz))
    return gx, gy, gz


def gather_rows(buckets, gather_idxs):
    """Concatenate the four buckets as [N,384] and reorder rows to original atom order
    (khan/training/trainer_multi_tower.py:324-334)."""
    packed = np.concatenate([b.reshape(-1, FEATS) for b in buckets], axis=0)
    return packed[np.asarray(gather_idxs)]


def scatter_rows(rows, A, SIs, acs):
    """Inverse of gather_rows: [N,384] in atom order -> four flat buckets."""
    rows = np.asarray(rows)
    outs = [np.zeros((int(c), FEATS), dtype=rows.dtype) for c in acs]
    for t in range(4):
        sel = np.nonzero(np.asarray(A) == t)[0]
        outs[t][np.asarray(SIs)[sel]] = rows[sel]
    return [o.reshape(-1) for o in outs]
