"""TEST INFRASTRUCTURE: numpy restatement of the reference's atomic networks and of the energy / gradient a
molecule gets from them.  Only tests, the smoke check and the benchmark's CPU leg may import this.

Follows khan/model/nn.py:62-68 (A_k = act(A_{k-1} W_k + b_k), no activation on the last layer),
nn.py:176-177 (concatenate the per-type outputs, gather into atom order),
khan/training/trainer_multi_tower.py:350 (segment_sum over molecules) and 401 (gradient with respect to the
coordinates), khan/model/activations.py:63-77 (celu, normal, gaussian, softplus).

Pinned by tests that do not retype these formulas: finite differences of the forward for every derivative,
zero-weight and single-layer closed forms, and the known values and limits of the activation functions.
"""
import numpy as np

from . import binding

FEATURE_SIZE = 384


def _celu(a, alpha=0.1):
    pos = (a >= 0) * a
    neg = (a < 0) * a
    return pos + alpha * (np.exp(neg / alpha) - 1.0)


def _celu_grad(a, alpha=0.1):
    return np.where(a >= 0, 1.0, np.exp(np.minimum(a, 0.0) / alpha))


ACTIVATIONS = {
    "celu": (_celu, _celu_grad),
    "normal": (lambda a: np.exp(-a ** 2 / 2.0), lambda a: -a * np.exp(-a ** 2 / 2.0)),
    "gaussian": (lambda a: np.exp(-a ** 2), lambda a: -2.0 * a * np.exp(-a ** 2)),
    "softplus": (lambda a: np.logaddexp(0.0, a) - 0.69314718056, lambda a: 1.0 / (1.0 + np.exp(-a))),
}


def atom_nn_forward(feats, Ws, bs, activation="celu"):
    """feats [n, in] -> (outputs [n], pre-activations per layer)."""
    act = ACTIVATIONS[activation][0]
    a = np.asarray(feats)
    pre = []
    for k, (W, b) in enumerate(zip(Ws, bs)):
        z = a @ W + b
        pre.append((a, z))
        a = act(z) if k != len(Ws) - 1 else z
    return a.reshape(-1), pre


def atom_nn_backward(pre, Ws, upstream, activation="celu"):
    """d (sum upstream * outputs) / d feats, [n, in]."""
    dact = ACTIVATIONS[activation][1]
    g = np.asarray(upstream).reshape(-1, 1)
    for k in range(len(Ws) - 1, -1, -1):
        _, z = pre[k]
        if k != len(Ws) - 1:
            g = g * dact(z)
        g = g @ Ws[k].T
    return g


def split_params(params, prefix, layer_sizes):
    """name -> array dict  ->  per type ([W...], [b...]) with the reference's variable names (nn.py:41)."""
    sizes = (FEATURE_SIZE,) + tuple(layer_sizes)
    out = []
    for t in ("H", "C", "N", "O"):
        Ws, bs = [], []
        for idx in range(1, len(sizes)):
            name = "_%s_%dx%d_l%d:0" % (t, sizes[idx - 1], sizes[idx], idx)
            Ws.append(np.asarray(params[prefix + "W" + name]))
            bs.append(np.asarray(params[prefix + "b" + name]))
        out.append((Ws, bs))
    return out


def energies_and_gradients(X, Y, Z, A, MOs, MACs, params, layer_sizes, activation="celu", dtype=np.float64,
                           need_grad=True, fit_charges=False):
    """Per-molecule energies [n_mols] and d (sum of energies) / d xyz [n_atoms, 3].  With fit_charges the
    `charge_` networks give per-atom charges whose pairwise energy is added
    (trainer_multi_tower.py:352-385); its gradient reaches the coordinates directly and through the charges."""
    X, Y, Z = (np.ascontiguousarray(v, dtype=dtype) for v in (X, Y, Z))
    A = np.ascontiguousarray(A, dtype=np.int32)
    scatter, gather, acs = binding.ani_sort(A)
    feats = binding.featurize(X, Y, Z, A, MOs, MACs, scatter, acs, dtype=dtype)
    rows = [np.asarray(feats[t], dtype=dtype).reshape(-1, FEATURE_SIZE) for t in range(4)]

    def run(prefix):
        nets = [([w.astype(dtype) for w in Ws], [b.astype(dtype) for b in bs])
                for Ws, bs in split_params(params, prefix, layer_sizes)]
        outs, pres = zip(*(atom_nn_forward(rows[t], nets[t][0], nets[t][1], activation) for t in range(4)))
        return nets, outs, pres

    nets, outs, pres = run("near_")
    mol_idxs = np.repeat(np.arange(len(MACs)), MACs)
    energies = np.zeros(len(MACs), dtype=dtype)
    np.add.at(energies, mol_idxs, np.concatenate(outs)[gather])
    if fit_charges:
        qnets, qouts, qpres = run("charge_")
        qs = np.ascontiguousarray(np.concatenate(qouts)[gather], dtype=dtype)
        energies = energies + binding.ani_charge(X, Y, Z, qs, MOs, MACs, dtype=dtype)
    if not need_grad:
        return energies, None
    ups = [atom_nn_backward(pres[t], nets[t][0], np.ones(len(outs[t]), dtype=dtype), activation) for t in range(4)]
    direct = np.zeros((X.size, 3), dtype=dtype)
    if fit_charges:
        ones = np.ones(len(MACs), dtype=dtype)
        dq = binding.ani_charge_grad(X, Y, Z, qs, MOs, MACs, ones, dtype=dtype)          # per atom, atom order
        # atom i takes element gather[i] of the concatenated per-type outputs, so that element gets atom i's dq
        by_type = np.zeros(X.size, dtype=dtype)
        by_type[gather] = dq
        start = 0
        for t in range(4):
            n_t = len(qouts[t])
            ups[t] = ups[t] + atom_nn_backward(qpres[t], qnets[t][0], by_type[start:start + n_t], activation)
            start += n_t
        direct = np.stack(binding.ani_charge_grad_xyz(X, Y, Z, qs, MOs, MACs, ones, dtype=dtype), axis=1)
    ups = [np.ascontiguousarray(g.reshape(-1), dtype=dtype) for g in ups]
    gx, gy, gz = binding.featurize_grad(X, Y, Z, A, MOs, MACs, scatter, acs, ups, dtype=dtype)
    return energies, np.stack((gx, gy, gz), axis=1) + direct
