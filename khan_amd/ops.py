"""Python mirror of the reference's custom ops, same names and argument orders as `ani_mod.<op>(...)`:

    ani_sort(as)                                   gpu_featurizer/ani_sort.cpp:27-31
    featurize(xs, ys, zs, as, mos, macs, sis, acs)                 ani_op.cpp:95-107
    featurize_grad(..., acs, h_grads, c_grads, n_grads, o_grads)   ani_op.cpp:200-215
    featurize_grad_inverse(..., acs, x_grads, y_grads, z_grads)    ani_op.cpp:309-324
    ani_charge(xs, ys, zs, qs, mos, macs)                          ani_charges.cpp:45-52
    ani_charge_grad(xs, ys, zs, qs, mos, macs, grads)              ani_charges.cpp:123-131
    mol_offsets(mol_idxs, n_mols)   the segment_sum + exclusive cumsum the trainer runs first
                                    (khan/training/trainer_multi_tower.py:302-303)

Tensors are torch CUDA tensors (PyTorch only owns the device memory and the stream); every op
enqueues HIP kernels from libkhan_aev.so on the current stream.  Flat 1-D tensors in, flat 1-D tensors
out, float32 or float64, int32 indices -- as in the reference.  There is no CPU implementation here.
"""
import ctypes

import torch

from . import _lib

FEATURE_SIZE = 384

_SUFFIX = {torch.float32: "f32", torch.float64: "f64"}


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, dtype, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a CUDA tensor" % name)
    if t.dtype != dtype:
        raise TypeError("%s must have dtype %s, got %s" % (name, dtype, t.dtype))
    if t.dim() != 1:
        raise ValueError("%s must be rank 1 (flat), got shape %s" % (name, tuple(t.shape)))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    return t


def _p(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None and t.numel() > 0 else None)


def _float_dtype(x):
    if x.dtype not in _SUFFIX:
        raise TypeError("coordinates must be float32 or float64, got %s" % x.dtype)
    return x.dtype


def _acs_host(acs):
    """atom_counts lives in host memory in the reference (ani_op.cpp:333); a device tensor is copied."""
    if isinstance(acs, torch.Tensor):
        vals = [int(v) for v in acs.detach().cpu().tolist()]
    else:
        vals = [int(v) for v in acs]
    if len(vals) != 4:
        raise ValueError("acs must hold 4 atom counts")
    return (ctypes.c_int32 * 4)(*vals), vals


def mol_offsets(mol_idxs, n_mols):
    """-> (mol_atom_counts, mol_offsets), both int32[n_mols]; mol_idxs sorted ascending."""
    lib = _lib.load()
    mol_idxs = _dev(mol_idxs, torch.int32, "mol_idxs")
    macs = torch.empty(n_mols, dtype=torch.int32, device=mol_idxs.device)
    mos = torch.empty(n_mols, dtype=torch.int32, device=mol_idxs.device)
    _lib.check(lib.khan_mol_offsets(_p(mol_idxs), mol_idxs.numel(), n_mols, _p(macs), _p(mos), _stream()))
    return macs, mos


def ani_sort(atomic_numbers):
    """-> (scatter_idxs, gather_idxs, atom_counts); atom_counts is an int32[4] DEVICE tensor."""
    lib = _lib.load()
    a = _dev(atomic_numbers, torch.int32, "atomic_numbers")
    scatter = torch.empty_like(a)
    gather = torch.empty_like(a)
    counts = torch.empty(4, dtype=torch.int32, device=a.device)
    _lib.check(lib.khan_ani_sort(_p(a), a.numel(), _p(scatter), _p(gather), _p(counts), _stream()))
    return scatter, gather, counts


SIZE_ORDER_EXTRA = 520


def set_reproducible_gradients(on):
    """Process-wide: with True, `featurize_grad` sums the forces of molecules of up to 256 atoms in a fixed order (the
    same bits on every run, no atomics) at some cost in speed; returns the previous setting."""
    return bool(_lib.load().khan_set_reproducible_gradients(1 if on else 0))


def size_order(macs):
    """-> int32[n_mols + 520]: the molecule indices by decreasing atom count and the per-size counts, to be
    passed as `order=` to featurize / featurize_grad / featurize_grad_inverse of the same batch (computed once
    per batch instead of once per call; the calls then allocate nothing -- except the sorted copy of molecules of more
    than 256 atoms, where a batch holds any -- and can be captured into a graph).
    Its last four elements (`order[-4:]`) count the molecules of up to 32, 33..64, 65..256 and more atoms: copied
    to the host and passed as `size_classes=`, they spare the passes the launches of kernels without work."""
    lib = _lib.load()
    macs = _dev(macs, torch.int32, "macs")
    order = torch.empty(macs.numel() + SIZE_ORDER_EXTRA, dtype=torch.int32, device=macs.device)
    _lib.check(lib.khan_size_order(_p(macs), macs.numel(), _p(order), _stream()))
    return order


def _order_arg(order, macs):
    order = _dev(order, torch.int32, "order")
    if order.numel() != macs.numel() + SIZE_ORDER_EXTRA:
        raise ValueError("order must come from size_order(macs) of this batch")
    return order


def _classes_arg(size_classes):
    """host copy of order[-4:] (a CPU tensor or 4 ints), or None"""
    if size_classes is None:
        return None
    vals = [int(v) for v in (size_classes.tolist() if isinstance(size_classes, torch.Tensor) else size_classes)]
    if len(vals) != 4:
        raise ValueError("size_classes must hold 4 counts")
    return (ctypes.c_int32 * 4)(*vals)


def _check_common(xs, ys, zs, as_, mos, macs, sis):
    dt = _float_dtype(xs)
    _dev(xs, dt, "xs"); _dev(ys, dt, "ys"); _dev(zs, dt, "zs")
    _dev(as_, torch.int32, "as"); _dev(mos, torch.int32, "mos"); _dev(macs, torch.int32, "macs")
    _dev(sis, torch.int32, "sis")
    n = xs.numel()
    if not (ys.numel() == n and zs.numel() == n and as_.numel() == n and sis.numel() == n):
        raise ValueError("xs, ys, zs, as, sis must have the same length")
    if mos.numel() != macs.numel():
        raise ValueError("mos and macs must have the same length")
    return dt, n


def featurize(xs, ys, zs, as_, mos, macs, sis, acs, order=None, size_classes=None):
    """-> (h_feat, c_feat, n_feat, o_feat), flat tensors of acs[t]*384 elements.

    The four outputs are consecutive slices of one allocation, so
    ``torch.cat([h, c, n, o]).view(-1, 384)[gather_idxs]`` needs no copy for the concatenation.
    """
    lib = _lib.load()
    dt, n = _check_common(xs, ys, zs, as_, mos, macs, sis)
    acs_c, acs_v = _acs_host(acs)
    if sum(acs_v) != n:
        raise ValueError("sum(acs)=%d does not match the number of atoms %d" % (sum(acs_v), n))
    packed = torch.empty(n * FEATURE_SIZE, dtype=dt, device=xs.device)
    outs, start = [], 0
    for c in acs_v:
        outs.append(packed[start * FEATURE_SIZE:(start + c) * FEATURE_SIZE])
        start += c
    args = (_p(xs), _p(ys), _p(zs), _p(as_), _p(mos), _p(macs), mos.numel(), _p(sis),
            _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), acs_c)
    if order is None:
        _lib.check(getattr(lib, "khan_featurize_" + _SUFFIX[dt])(*args, _stream()))
    else:
        _lib.check(getattr(lib, "khan_featurize_ordered_" + _SUFFIX[dt])(*args, _p(_order_arg(order, macs)), _classes_arg(size_classes), _stream()))
    return tuple(outs)


def featurize_grad(xs, ys, zs, as_, mos, macs, sis, acs, h_grads, c_grads, n_grads, o_grads, order=None, size_classes=None):
    """-> (x_grads, y_grads, z_grads), each [n_atoms] in original atom order."""
    lib = _lib.load()
    dt, n = _check_common(xs, ys, zs, as_, mos, macs, sis)
    acs_c, acs_v = _acs_host(acs)
    if sum(acs_v) != n:
        raise ValueError("sum(acs)=%d does not match the number of atoms %d" % (sum(acs_v), n))
    grads = []
    for name, g, c in zip("hcno", (h_grads, c_grads, n_grads, o_grads), acs_v):
        g = _dev(g.reshape(-1), dt, name + "_grads")
        if g.numel() != c * FEATURE_SIZE:
            raise ValueError("%s_grads has %d elements, expected %d" % (name, g.numel(), c * FEATURE_SIZE))
        grads.append(g)
    gx = torch.empty(n, dtype=dt, device=xs.device)
    gy = torch.empty_like(gx)
    gz = torch.empty_like(gx)
    args = (_p(xs), _p(ys), _p(zs), _p(as_), _p(mos), _p(macs), mos.numel(), _p(sis),
            _p(grads[0]), _p(grads[1]), _p(grads[2]), _p(grads[3]), _p(gx), _p(gy), _p(gz), acs_c)
    if order is None:
        _lib.check(getattr(lib, "khan_featurize_grad_" + _SUFFIX[dt])(*args, _stream()))
    else:
        _lib.check(getattr(lib, "khan_featurize_grad_ordered_" + _SUFFIX[dt])(*args, _p(_order_arg(order, macs)), _classes_arg(size_classes), _stream()))
    return gx, gy, gz


def featurize_grad_inverse(xs, ys, zs, as_, mos, macs, sis, acs, x_grads, y_grads, z_grads, order=None, size_classes=None):
    """-> (h_grads, c_grads, n_grads, o_grads) laid out like `featurize`'s outputs: the Jacobian of the
    features applied to one vector per atom, row_i[f] = sum_a dAEV_i[f]/dxyz_a . (x,y,z)_grads[a].
    It is the gradient of `featurize_grad` with respect to its upstream gradients
    (khan/training/trainer_multi_tower.py:64-91)."""
    lib = _lib.load()
    dt, n = _check_common(xs, ys, zs, as_, mos, macs, sis)
    acs_c, acs_v = _acs_host(acs)
    if sum(acs_v) != n:
        raise ValueError("sum(acs)=%d does not match the number of atoms %d" % (sum(acs_v), n))
    vs = []
    for name, v in zip("xyz", (x_grads, y_grads, z_grads)):
        v = _dev(v, dt, name + "_grads")
        if v.numel() != n:
            raise ValueError("%s_grads has %d elements, expected %d" % (name, v.numel(), n))
        vs.append(v)
    packed = torch.empty(n * FEATURE_SIZE, dtype=dt, device=xs.device)
    outs, start = [], 0
    for c in acs_v:
        outs.append(packed[start * FEATURE_SIZE:(start + c) * FEATURE_SIZE])
        start += c
    args = (_p(xs), _p(ys), _p(zs), _p(as_), _p(mos), _p(macs), mos.numel(), _p(sis),
            _p(vs[0]), _p(vs[1]), _p(vs[2]), _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]), acs_c)
    if order is None:
        _lib.check(getattr(lib, "khan_featurize_grad_inverse_" + _SUFFIX[dt])(*args, _stream()))
    else:
        _lib.check(getattr(lib, "khan_featurize_grad_inverse_ordered_" + _SUFFIX[dt])(*args, _p(_order_arg(order, macs)), _classes_arg(size_classes), _stream()))
    return tuple(outs)


def _check_charge(xs, ys, zs, qs, mos, macs):
    dt = _float_dtype(xs)
    for name, t in (("xs", xs), ("ys", ys), ("zs", zs), ("qs", qs)):
        _dev(t, dt, name)
    _dev(mos, torch.int32, "mos"); _dev(macs, torch.int32, "macs")
    n = xs.numel()
    if not (ys.numel() == n and zs.numel() == n and qs.numel() == n):
        raise ValueError("xs, ys, zs, qs must have the same length")
    if mos.numel() != macs.numel():
        raise ValueError("mos and macs must have the same length")
    return dt, n


def ani_charge(xs, ys, zs, qs, mos, macs):
    """-> charge_energies[n_mols]"""
    lib = _lib.load()
    dt, _ = _check_charge(xs, ys, zs, qs, mos, macs)
    e = torch.empty(mos.numel(), dtype=dt, device=xs.device)
    fn = getattr(lib, "khan_ani_charge_" + _SUFFIX[dt])
    _lib.check(fn(_p(xs), _p(ys), _p(zs), _p(qs), _p(mos), _p(macs), mos.numel(), _p(e), _stream()))
    return e


def ani_charge_grad(xs, ys, zs, qs, mos, macs, grads):
    """-> q_grads[n_atoms]"""
    lib = _lib.load()
    dt, n = _check_charge(xs, ys, zs, qs, mos, macs)
    grads = _dev(grads, dt, "grads")
    if grads.numel() != mos.numel():
        raise ValueError("grads must have one element per molecule")
    qg = torch.zeros(n, dtype=dt, device=xs.device)
    fn = getattr(lib, "khan_ani_charge_grad_" + _SUFFIX[dt])
    _lib.check(fn(_p(xs), _p(ys), _p(zs), _p(qs), _p(mos), _p(macs), mos.numel(), _p(grads), _p(qg), _stream()))
    return qg


def ani_charge_grad_xyz(xs, ys, zs, qs, mos, macs, grads):
    """-> (q_grads, x_grads, y_grads, z_grads); the coordinate gradient is not offered by the reference."""
    lib = _lib.load()
    dt, n = _check_charge(xs, ys, zs, qs, mos, macs)
    grads = _dev(grads, dt, "grads")
    if grads.numel() != mos.numel():
        raise ValueError("grads must have one element per molecule")
    qg = torch.zeros(n, dtype=dt, device=xs.device)
    gx = torch.zeros(n, dtype=dt, device=xs.device)
    gy = torch.zeros_like(gx)
    gz = torch.zeros_like(gx)
    fn = getattr(lib, "khan_ani_charge_grad_xyz_" + _SUFFIX[dt])
    _lib.check(fn(_p(xs), _p(ys), _p(zs), _p(qs), _p(mos), _p(macs), mos.numel(), _p(grads), _p(qg),
                  _p(gx), _p(gy), _p(gz), _stream()))
    return qg, gx, gy, gz


def ani_charge_all(xs, ys, zs, qs, mos, macs, grads):
    """`ani_charge` and `ani_charge_grad_xyz` in one pass over the pairs
    -> (charge_energies, q_grads, x_grads, y_grads, z_grads); the energies are not multiplied by `grads`."""
    lib = _lib.load()
    dt, n = _check_charge(xs, ys, zs, qs, mos, macs)
    grads = _dev(grads, dt, "grads")
    if grads.numel() != mos.numel():
        raise ValueError("grads must have one element per molecule")
    e = torch.zeros(mos.numel(), dtype=dt, device=xs.device)
    qg = torch.zeros(n, dtype=dt, device=xs.device)
    gx = torch.zeros(n, dtype=dt, device=xs.device)
    gy = torch.zeros_like(gx)
    gz = torch.zeros_like(gx)
    fn = getattr(lib, "khan_ani_charge_all_" + _SUFFIX[dt])
    _lib.check(fn(_p(xs), _p(ys), _p(zs), _p(qs), _p(mos), _p(macs), mos.numel(), _p(grads), _p(e), _p(qg),
                  _p(gx), _p(gy), _p(gz), _stream()))
    return e, qg, gx, gy, gz


def mol_energy(type_outputs, atom_types, sis, mos, macs):
    """Per-molecule sums of the four per-type output vectors (`type_outputs[t]` is [acs[t]], float32 or float64; atom
    g's value is type_outputs[as[g]][sis[g]]) -> [n_mols]: the reference's gather to atom order + segment_sum by
    molecule (khan/model/nn.py:165-177) in one launch, summed in a fixed order."""
    lib = _lib.load()
    dt = type_outputs[0].dtype
    if dt not in _SUFFIX:
        raise TypeError("type_outputs must be float32 or float64, got %s" % dt)
    outs = [_dev(o.reshape(-1), dt, "type_outputs[%d]" % t) for t, o in enumerate(type_outputs)]
    if len(outs) != 4:
        raise ValueError("type_outputs must hold the four per-type vectors")
    a, s_, mo, ma = (_dev(v, torch.int32, n) for v, n in ((atom_types, "atom_types"), (sis, "sis"), (mos, "mos"), (macs, "macs")))
    if sum(o.numel() for o in outs) != a.numel() or s_.numel() != a.numel() or mo.numel() != ma.numel():
        raise ValueError("the four vectors must hold one value per atom, and mos / macs one entry per molecule")
    e = torch.empty(ma.numel(), dtype=dt, device=a.device)
    fn = getattr(lib, "khan_mol_energy_" + _SUFFIX[dt])
    _lib.check(fn(_ptr4(outs), _p(a), _p(s_), _p(mo), _p(ma), ma.numel(), _p(e), _stream()))
    return e


def mol_energy_grad(e_grads, atom_types, sis, mos, macs, acs):
    """The way back through `mol_energy`: -> four vectors [acs[t]] with grad_t[sis[g]] = e_grads[molecule of g]."""
    lib = _lib.load()
    dt = e_grads.dtype
    if dt not in _SUFFIX:
        raise TypeError("e_grads must be float32 or float64, got %s" % dt)
    eg = _dev(e_grads, dt, "e_grads")
    a, s_, mo, ma = (_dev(v, torch.int32, n) for v, n in ((atom_types, "atom_types"), (sis, "sis"), (mos, "mos"), (macs, "macs")))
    counts = _acs_host(acs)[1]
    if sum(counts) != a.numel() or s_.numel() != a.numel() or mo.numel() != ma.numel() or eg.numel() != ma.numel():
        raise ValueError("acs must add up to the number of atoms, and e_grads / mos / macs hold one entry per molecule")
    # one cleared array cut into the four vectors (atoms outside every molecule keep 0)
    outs = list(torch.zeros(sum(counts), dtype=dt, device=a.device).split(counts))
    fn = getattr(lib, "khan_mol_energy_grad_" + _SUFFIX[dt])
    _lib.check(fn(_p(eg), _p(a), _p(s_), _p(mo), _p(ma), ma.numel(), _ptr4(outs), _stream()))
    return tuple(outs)


def coulomb(xs, ys, zs, qs, mos, macs, k=1.0):
    """-> energies[n_mols] = k * sum_{i<j} q_i q_j / r_ij: the charge kernel without the reference's damping
    and constant (the reference's op is `ani_charge`)."""
    lib = _lib.load()
    dt, _ = _check_charge(xs, ys, zs, qs, mos, macs)
    e = torch.empty(mos.numel(), dtype=dt, device=xs.device)
    fn = getattr(lib, "khan_coulomb_" + _SUFFIX[dt])
    _lib.check(fn(_p(xs), _p(ys), _p(zs), _p(qs), _p(mos), _p(macs), mos.numel(), float(k), _p(e), _stream()))
    return e


def coulomb_grad(xs, ys, zs, qs, mos, macs, grads, k=1.0):
    """-> (q_grads, x_grads, y_grads, z_grads) of `coulomb`, weighted by grads[n_mols]."""
    lib = _lib.load()
    dt, n = _check_charge(xs, ys, zs, qs, mos, macs)
    grads = _dev(grads, dt, "grads")
    if grads.numel() != mos.numel():
        raise ValueError("grads must have one element per molecule")
    qg = torch.zeros(n, dtype=dt, device=xs.device)
    gx = torch.zeros(n, dtype=dt, device=xs.device)
    gy = torch.zeros_like(gx)
    gz = torch.zeros_like(gx)
    fn = getattr(lib, "khan_coulomb_grad_" + _SUFFIX[dt])
    _lib.check(fn(_p(xs), _p(ys), _p(zs), _p(qs), _p(mos), _p(macs), mos.numel(), _p(grads), float(k), _p(qg),
                  _p(gx), _p(gy), _p(gz), _stream()))
    return qg, gx, gy, gz


ACT_NONE, ACT_CELU = 0, 1


def dense(inputs, weights_nk, biases=None, activation=ACT_NONE, alpha=0.1, deriv_of=None):
    """A dense layer of the four atomic networks, forward or on the way back, float32, one launch:
    -> four [n_t, n_out] tensors act(in_t' . W_t + b_t), with in_t' = inputs[t] ([n_t, k]) or, with `deriv_of`, inputs[t]
    times the CELU derivative taken from the activations deriv_of[t] ([n_t, k]).  `weights_nk[t]` is [n_out, k]
    (the summed index contiguous): a layer's weights transposed for its forward pass, the weights as they are for
    its data gradient.  k a multiple of 32, n_out a multiple of 64."""
    lib = _lib.load()
    n_out, k = (int(v) for v in weights_nk[0].shape)
    rows, ders, wts, bs, outs, ns = [], [], [], [], [], []
    for t in range(4):
        r = _dense_matrix(inputs[t], k, "inputs[%d]" % t)
        wts.append(_dense_weights(weights_nk[t], n_out, k, "weights_nk[%d]" % t))
        if deriv_of is not None:
            d = _dense_matrix(deriv_of[t], k, "deriv_of[%d]" % t)
            if d.shape[0] != r.shape[0]:
                raise ValueError("deriv_of[%d] must be shaped like inputs[%d]" % (t, t))
            ders.append(d)
        if biases is not None:
            b = _dev(biases[t], torch.float32, "bias")
            if b.numel() != n_out:
                raise ValueError("bias %d must have %d elements" % (t, n_out))
            bs.append(b)
        rows.append(r); ns.append(int(r.shape[0]))
        outs.append(torch.empty((r.shape[0], n_out), dtype=torch.float32, device=r.device))
    _lib.check(lib.khan_dense_f32(_ptr4(rows), (ctypes.c_int32 * 4)(*ns), k, n_out, _ptr4(wts),
                                  _ptr4(bs) if biases is not None else None, int(activation), float(alpha),
                                  _ptr4(ders) if deriv_of is not None else None, _ptr4(outs), _stream()))
    return tuple(outs)


def _dense_matrix(x, k, name):
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != torch.float32:
        raise TypeError("%s must be a float32 CUDA tensor" % name)
    if x.dim() != 2 or x.shape[1] != k or not x.is_contiguous():
        raise ValueError("%s must be a contiguous [n, %d] tensor, got %s" % (name, k, tuple(x.shape)))
    return x


def _dense_weights(w, n_out, k, name):
    if tuple(w.shape) != (n_out, k) or w.dtype != torch.float32 or not w.is_contiguous() or not w.is_cuda:
        raise ValueError("%s must be a contiguous float32 CUDA tensor of shape [%d, %d]" % (name, n_out, k))
    return w


def _ptr4(ts):
    return (ctypes.c_void_p * 4)(*[t.data_ptr() if t.numel() else None for t in ts])


def dense_head(inputs, weights_nk, biases, head_weights, head_biases=None, activation=ACT_CELU, alpha=0.1):
    """The last hidden layer of the four atomic networks (width 64) with the output layer (64 -> 1, no activation)
    folded into the same launch, float32: -> (outs, head_outs), outs[t] = act(inputs[t] . W_t + b_t) as `dense`
    gives it ([n_t, 64]; the way back needs it) and head_outs[t][r] = outs[t][r, :] . head_weights[t] + head_biases[t]
    ([n_t]).  `weights_nk[t]` is [64, k]; `head_weights[t]` has 64 elements, `head_biases[t]` one."""
    lib = _lib.load()
    n_out, k = (int(v) for v in weights_nk[0].shape)
    if n_out != 64:
        raise ValueError("the fused output layer needs a last hidden layer of width 64, got %d" % n_out)
    rows, wts, bs, hws, hbs, outs, houts, ns = [], [], [], [], [], [], [], []
    for t in range(4):
        r = _dense_matrix(inputs[t], k, "inputs[%d]" % t)
        wts.append(_dense_weights(weights_nk[t], n_out, k, "weights_nk[%d]" % t))
        if biases is not None:
            b = _dev(biases[t], torch.float32, "bias")
            if b.numel() != n_out:
                raise ValueError("bias %d must have %d elements" % (t, n_out))
            bs.append(b)
        hw = _dev(head_weights[t].reshape(-1), torch.float32, "head_weights")
        if hw.numel() != n_out:
            raise ValueError("head_weights[%d] must have %d elements" % (t, n_out))
        hws.append(hw)
        if head_biases is not None:
            hb = _dev(head_biases[t].reshape(-1), torch.float32, "head_biases")
            if hb.numel() != 1:
                raise ValueError("head_biases[%d] must have one element" % t)
            hbs.append(hb)
        rows.append(r); ns.append(int(r.shape[0]))
        outs.append(torch.empty((r.shape[0], n_out), dtype=torch.float32, device=r.device))
        houts.append(torch.empty((r.shape[0],), dtype=torch.float32, device=r.device))
    _lib.check(lib.khan_dense_head_f32(_ptr4(rows), (ctypes.c_int32 * 4)(*ns), k, n_out, _ptr4(wts),
                                       _ptr4(bs) if biases is not None else None, int(activation), float(alpha),
                                       _ptr4(hws), _ptr4(hbs) if head_biases is not None else None, _ptr4(outs),
                                       _ptr4(houts), _stream()))
    return tuple(outs), tuple(houts)


def dense_head_grad(scales, head_weights, weights_nk, deriv_of, alpha=0.1):
    """The way back through the output layer and the last hidden layer, float32, one launch: given scales[t] ([n_t],
    the gradient with respect to each row's output value), -> four [n_t, n_out] tensors
    (scales[t][:, None] * head_weights[t][None, :] * CELU'(z)) . W_t, CELU(z) = deriv_of[t] ([n_t, k], the hidden
    layer's activations); `weights_nk[t]` is [n_out, k], the hidden layer's weights as stored (input width x layer
    width).  The outer product is formed inside the kernel."""
    lib = _lib.load()
    n_out, k = (int(v) for v in weights_nk[0].shape)
    scs, hws, wts, ders, outs, ns = [], [], [], [], [], []
    for t in range(4):
        d = _dense_matrix(deriv_of[t], k, "deriv_of[%d]" % t)
        sc = _dev(scales[t].reshape(-1), torch.float32, "scales")
        if sc.numel() != d.shape[0]:
            raise ValueError("scales[%d] must have %d elements" % (t, d.shape[0]))
        hw = _dev(head_weights[t].reshape(-1), torch.float32, "head_weights")
        if hw.numel() != k:
            raise ValueError("head_weights[%d] must have %d elements" % (t, k))
        wts.append(_dense_weights(weights_nk[t], n_out, k, "weights_nk[%d]" % t))
        scs.append(sc); hws.append(hw); ders.append(d); ns.append(int(d.shape[0]))
        outs.append(torch.empty((d.shape[0], n_out), dtype=torch.float32, device=d.device))
    _lib.check(lib.khan_dense_head_grad_f32(_ptr4(scs), _ptr4(hws), (ctypes.c_int32 * 4)(*ns), k, n_out, _ptr4(wts),
                                            float(alpha), _ptr4(ders), _ptr4(outs), _stream()))
    return tuple(outs)


NETWORK_WIDTHS = (384, 128, 128, 64)      # the layer widths `atomic_networks` is built for (then 64 -> 1)


_NETWORK_SHAPES_T = ((128, 384), (128, 128), (64, 128))


def pack_network_weights(weights_t, weights):
    """The 24 weight matrices of `atomic_networks` (weights_t[l][t] transposed, weights[l][t] as stored) split once into
    their half-precision parts: -> a uint8 device buffer to pass as `packed=`.  Pack again after the weights change."""
    lib = _lib.load()
    wts, ws = [], []
    for l in range(3):
        for t in range(4):
            n_out, k = _NETWORK_SHAPES_T[l]
            wts.append(_dense_weights(weights_t[l][t], n_out, k, "weights_t[%d][%d]" % (l, t)))
            ws.append(_dense_weights(weights[l][t], k, n_out, "weights[%d][%d]" % (l, t)))
    packed = torch.empty(int(lib.khan_atomic_networks_packed_bytes()), dtype=torch.uint8, device=wts[0].device)
    p12 = lambda ts: (ctypes.c_void_p * 12)(*[t.data_ptr() for t in ts])
    _lib.check(lib.khan_atomic_networks_pack_f32(p12(wts), p12(ws), _p(packed), _stream()))
    return packed


def atomic_networks(rows, weights_t, biases, head_weights, head_biases=None, weights=None, scales=None, want_grad=False,
                    alpha=0.1, packed=None):
    """The 384-128-128-64-1 CELU networks of the four atom types in one launch, float32: -> (values, grads).
    values[t] is [n_t], the network's output for every feature row of rows[t] ([n_t, 384] or a flat bucket); with
    `want_grad`, grads[t] ([n_t, 384]) is scales[t][:, None] * d values[t] / d rows[t] (scales None: ones), formed in
    the same launch without any hidden layer's activations going to memory; otherwise grads is None.
    weights_t[l][t]: layer l = 0, 1, 2 transposed ([128, 384], [128, 128], [64, 128]); weights[l][t]: the same layers as
    stored ([384, 128], [128, 128], [128, 64]; needed with want_grad); or `packed` = pack_network_weights(...) of the
    same matrices (then weights_t and weights may be None).  biases[l][t]; head_weights[t] (64 values),
    head_biases[t] (one value).  The products are float32 products to float32 accuracy from two half-precision parts
    per operand: features, activations and weights have to stay below 65,504 in size (beyond it the row's results are
    NaN); the size of `scales` does not matter."""
    lib = _lib.load()
    xs, ns, vals, grads = [], [], [], []
    for t in range(4):
        x = _dense_matrix(rows[t].reshape(-1, 384), 384, "rows[%d]" % t)
        xs.append(x)
        ns.append(int(x.shape[0]))
        vals.append(torch.empty(x.shape[0], dtype=torch.float32, device=x.device))
        if want_grad:
            grads.append(torch.empty((x.shape[0], 384), dtype=torch.float32, device=x.device))
    wts, ws, bs = [], [], []
    for l in range(3):
        for t in range(4):
            n_out, k = _NETWORK_SHAPES_T[l]
            bs.append(_dev(biases[l][t].reshape(-1), torch.float32, "biases"))
            if bs[-1].numel() != n_out:
                raise ValueError("biases[%d][%d] must have %d elements" % (l, t, n_out))
            if packed is None:
                wts.append(_dense_weights(weights_t[l][t], n_out, k, "weights_t[%d][%d]" % (l, t)))
                if want_grad:
                    ws.append(_dense_weights(weights[l][t], k, n_out, "weights[%d][%d]" % (l, t)))
    if packed is not None and (packed.dtype != torch.uint8 or not packed.is_cuda
                               or packed.numel() != int(lib.khan_atomic_networks_packed_bytes())):
        raise ValueError("packed must be the buffer pack_network_weights returned")
    hws = [_dev(h.reshape(-1), torch.float32, "head_weights") for h in head_weights]
    if any(h.numel() != 64 for h in hws):
        raise ValueError("head_weights must have 64 elements each")
    hbs = None if head_biases is None else [_dev(h.reshape(-1), torch.float32, "head_biases") for h in head_biases]
    scs = None
    if scales is not None:
        scs = [_dev(sc.reshape(-1), torch.float32, "scales") for sc in scales]
        if any(sc.numel() != n for sc, n in zip(scs, ns)):
            raise ValueError("scales[t] must have one element per row")
    p12 = lambda ts: (ctypes.c_void_p * 12)(*[t.data_ptr() for t in ts])
    _lib.check(lib.khan_atomic_networks_f32(_ptr4(xs), (ctypes.c_int32 * 4)(*ns), p12(wts) if wts else None,
                                            p12(ws) if ws else None, None if packed is None else _p(packed),
                                            p12(bs), _ptr4(hws), None if hbs is None else _ptr4(hbs),
                                            None if scs is None else _ptr4(scs), float(alpha), _ptr4(vals),
                                            _ptr4(grads) if want_grad else None, _stream()))
    return tuple(vals), (tuple(grads) if want_grad else None)


def dense_first(atom_type_features, acs, weights_t, biases, activation=ACT_CELU, alpha=0.1):
    """First dense layer of the four atomic networks on the featurizer's buckets, float32, one launch:
    -> four [acs[t], 128] tensors act(rows_t . W_t + b_t).  `weights_t[t]` is W_t TRANSPOSED, [128, 384]."""
    lib = _lib.load()
    acs_c, acs_v = _acs_host(acs)
    rows, wts, bs, outs = [], [], [], []
    for t in range(4):
        r = _dev(atom_type_features[t].reshape(-1), torch.float32, "features")
        if r.numel() != acs_v[t] * FEATURE_SIZE:
            raise ValueError("bucket %d has %d elements, expected %d" % (t, r.numel(), acs_v[t] * FEATURE_SIZE))
        w = weights_t[t]
        if tuple(w.shape) != (128, FEATURE_SIZE) or w.dtype != torch.float32 or not w.is_contiguous() or not w.is_cuda:
            raise ValueError("weights_t[%d] must be a contiguous float32 CUDA tensor of shape [128, 384]" % t)
        b = _dev(biases[t], torch.float32, "bias")
        if b.numel() != 128:
            raise ValueError("bias %d must have 128 elements" % t)
        rows.append(r); wts.append(w); bs.append(b)
        outs.append(torch.empty((acs_v[t], 128), dtype=torch.float32, device=r.device))
    arr = lambda ts: (ctypes.c_void_p * 4)(*[t.data_ptr() if t.numel() else None for t in ts])
    _lib.check(lib.khan_dense_first_f32(arr(rows), acs_c, arr(wts), arr(bs), int(activation), float(alpha), arr(outs), _stream()))
    return tuple(outs)
