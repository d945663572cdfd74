"""The per-type atomic networks behind the featurizer, their npz checkpoint format, and batched inference.

Mirror of khan/model/nn.py (AtomNN 3-88, MoleculeNN 122-201), of the activation functions in
khan/model/activations.py:63-77, and of the inference half of khan/training/trainer_multi_tower.py:
save_numpy / load_numpy (451-499), predict (655-678), coordinate_gradients (580-615), and the tower wiring
features -> per-type networks -> gather -> segment_sum (+ ani_charge) of lines 306-385.

The featurizer, its gradient and the charge energy are the HIP kernels of this package (through
`khan_amd.autograd`).  In float32 the dense layers with CELU (all but the last of the reference's default network) run in
this package's matrix-core kernel (`ops.dense`: bias and activation in the product's epilogue, the activation's
derivative in the prologue of the data gradient), the first one right behind the featurizer; the last layer and every
float64 layer are plain matrix products: PyTorch's (rocBLAS).  Parameter
names are the reference's TensorFlow variable names, `<prefix>W_<type>_<in>x<out>_l<k>:0` and
`<prefix>b_...` (nn.py:41-60), so a checkpoint written by the reference's `save_numpy` loads unchanged;
whatever else such a file holds (optimizer slots, learning rate, moving averages) is ignored.
"""
import os

import numpy as np
import torch

TYPE_MAP = ("H", "C", "N", "O")
DEFAULT_LAYERS = (128, 128, 64, 1)                       # energy_server.py:121
DEEP_LAYERS = (256, 256, 256, 256, 256, 256, 256, 128, 64, 8, 1)   # energy_server.py:123
FEATURE_SIZE = 384


# ------------------------------------------------------------------ activation functions (activations.py:63-77)
def celu(a, alpha=0.1):
    # a for a >= 0, alpha (exp(a / alpha) - 1) below.  float32: PyTorch's celu, one elementwise kernel forward and
    # one backward.  float64: spelled out, because that kernel's backward rounds alpha to float (1e-8 off).
    if a.dtype == torch.float32:
        return torch.nn.functional.celu(a, alpha)
    return torch.where(a >= 0, a, alpha * torch.expm1(torch.clamp(a, max=0.0) / alpha))


def normal(a, mean=0.0, std=1.0):
    return torch.exp(-((a - mean) / std) ** 2 / 2.0)


def gaussian(a):
    return torch.exp(-a * a)


def softplus(a, shift=0.69314718056):
    return torch.nn.functional.softplus(a) - shift


ACTIVATIONS = {"celu": celu, "normal": normal, "gaussian": gaussian, "softplus": softplus}


def get_fn_by_name(name, *args):
    """activations.get_fn_by_name: the function with its leading extra arguments bound."""
    if name not in ACTIVATIONS:
        raise KeyError("unknown activation function %r (have %s)" % (name, sorted(ACTIVATIONS)))
    fn = ACTIVATIONS[name]
    return (lambda a: fn(a, *args)) if args else fn


def parameter_names(prefix, layer_sizes):
    """[(W name, b name, in, out)] per type and layer, in the reference's order (nn.py:38-60)."""
    out = {}
    for t in TYPE_MAP:
        rows = []
        for idx in range(1, len(layer_sizes)):
            x, y = layer_sizes[idx - 1], layer_sizes[idx]
            name = "_%s_%dx%d_l%d" % (t, x, y, idx)
            rows.append((prefix + "W" + name + ":0", prefix + "b" + name + ":0", x, y))
        out[t] = rows
    return out


class MoleculeNN:
    """Four atomic networks (H, C, N, O) mapping feature rows to one number per atom."""

    def __init__(self, layer_sizes=DEFAULT_LAYERS, activation_fn=celu, dtype=torch.float32, device="cpu",
                 prefix="near_", seed=None, first_layer_kernel=True):
        self.first_layer_kernel = bool(first_layer_kernel)
        self.whole_network_kernel = True    # the one-launch network where it applies (`one_launch`); False: layer by layer
        self.weights_need_grad = False      # set it to differentiate through the kernel layers' weights (training)
        layer_sizes = tuple(int(v) for v in layer_sizes)
        if layer_sizes[-1] != 1:
            raise ValueError("the last layer must have size 1")
        self.layer_sizes = (FEATURE_SIZE,) + layer_sizes
        self.activation_fn = activation_fn
        self.dtype, self.device, self.prefix = dtype, torch.device(device), prefix
        self.names = parameter_names(prefix, self.layer_sizes)
        gen = torch.Generator().manual_seed(0 if seed is None else int(seed))
        self.params = {}
        for t in TYPE_MAP:
            for wn, bn, x, y in self.names[t]:
                # random normal with standard deviation sqrt(2 / (in + out)), zero biases (nn.py:49-58)
                w = torch.randn((x, y), generator=gen, dtype=torch.float64) * (2.0 / (x + y)) ** 0.5
                self.params[wn] = w.to(dtype).to(self.device).requires_grad_(True)
                self.params[bn] = torch.zeros((y,), dtype=dtype, device=self.device).requires_grad_(True)

    def parameters(self):
        return [self.params[k] for k in self.params]

    def atom_type_outputs(self, type_idx, feats, layers_done=0):
        """[n_t, 384] feature rows of one type -> [n_t] network outputs (`layers_done`: `feats` are the activations of
        that many leading layers already)."""
        rows = self.names[TYPE_MAP[type_idx]]
        a = feats
        for k, (wn, bn, _, _) in enumerate(rows):
            if k < layers_done:
                continue
            a = torch.addmm(self.params[bn], a, self.params[wn])
            if k != len(rows) - 1:
                a = self.activation_fn(a)
        return a.reshape(-1)

    def layer_transposed(self, k):
        """The four weights of layer k transposed ([out, in], the summed index contiguous), as `ops.dense` takes them;
        kept until a weight is written again."""
        ws = [self.params[self.names[t][k][0]] for t in TYPE_MAP]
        key = tuple((w.data_ptr(), w._version) for w in ws)
        cache = self.__dict__.setdefault("_wt_cache", {})
        if k not in cache or cache[k][0] != key:
            cache[k] = (key, [w.detach().t().contiguous() for w in ws])
        return cache[k][1]

    def kernel_layers(self):
        """How many leading layers run in this package's matrix-core kernel (`ops.dense`): float32 on the GPU, CELU
        with its default alpha, input width a multiple of 32 and output width a multiple of 64 -- for the reference's
        default network 384-128-128-64-1 all but the last, which `atom_outputs` folds into the launch of the one
        before it (`ops.dense_head`)."""
        if not (self.first_layer_kernel and self.dtype == torch.float32 and self.device.type == "cuda"
                and self.activation_fn is celu):
            return 0
        n = 0
        for x, y in zip(self.layer_sizes[:-2], self.layer_sizes[1:-1]):      # the last layer has no activation
            if x % 32 or y % 64:
                break
            n += 1
        return n

    def one_launch(self):
        """True if the whole network runs in `ops.atomic_networks` (one launch for the three CELU layers and the output
        layer of the four types, and for the gradient back to the feature rows): the reference's default widths
        384-128-128-64-1 in float32 on the GPU with CELU, the weights taken as constants (inference)."""
        from . import ops
        return (self.whole_network_kernel and self.kernel_layers() == 3 and self.layer_sizes == ops.NETWORK_WIDTHS + (1,)
                and not self.weights_need_grad)

    def one_launch_operands(self):
        """-> (packed weights, biases, head_weights, head_biases) as `ops.atomic_networks` takes them; the weights are
        split into their half-precision parts once and kept until a weight is written again."""
        from . import ops
        rows = [[self.names[t][k] for t in TYPE_MAP] for k in range(4)]
        ws = [self.params[r[0]] for k in range(3) for r in rows[k]]
        key = tuple((w.data_ptr(), w._version) for w in ws)
        cache = self.__dict__.setdefault("_packed_cache", {})
        if cache.get("key") != key:
            weights_t = [self.layer_transposed(k) for k in range(3)]
            weights = [[self.params[r[0]].detach() for r in rows[k]] for k in range(3)]
            cache["key"], cache["packed"] = key, ops.pack_network_weights(weights_t, weights)
        biases = [[self.params[r[1]].detach() for r in rows[k]] for k in range(3)]
        return cache["packed"], biases, [self.params[r[0]].detach() for r in rows[3]], [self.params[r[1]].detach() for r in rows[3]]

    def atom_outputs(self, atom_type_features, gather_idxs):
        """Per-type flat feature buckets -> one number per atom in the batch's atom order (nn.py:176-177)."""
        # gather_idxs is a permutation: index_select's backward is a scatter-add, where indexing with [] sorts the
        # indices first (a merge sort of n atoms in every backward pass)
        return torch.index_select(torch.cat(self.type_outputs(atom_type_features)), 0, gather_idxs.long())

    def type_outputs(self, atom_type_features):
        """Per-type flat feature buckets -> the four per-type output vectors [acs[t]] (nn.py:165-175)."""
        nk = self.kernel_layers()
        if nk > 0:
            from . import autograd
            # inference: the weights are constants here (a custom autograd function cannot tell that only the
            # coordinates' gradient was asked for, and would form the weights' gradient, a second product, every time)
            par = (lambda k: self.params[k]) if self.weights_need_grad else (lambda k: self.params[k].detach())
            a = atom_type_features
            # the output layer rides in the last hidden layer's launch when that layer is a kernel layer of width 64
            fuse_head = nk == len(self.layer_sizes) - 2 and self.layer_sizes[-2] == 64
            for k in range(nk - 1 if fuse_head else nk):
                rows = [self.names[t][k] for t in TYPE_MAP]
                a = autograd.dense(a, [par(r[0]) for r in rows], [par(r[1]) for r in rows], alpha=0.1,
                                   weights_t=self.layer_transposed(k))
            if fuse_head:
                rows = [self.names[t][nk - 1] for t in TYPE_MAP]
                head = [self.names[t][nk] for t in TYPE_MAP]
                outs = autograd.dense_head(a, [par(r[0]) for r in rows], [par(r[1]) for r in rows],
                                           [par(r[0]) for r in head], [par(r[1]) for r in head], alpha=0.1,
                                           weights_t=self.layer_transposed(nk - 1))
            else:
                outs = [self.atom_type_outputs(t, a[t], layers_done=nk) for t in range(4)]
        else:
            outs = [self.atom_type_outputs(t, f.reshape(-1, FEATURE_SIZE)) for t, f in enumerate(atom_type_features)]
        return list(outs)


class AniModel:
    """Near-field network, optional charge network with the pairwise charge energy, and their checkpoint."""

    def __init__(self, layer_sizes=DEFAULT_LAYERS, activation_fn=celu, dtype=torch.float32, device="cuda:0",
                 fit_charges=False, seed=None, first_layer_kernel=True):
        self.dtype, self.device = dtype, torch.device(device)
        self.near = MoleculeNN(layer_sizes, activation_fn, dtype, device, "near_", seed, first_layer_kernel)
        self.charge = None
        if fit_charges:
            self.charge = MoleculeNN(layer_sizes, activation_fn, dtype, device, "charge_",
                                     None if seed is None else seed + 1, first_layer_kernel)

    # -------------------------------------------------------------------------------------- checkpoint
    def named_parameters(self):
        out = dict(self.near.params)
        if self.charge is not None:
            out.update(self.charge.params)
        return out

    def save_numpy(self, npz_file):
        """trainer_multi_tower.py:451-470: one array per variable, keyed by the variable's name."""
        if os.path.splitext(npz_file)[1] != ".npz":
            raise ValueError("the checkpoint file name must end in .npz")
        np.savez(npz_file, **{k: v.detach().cpu().numpy() for k, v in self.named_parameters().items()})

    def load_numpy(self, npz_file, strict=False):
        """trainer_multi_tower.py:472-499.  `strict` refuses a checkpoint of another precision; arrays the model
        has no parameter for are ignored; a parameter missing from the file is an error."""
        objs = np.load(npz_file, allow_pickle=False)
        mine = self.named_parameters()
        missing = [k for k in mine if k not in objs.files]
        if missing:
            raise KeyError("checkpoint %s lacks %d parameters, e.g. %s" % (npz_file, len(missing), missing[0]))
        np_dtype = np.float32 if self.dtype == torch.float32 else np.float64
        for k, p in mine.items():
            arr = objs[k]
            if arr.dtype != np_dtype and strict:
                raise TypeError("Cannot deserialize %s into %s. You may want to set strict=False."
                                % (arr.dtype, np.dtype(np_dtype)))
            if tuple(arr.shape) != tuple(p.shape):
                raise ValueError("%s has shape %s in the checkpoint, %s in the model" % (k, arr.shape, tuple(p.shape)))
            with torch.no_grad():
                p.copy_(torch.from_numpy(np.ascontiguousarray(arr.astype(np_dtype))).to(self.device))

    # --------------------------------------------------------------------------------------- inference
    def batch_energies(self, b, need_grad=False):
        """DeviceBatch -> per-molecule energies [n_mols] (and d energy / d xyz when need_grad)."""
        from . import autograd, ops
        xs, ys, zs = b.xs, b.ys, b.zs
        acs, order, classes = b.host_counts()
        if self.charge is None and self.near.one_launch():
            # featurize -> the four networks in one launch (values, and the gradient of their sum with respect to the
            # feature rows) -> sums by molecule; the coordinate gradient is featurize_grad of those rows' gradients
            feats = ops.featurize(xs, ys, zs, b.atom_types, b.mol_offsets, b.mol_atom_counts, b.scatter_idxs, acs,
                                  order=order, size_classes=classes)
            packed, biases, head_w, head_b = self.near.one_launch_operands()
            values, grads = ops.atomic_networks(feats, None, biases, head_w, head_b, want_grad=need_grad, packed=packed)
            energies = ops.mol_energy(values, b.atom_types, b.scatter_idxs, b.mol_offsets, b.mol_atom_counts)
            if not need_grad:
                return energies, None
            gx, gy, gz = ops.featurize_grad(xs, ys, zs, b.atom_types, b.mol_offsets, b.mol_atom_counts, b.scatter_idxs, acs,
                                            *[g.reshape(-1) for g in grads], order=order, size_classes=classes)
            return energies, torch.stack((gx, gy, gz), dim=1)
        if need_grad:
            xs, ys, zs = (t.detach().clone().requires_grad_(True) for t in (xs, ys, zs))
        feats = autograd.featurize(xs, ys, zs, b.atom_types, b.mol_offsets, b.mol_atom_counts, b.scatter_idxs, acs,
                                   order=order, size_classes=classes)
        # the networks' outputs summed by molecule straight from the four per-type vectors (nn.py:165-177 in one launch)
        energies = autograd.mol_energy(self.near.type_outputs(feats), b.atom_types, b.scatter_idxs, b.mol_offsets,
                                       b.mol_atom_counts)
        if self.charge is not None:
            qs = self.charge.atom_outputs(feats, b.gather_idxs)
            energies = energies + autograd.ani_charge(xs, ys, zs, qs.contiguous(), b.mol_offsets, b.mol_atom_counts)
        if not need_grad:
            return energies.detach(), None
        gx, gy, gz = torch.autograd.grad(energies, (xs, ys, zs), grad_outputs=torch.ones_like(energies))
        return energies.detach(), torch.stack((gx, gy, gz), dim=1)

    def _feeder(self, dataset, batch_size):
        from .batching import DeviceFeeder
        np_dtype = np.float32 if self.dtype == torch.float32 else np.float64
        return DeviceFeeder(dataset, batch_size, shuffle=False, dtype=np_dtype, device=self.device)

    def predict(self, dataset, batch_size=2048):
        """-> [y0, y1, ...] in the order of the dataset's molecules (trainer_multi_tower.py:655-678)."""
        ys = []
        for b in self._feeder(dataset, batch_size):
            b.wait()
            e, _ = self.batch_energies(b)
            ys.extend(e.cpu().tolist())
        return ys

    def coordinate_gradients(self, dataset, batch_size=1024):
        """Yields one [n_atoms, 3] array of d energy / d (x, y, z) per molecule (trainer_multi_tower.py:580-615)."""
        for b in self._feeder(dataset, batch_size):
            b.wait()
            _, g = self.batch_energies(b, need_grad=True)
            g = g.cpu().numpy()
            mos = b.mol_offsets.cpu().numpy()
            macs = b.mol_atom_counts.cpu().numpy()
            for off, cnt in zip(mos, macs):
                yield g[off:off + cnt]
