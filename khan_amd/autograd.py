"""Gradient wiring of the featurization ops for torch.autograd, the counterpart of the
`ops.RegisterGradient` blocks in khan/training/trainer_multi_tower.py:23-120:

    Featurize      d/d(xs,ys,zs) through `featurize_grad`; no gradient for the index inputs
                   (trainer_multi_tower.py:23-51)
    FeaturizeGrad  d/d(upstream gradients) through `featurize_grad_inverse`, so that a loss on forces
                   can be differentiated with respect to the network parameters; like the reference
                   it offers no second derivative with respect to the coordinates
                   (trainer_multi_tower.py:64-91)
    AniCharge      d/dqs through `ani_charge_grad` (trainer_multi_tower.py:88-120); here the
                coordinates get a gradient too (`ani_charge_grad_xyz`), which the reference
                leaves as None

Both call the HIP library through `khan_amd.ops`; there is no other implementation behind them.
"""
import torch

from . import ops


class _FeaturizeGrad(torch.autograd.Function):
    @staticmethod
    def forward(ctx, xs, ys, zs, as_, mos, macs, sis, acs_host, order, size_classes, grad_h, grad_c, grad_n, grad_o):
        ctx.save_for_backward(xs, ys, zs, as_, mos, macs, sis)
        ctx.acs_host, ctx.order, ctx.size_classes = acs_host, order, size_classes
        return ops.featurize_grad(xs, ys, zs, as_, mos, macs, sis, acs_host,
                                  grad_h.contiguous(), grad_c.contiguous(), grad_n.contiguous(), grad_o.contiguous(),
                                  order=order, size_classes=size_classes)

    @staticmethod
    def backward(ctx, dx, dy, dz):
        xs, ys, zs, as_, mos, macs, sis = ctx.saved_tensors
        zero = lambda: torch.zeros_like(xs)
        dx, dy, dz = (zero() if d is None else d.contiguous() for d in (dx, dy, dz))
        dh, dc, dn, do = ops.featurize_grad_inverse(xs, ys, zs, as_, mos, macs, sis, ctx.acs_host, dx, dy, dz,
                                                    order=ctx.order, size_classes=ctx.size_classes)
        return (None,) * 10 + (dh, dc, dn, do)


class _Featurize(torch.autograd.Function):
    @staticmethod
    def forward(ctx, xs, ys, zs, as_, mos, macs, sis, acs, order, size_classes):
        acs_host = [int(v) for v in (acs.detach().cpu().tolist() if isinstance(acs, torch.Tensor) else acs)]
        ctx.save_for_backward(xs, ys, zs, as_, mos, macs, sis)
        ctx.acs_host, ctx.order, ctx.size_classes = acs_host, order, size_classes
        return ops.featurize(xs.detach(), ys.detach(), zs.detach(), as_, mos, macs, sis, acs_host,
                             order=order, size_classes=size_classes)

    @staticmethod
    def backward(ctx, grad_h, grad_c, grad_n, grad_o):
        xs, ys, zs, as_, mos, macs, sis = ctx.saved_tensors
        grads = []
        for g, c in zip((grad_h, grad_c, grad_n, grad_o), ctx.acs_host):
            if g is None:
                g = torch.zeros(c * ops.FEATURE_SIZE, dtype=xs.dtype, device=xs.device)
            grads.append(g)
        gx, gy, gz = _FeaturizeGrad.apply(xs.detach(), ys.detach(), zs.detach(), as_, mos, macs, sis,
                                          ctx.acs_host, ctx.order, ctx.size_classes, *grads)
        return gx, gy, gz, None, None, None, None, None, None, None


class _AniCharge(torch.autograd.Function):
    @staticmethod
    def forward(ctx, xs, ys, zs, qs, mos, macs):
        ctx.save_for_backward(xs, ys, zs, qs, mos, macs)
        return ops.ani_charge(xs.detach(), ys.detach(), zs.detach(), qs.detach(), mos, macs)

    @staticmethod
    def backward(ctx, grads):
        xs, ys, zs, qs, mos, macs = ctx.saved_tensors
        need_xyz = any(ctx.needs_input_grad[:3])
        args = (xs.detach(), ys.detach(), zs.detach(), qs.detach(), mos, macs, grads.contiguous())
        if need_xyz:
            qg, gx, gy, gz = ops.ani_charge_grad_xyz(*args)
            return gx, gy, gz, qg, None, None
        return None, None, None, ops.ani_charge_grad(*args), None, None



def _library_layer_backward(ctx, xs, ws, bs, gouts, celu_act, alpha, head=None):
    """The gradients of one dense layer of the four atomic networks (with `head`: followed by the output layer) formed
    from library operations under autograd, so that they carry a graph of their own: what `_Dense.backward` and
    `_DenseHead.backward` return when they are differentiated again.  -> the gradients in the order of the layer's
    tensor inputs (inputs, weights, biases[, output weights, output biases]), None where none was asked for."""
    groups = 5 if head is not None else 3
    res = [[None] * 4 for _ in range(groups)]
    with torch.enable_grad():
        for t in range(4):
            if gouts[t] is None:
                continue
            k = ws[t].shape[0]
            x = xs[t].reshape(-1, k)
            a = torch.addmm(bs[t], x, ws[t])
            if celu_act:
                a = torch.nn.functional.celu(a, alpha)
            operands = [xs[t], ws[t], bs[t]]
            if head is not None:
                a = (a @ head[0][t].reshape(-1, 1)).reshape(-1) + head[1][t].reshape(-1)
                operands += [head[0][t], head[1][t]]
            asked = [j for j in range(groups) if ctx.needs_input_grad[3 + 4 * j + t] and operands[j].requires_grad]
            if not asked or not a.requires_grad:
                continue
            gs = torch.autograd.grad(a, [operands[j] for j in asked], gouts[t].reshape(a.shape), create_graph=True,
                                     allow_unused=True)
            for j, g in zip(asked, gs):
                res[j][t] = g
    return tuple(g for group in res for g in group)


class _Dense(torch.autograd.Function):
    """act(in_t . W_t + b_t) for the four atom types through `ops.dense` (float32; CELU or no activation), forward on
    the matrix-core kernel and the data gradient too: d/d in = (g .* act'(out)) . W^T, with the activation's derivative
    taken from the saved outputs inside the kernel (CELU: 1 for out >= 0, out / alpha + 1 = exp(z / alpha) below)."""

    @staticmethod
    def forward(ctx, activation, alpha, weights_t, *tensors):
        xs, ws, bs = tensors[0:4], tensors[4:8], tensors[8:12]
        k = ws[0].shape[0]
        if weights_t is None:
            weights_t = [w.detach().t().contiguous() for w in ws]
        outs = ops.dense([x.detach().reshape(-1, k) for x in xs], weights_t, [b.detach() for b in bs], activation, alpha)
        ctx.save_for_backward(*xs, *ws, *outs, *bs)
        ctx.activation, ctx.alpha = activation, alpha
        return outs

    @staticmethod
    def backward(ctx, *gouts):
        saved = ctx.saved_tensors
        xs, ws, outs = saved[0:4], saved[4:8], saved[8:12]
        k, n_out = ws[0].shape
        celu_act = ctx.activation == ops.ACT_CELU
        if torch.is_grad_enabled():
            # A graph of this gradient was asked for (create_graph: a loss on forces differentiated with respect to
            # the weights).  The kernels record nothing, so the layer is formed again from library operations, which
            # do, and differentiated by them.
            return (None, None, None) + _library_layer_backward(ctx, xs, ws, saved[12:16], gouts, celu_act, ctx.alpha)
        gs = [torch.zeros_like(outs[t]) if gouts[t] is None else gouts[t].contiguous() for t in range(4)]
        gx = (None,) * 4
        if any(ctx.needs_input_grad[3:7]):
            # one launch for the four types: in = g, the derivative from the saved activations, W as it is
            gx = ops.dense(gs, [w.detach() for w in ws], None, ops.ACT_NONE, ctx.alpha, deriv_of=outs if celu_act else None)
            gx = tuple(g.reshape(xs[t].shape) if ctx.needs_input_grad[3 + t] else None for t, g in enumerate(gx))
        gw, gb = [None] * 4, [None] * 4
        if any(ctx.needs_input_grad[7:15]):
            for t in range(4):
                g = gs[t]
                if celu_act:     # CELU is ELU with input scale 1 / alpha, differentiated from its result
                    g = torch.ops.aten.elu_backward(g, ctx.alpha, 1.0, 1.0 / ctx.alpha, True, outs[t])
                if ctx.needs_input_grad[7 + t]:
                    gw[t] = xs[t].reshape(-1, k).t() @ g
                if ctx.needs_input_grad[11 + t]:
                    gb[t] = g.sum(dim=0)
        return (None, None, None) + tuple(gx) + tuple(gw) + tuple(gb)


def dense(inputs, weights, biases, activation=ops.ACT_CELU, alpha=0.1, weights_t=None):
    """Differentiable dense layer of the four atomic networks: four inputs ([n_t, k], or flat buckets of n_t * k), four
    [k, n_out] weights, four [n_out] biases -> four [n_t, n_out] activations (float32; k a multiple of 32, n_out of 64).
    `weights_t`: the four weights transposed ([n_out, k], contiguous), if the caller keeps them; otherwise they are
    transposed here on every call."""
    return _Dense.apply(int(activation), float(alpha), weights_t, *inputs, *weights, *biases)


class _DenseHead(torch.autograd.Function):
    """The last hidden layer (width 64) and the output layer (64 -> 1, no activation) of the four atomic networks in
    one launch each way (`ops.dense_head`, `ops.dense_head_grad`): -> four [n_t] vectors of atomic values.  On the way
    back the gradient with respect to the hidden activations, g_t[r] * w_out_t[c], is never materialised for the data
    gradient; the weight gradients (when asked for) are library products."""

    @staticmethod
    def forward(ctx, activation, alpha, weights_t, *tensors):
        xs, ws, bs, hws, hbs = tensors[0:4], tensors[4:8], tensors[8:12], tensors[12:16], tensors[16:20]
        k = ws[0].shape[0]
        if weights_t is None:
            weights_t = [w.detach().t().contiguous() for w in ws]
        outs, heads = ops.dense_head([x.detach().reshape(-1, k) for x in xs], weights_t, [b.detach() for b in bs],
                                     [w.detach() for w in hws], [b.detach() for b in hbs], activation, alpha)
        ctx.save_for_backward(*xs, *ws, *hws, *outs, *bs, *hbs)
        ctx.activation, ctx.alpha = activation, alpha
        return heads

    @staticmethod
    def backward(ctx, *gheads):
        saved = ctx.saved_tensors
        xs, ws, hws, outs = saved[0:4], saved[4:8], saved[8:12], saved[12:16]
        k, n_out = ws[0].shape
        celu_act = ctx.activation == ops.ACT_CELU
        if torch.is_grad_enabled():      # create_graph: see _Dense.backward
            return (None, None, None) + _library_layer_backward(ctx, xs, ws, saved[16:20], gheads, celu_act, ctx.alpha,
                                                                head=(hws, saved[20:24]))
        gs = [torch.zeros(outs[t].shape[0], dtype=outs[t].dtype, device=outs[t].device) if gheads[t] is None
              else gheads[t].contiguous() for t in range(4)]
        gx = (None,) * 4
        if any(ctx.needs_input_grad[3:7]):
            if celu_act:
                gx = ops.dense_head_grad(gs, [w.detach() for w in hws], [w.detach() for w in ws], outs, ctx.alpha)
            else:
                gx = ops.dense([gs[t][:, None] * hws[t].detach().reshape(1, -1) for t in range(4)], [w.detach() for w in ws])
            gx = tuple(g.reshape(xs[t].shape) if ctx.needs_input_grad[3 + t] else None for t, g in enumerate(gx))
        gw, gb, ghw, ghb = [None] * 4, [None] * 4, [None] * 4, [None] * 4
        if any(ctx.needs_input_grad[7:23]):
            for t in range(4):
                if ctx.needs_input_grad[15 + t]:
                    ghw[t] = (outs[t].t() @ gs[t]).reshape(hws[t].shape)
                if ctx.needs_input_grad[19 + t]:
                    ghb[t] = gs[t].sum().reshape(1)
                if ctx.needs_input_grad[7 + t] or ctx.needs_input_grad[11 + t]:
                    g = gs[t][:, None] * hws[t].detach().reshape(1, -1)
                    if celu_act:
                        g = torch.ops.aten.elu_backward(g, ctx.alpha, 1.0, 1.0 / ctx.alpha, True, outs[t])
                    if ctx.needs_input_grad[7 + t]:
                        gw[t] = xs[t].reshape(-1, k).t() @ g
                    if ctx.needs_input_grad[11 + t]:
                        gb[t] = g.sum(dim=0)
        return (None, None, None) + tuple(gx) + tuple(gw) + tuple(gb) + tuple(ghw) + tuple(ghb)


def dense_head(inputs, weights, biases, head_weights, head_biases, activation=ops.ACT_CELU, alpha=0.1, weights_t=None):
    """Differentiable last hidden layer + output layer of the four atomic networks: four inputs [n_t, k], four
    [k, 64] weights, four [64] biases, four [64, 1] output-layer weights, four [1] output-layer biases -> four [n_t]
    vectors (float32; k a multiple of 32)."""
    return _DenseHead.apply(int(activation), float(alpha), weights_t, *inputs, *weights, *biases, *head_weights, *head_biases)


class _MolEnergy(torch.autograd.Function):
    """Per-molecule sums of the four per-type output vectors (`ops.mol_energy`); the way back hands every atom's
    entry its molecule's gradient (`ops.mol_energy_grad`)."""

    @staticmethod
    def forward(ctx, atom_types, sis, mos, macs, *outs):
        ctx.save_for_backward(atom_types, sis, mos, macs)
        ctx.counts = [int(o.numel()) for o in outs]
        ctx.shapes = [o.shape for o in outs]
        return ops.mol_energy([o.detach() for o in outs], atom_types, sis, mos, macs)

    @staticmethod
    def backward(ctx, ge):
        atom_types, sis, mos, macs = ctx.saved_tensors
        gs = _MolEnergyGrad.apply(atom_types, sis, mos, macs, tuple(ctx.counts), ge)
        return (None, None, None, None) + tuple(g.reshape(sh) for g, sh in zip(gs, ctx.shapes))


class _MolEnergyGrad(torch.autograd.Function):
    """Every atom's entry of the four per-type vectors takes its molecule's value (`ops.mol_energy_grad`), the
    transpose of the sums by molecule -- whose own way back is therefore those sums again (`ops.mol_energy`).  Both
    maps are linear, so the pair is differentiable to any order."""

    @staticmethod
    def forward(ctx, atom_types, sis, mos, macs, counts, ge):
        ctx.save_for_backward(atom_types, sis, mos, macs)
        ctx.counts, ctx.dt, ctx.dev = counts, ge.dtype, ge.device
        return tuple(ops.mol_energy_grad(ge.detach().contiguous(), atom_types, sis, mos, macs, list(counts)))

    @staticmethod
    def backward(ctx, *dgs):
        atom_types, sis, mos, macs = ctx.saved_tensors
        dgs = [torch.zeros(c, dtype=ctx.dt, device=ctx.dev) if d is None else d.contiguous()
               for d, c in zip(dgs, ctx.counts)]
        return (None,) * 5 + (_MolEnergy.apply(atom_types, sis, mos, macs, *dgs),)


def mol_energy(type_outputs, atom_types, sis, mos, macs):
    """Differentiable per-molecule sums of the four per-type network outputs: -> [n_mols]."""
    return _MolEnergy.apply(atom_types, sis, mos, macs, *type_outputs)


def dense_first(atom_type_features, acs_host, weights, biases, activation=ops.ACT_CELU, alpha=0.1, weights_t=None):
    """The first dense layer on the featurizer's four flat buckets: `dense` with k = 384."""
    for f, c in zip(atom_type_features, acs_host):
        if f.numel() != int(c) * ops.FEATURE_SIZE:
            raise ValueError("a bucket of %d elements for %d atoms" % (f.numel(), int(c)))
    return dense(atom_type_features, weights, biases, activation, alpha, weights_t)


def featurize(xs, ys, zs, as_, mos, macs, sis, acs, order=None, size_classes=None):
    """Differentiable `featurize`: -> (h_feat, c_feat, n_feat, o_feat); gradients flow to xs, ys, zs.
    `order`, `size_classes`: the batch's size order (`ops.size_order`) and its four class totals on the host, shared
    by the forward pass and every derivative of it."""
    return _Featurize.apply(xs, ys, zs, as_, mos, macs, sis, acs, order, size_classes)


def ani_charge(xs, ys, zs, qs, mos, macs):
    """Differentiable `ani_charge`: -> charge_energies[n_mols]; gradients flow to qs and to xs, ys, zs."""
    return _AniCharge.apply(xs, ys, zs, qs, mos, macs)
