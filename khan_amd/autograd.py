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


class _DenseFirst(torch.autograd.Function):
    """act(rows_t . W_t + b_t) for the four atom types through `ops.dense_first` (float32, width 128, CELU or no
    activation).  Backward: plain matrix products; the activation's derivative comes from the saved outputs
    (CELU: 1 for out >= 0, out / alpha + 1 = exp(z / alpha) below)."""

    @staticmethod
    def forward(ctx, acs_host, activation, alpha, weights_t, *tensors):
        feats, ws, bs = tensors[0:4], tensors[4:8], tensors[8:12]
        if weights_t is None:
            weights_t = [w.detach().t().contiguous() for w in ws]
        outs = ops.dense_first([f.detach() for f in feats], acs_host, weights_t, [b.detach() for b in bs], activation, alpha)
        ctx.save_for_backward(*feats, *ws, *outs)
        ctx.activation, ctx.alpha = activation, alpha
        return outs

    @staticmethod
    def backward(ctx, *gouts):
        saved = ctx.saved_tensors
        feats, ws, outs = saved[0:4], saved[4:8], saved[8:12]
        gf, gw, gb = [], [], []
        for t in range(4):
            g = gouts[t]
            if g is None or outs[t].numel() == 0:
                gf.append(torch.zeros_like(feats[t]) if ctx.needs_input_grad[4 + t] else None)
                gw.append(torch.zeros_like(ws[t]) if ctx.needs_input_grad[8 + t] else None)
                gb.append(torch.zeros(ws[t].shape[1], dtype=ws[t].dtype, device=ws[t].device) if ctx.needs_input_grad[12 + t] else None)
                continue
            if ctx.activation == ops.ACT_CELU:
                # one elementwise kernel: CELU is ELU with input scale 1 / alpha, differentiated from its result
                g = torch.ops.aten.elu_backward(g.contiguous(), ctx.alpha, 1.0, 1.0 / ctx.alpha, True, outs[t])
            rows = feats[t].reshape(-1, ops.FEATURE_SIZE)
            gf.append((g @ ws[t].t()).reshape(feats[t].shape) if ctx.needs_input_grad[4 + t] else None)
            gw.append(rows.t() @ g if ctx.needs_input_grad[8 + t] else None)
            gb.append(g.sum(dim=0) if ctx.needs_input_grad[12 + t] else None)
        return (None, None, None, None) + tuple(gf) + tuple(gw) + tuple(gb)


def dense_first(atom_type_features, acs_host, weights, biases, activation=ops.ACT_CELU, alpha=0.1, weights_t=None):
    """Differentiable first dense layer of the four atomic networks: four flat feature buckets, four [384, 128]
    weights, four [128] biases -> four [n_t, 128] activations (float32).  `weights_t`: the four weights transposed
    ([128, 384], contiguous), if the caller keeps them; otherwise they are transposed here on every call."""
    return _DenseFirst.apply([int(v) for v in acs_host], int(activation), float(alpha), weights_t,
                             *atom_type_features, *weights, *biases)


def featurize(xs, ys, zs, as_, mos, macs, sis, acs, order=None, size_classes=None):
    """Differentiable `featurize`: -> (h_feat, c_feat, n_feat, o_feat); gradients flow to xs, ys, zs.
    `order`, `size_classes`: the batch's size order (`ops.size_order`) and its four class totals on the host, shared
    by the forward pass and every derivative of it."""
    return _Featurize.apply(xs, ys, zs, as_, mos, macs, sis, acs, order, size_classes)


def ani_charge(xs, ys, zs, qs, mos, macs):
    """Differentiable `ani_charge`: -> charge_energies[n_mols]; gradients flow to qs and to xs, ys, zs."""
    return _AniCharge.apply(xs, ys, zs, qs, mos, macs)
