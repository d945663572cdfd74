"""The atomic networks, their npz checkpoint and the energy server's wire format (khan/model/nn.py,
khan/model/activations.py, trainer_multi_tower.py:451-499 and 580-678, energy_server.py:141-187)."""
import json
import threading

import numpy as np
import pytest
import torch

from khan_amd import autograd, datagen, model, server
from khan_amd.batching import RawDataset
from oracle import nn_ref


def _molecules(n_mols=9, first=3):
    b = datagen.make_batch("organic", n_mols, first_mol=first)
    mols = []
    for m in range(n_mols):
        s = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
        mols.append(np.stack([b.A[s].astype(np.float64), b.X[s], b.Y[s], b.Z[s]], axis=1))
    return b, mols


def _np_params(m):
    return {k: v.detach().cpu().numpy() for k, v in m.named_parameters().items()}


# ------------------------------------------------------------------------------------- oracle pins
@pytest.mark.parametrize("name", sorted(nn_ref.ACTIVATIONS))
def test_oracle_activation_derivatives_by_finite_differences(name):
    f, df = nn_ref.ACTIVATIONS[name]
    a = np.linspace(-3.0, 3.0, 241) + 1e-3          # keeps clear of celu's kink at 0
    h = 1e-6
    fd = (f(a + h) - f(a - h)) / (2 * h)
    assert np.allclose(df(a), fd, rtol=1e-7, atol=1e-8)


def test_oracle_activation_known_values():
    celu = nn_ref.ACTIVATIONS["celu"][0]
    assert celu(np.array([0.0, 2.5]))[1] == 2.5 and celu(np.array([0.0]))[0] == 0.0
    assert abs(celu(np.array([-50.0]))[0] + 0.1) < 1e-15             # tends to -alpha
    assert abs(celu(np.array([-0.1]))[0] - 0.1 * (np.exp(-1.0) - 1.0)) < 1e-16
    assert abs(nn_ref.ACTIVATIONS["softplus"][0](np.array([0.0]))[0]) < 1e-11        # shifted by ln 2
    assert nn_ref.ACTIVATIONS["gaussian"][0](np.array([1.0]))[0] == pytest.approx(np.exp(-1.0))
    assert nn_ref.ACTIVATIONS["normal"][0](np.array([2.0]))[0] == pytest.approx(np.exp(-2.0))


def test_oracle_network_closed_forms_and_gradient():
    rng = np.random.default_rng(0)
    feats = rng.normal(size=(7, 12))
    # one layer: the network is linear
    W, b = rng.normal(size=(12, 1)), rng.normal(size=(1,))
    out, pre = nn_ref.atom_nn_forward(feats, [W], [b])
    assert np.allclose(out, feats @ W[:, 0] + b[0], rtol=0, atol=1e-14)
    assert np.allclose(nn_ref.atom_nn_backward(pre, [W], np.ones(7)), np.tile(W[:, 0], (7, 1)))
    # zero weights: the output is what the biases alone give
    Ws = [np.zeros((12, 5)), np.zeros((5, 1))]
    bs = [np.full(5, -0.05), np.array([0.25])]
    out, _ = nn_ref.atom_nn_forward(feats, Ws, bs)
    assert np.allclose(out, 0.25)
    # three layers: the backward pass against central differences of the forward pass
    Ws = [rng.normal(size=(12, 6)) * 0.5, rng.normal(size=(6, 4)) * 0.5, rng.normal(size=(4, 1))]
    bs = [rng.normal(size=6) * 0.1, rng.normal(size=4) * 0.1, rng.normal(size=1)]
    up = rng.normal(size=7)
    for act in sorted(nn_ref.ACTIVATIONS):
        _, pre = nn_ref.atom_nn_forward(feats, Ws, bs, act)
        g = nn_ref.atom_nn_backward(pre, Ws, up, act)
        h = 1e-6
        for (r, c) in [(0, 0), (3, 5), (6, 11)]:
            fp, fm = feats.copy(), feats.copy()
            fp[r, c] += h
            fm[r, c] -= h
            fd = (np.dot(up, nn_ref.atom_nn_forward(fp, Ws, bs, act)[0]) - np.dot(up, nn_ref.atom_nn_forward(fm, Ws, bs, act)[0])) / (2 * h)
            assert abs(g[r, c] - fd) < 1e-7 * max(1.0, abs(fd)), (act, r, c)


# ------------------------------------------------------------------------------------- host logic
@pytest.mark.parametrize("name", sorted(model.ACTIVATIONS))
def test_activations_match_the_oracle(name):
    a = np.linspace(-4.0, 4.0, 161)
    got = model.ACTIVATIONS[name](torch.from_numpy(a)).numpy()
    assert np.allclose(got, nn_ref.ACTIVATIONS[name][0](a), rtol=1e-13, atol=1e-15)


def test_get_fn_by_name_binds_arguments():
    a = torch.tensor([-1.0, 2.0], dtype=torch.float64)
    assert torch.equal(model.get_fn_by_name("celu")(a), model.celu(a))
    assert torch.allclose(model.get_fn_by_name("celu", 0.2)(a), model.celu(a, 0.2))
    with pytest.raises(KeyError):
        model.get_fn_by_name("relu6")


def test_network_matches_the_oracle_on_cpu():
    m = model.MoleculeNN(model.DEFAULT_LAYERS, model.celu, torch.float64, "cpu", "near_", seed=4)
    with torch.no_grad():
        for k, p in m.params.items():           # biases start at zero: give them values
            if "b_" in k:
                p.copy_(torch.linspace(-0.2, 0.3, p.numel(), dtype=torch.float64))
    nets = nn_ref.split_params({k: v.detach().numpy() for k, v in m.params.items()}, "near_", model.DEFAULT_LAYERS)
    rng = np.random.default_rng(2)
    for t in range(4):
        feats = rng.normal(size=(5 + t, 384)) * 0.3
        want, _ = nn_ref.atom_nn_forward(feats, nets[t][0], nets[t][1], "celu")
        got = m.atom_type_outputs(t, torch.from_numpy(feats)).detach().numpy()
        assert np.allclose(got, want, rtol=1e-12, atol=1e-13)
    # names and shapes are the reference's (nn.py:41): near_W_H_384x128_l1:0 ...
    assert "near_W_H_384x128_l1:0" in m.params and m.params["near_W_O_64x1_l4:0"].shape == (64, 1)
    assert m.params["near_b_C_128x128_l2:0"].shape == (128,)
    assert len(m.parameters()) == 4 * 4 * 2


def test_checkpoint_round_trip_names_extras_and_precision(tmp_path):
    a = model.AniModel(model.DEFAULT_LAYERS, model.celu, torch.float64, "cpu", fit_charges=True, seed=1)
    f = str(tmp_path / "save_file.npz")
    a.save_numpy(f)
    with pytest.raises(ValueError):
        a.save_numpy(str(tmp_path / "save_file.bin"))
    # what a TensorFlow checkpoint also holds (optimizer slots, step counters) is ignored
    objs = dict(np.load(f))
    objs["beta1_power:0"] = np.float32(0.9)
    objs["near_W_H_384x128_l1/Adam:0"] = np.zeros((384, 128), dtype=np.float64)
    np.savez(f, **objs)
    b = model.AniModel(model.DEFAULT_LAYERS, model.celu, torch.float64, "cpu", fit_charges=True, seed=9)
    b.load_numpy(f, strict=True)
    for k, v in a.named_parameters().items():
        assert torch.equal(v, b.named_parameters()[k]), k
    # another precision: refused when strict, converted otherwise
    c = model.AniModel(model.DEFAULT_LAYERS, model.celu, torch.float32, "cpu", fit_charges=False, seed=9)
    with pytest.raises(TypeError):
        c.load_numpy(f, strict=True)
    c.load_numpy(f, strict=False)
    k = "near_W_N_128x64_l3:0"
    assert c.named_parameters()[k].dtype == torch.float32
    assert torch.equal(c.named_parameters()[k], a.named_parameters()[k].float())
    # a file that lacks a parameter, or holds it with another shape
    del objs["near_b_O_64x1_l4:0"]
    np.savez(f, **objs)
    with pytest.raises(KeyError):
        b.load_numpy(f)
    d = model.AniModel((64, 1), model.celu, torch.float64, "cpu")
    with pytest.raises(KeyError):
        d.load_numpy(f)


def test_wire_format():
    X = [[0, 0.0, 0.0, 0.0], [3, 0.96, 0.0, 0.0], [0, -0.24, 0.93, 0.0]]
    arr = server.parse_request(json.dumps({"X": X}))
    assert arr.dtype == np.float64 and arr.shape == (3, 4)
    # two hydrogens and an oxygen (data_utils.py:28-33)
    assert server.self_interaction(arr) == pytest.approx(2 * -0.49932123901 + -75.04147134502, rel=1e-7)
    g = np.arange(9, dtype=np.float64).reshape(3, 3)
    doc = json.loads(server.format_response(-1.5, g))
    assert doc["energy"] == -1.5
    assert doc["gradient"] == [float(v) * 0.52917721092 for v in range(9)]      # atom-major, Hartree/Bohr
    for bad in ('{"Y": 1}', '{"X": []}', '{"X": [[0, 1, 2]]}', '{"X": [[4, 0, 0, 0]]}', '{"X": [[0.5, 0, 0, 0]]}', "[1]"):
        with pytest.raises(ValueError):
            server.parse_request(bad)


def test_serve_loop_survives_split_requests_and_bytes_that_are_not_text(monkeypatch):
    """The socket protocol has no framing: a request may arrive in several segments, and a peer may send bytes
    that are not UTF-8.  The loop reassembles the first and answers the second with an error; it never dies."""
    import socket
    import time
    seen = []

    def fake_handle(model_, text):
        seen.append(text)
        return json.dumps({"n": len(json.loads(text)["X"])})

    monkeypatch.setattr(server, "handle_request", fake_handle)
    listening = server.connect_socket("127.0.0.1", 0, server=True)
    port = listening.getsockname()[1]
    th = threading.Thread(target=server.serve_on, args=(listening, None, 2), daemon=True)
    th.start()
    big = json.dumps({"X": [[0, 0.1 * k, 0.0, 0.0] for k in range(3000)]})
    c = server.connect_socket("127.0.0.1", port, server=False)
    c.setsockopt(socket.IPPROTO_TCP, socket.TCP_NODELAY, 1)
    try:
        c.sendall(big[:1000].encode())                 # a request in three segments
        time.sleep(0.05)
        c.sendall(big[1000:50000].encode())
        time.sleep(0.05)
        c.sendall(big[50000:].encode())
        assert json.loads(server.receive(c)) == {"n": 3000}
        c.sendall(b"\xff\xfe{not text")                # not UTF-8, not JSON
        assert "error" in json.loads(server.receive(c))
    finally:
        server.close_connection(c)
    c2 = server.connect_socket("127.0.0.1", port, server=False)     # the loop is still serving
    try:
        server.send(c2, json.dumps({"X": [[0, 0, 0, 0]]}))
        assert json.loads(server.receive(c2)) == {"n": 1}
    finally:
        server.close_connection(c2)
    th.join(30)
    assert not th.is_alive()
    assert seen[0] == big


# ------------------------------------------------------------------------------------------- GPU
def _gpu_model(dtype, seed=7, layers=model.DEFAULT_LAYERS):
    m = model.AniModel(layers, model.celu, dtype, "cuda:0", seed=seed)
    with torch.no_grad():
        for k, p in m.named_parameters().items():
            if "b_" in k:
                p.copy_(torch.linspace(-0.1, 0.2, p.numel(), dtype=dtype, device=p.device))
    return m


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float64, 1e-10), (torch.float32, 2e-4)])
def test_predict_and_coordinate_gradients_match_the_oracle(dtype, tol):
    b, mols = _molecules(n_mols=21)
    m = _gpu_model(dtype)
    ds = RawDataset(mols, [0.0] * len(mols))
    np_dtype = np.float64 if dtype == torch.float64 else np.float32
    want_e, want_g = nn_ref.energies_and_gradients(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, _np_params(m), model.DEFAULT_LAYERS,
                                                   dtype=np.float64)
    got_e = np.array(m.predict(ds, batch_size=8))                # three batches, the last one short
    scale = np.max(np.abs(want_e))
    assert got_e.shape == want_e.shape
    assert np.max(np.abs(got_e - want_e)) <= tol * scale
    grads = list(m.coordinate_gradients(ds, batch_size=8))
    assert len(grads) == len(mols)
    for k, g in enumerate(grads):
        ref = want_g[b.MOs[k]:b.MOs[k] + b.MACs[k]]
        assert g.shape == ref.shape and g.dtype == np_dtype
        assert np.max(np.abs(g - ref)) <= tol * max(1.0, np.max(np.abs(ref))), k


@pytest.mark.gpu
def test_charge_model_energy_and_gradient_match_the_oracle():
    b, mols = _molecules(n_mols=6, first=60)
    m = model.AniModel((32, 1), model.celu, torch.float64, "cuda:0", fit_charges=True, seed=2)
    with torch.no_grad():                       # small charges keep the pairwise energy comparable to the near-field one
        for k, p in m.named_parameters().items():
            if k.startswith("charge_W") and k.endswith("l2:0"):
                p.mul_(0.05)
    ds = RawDataset(mols, [0.0] * len(mols))
    want_e, want_g = nn_ref.energies_and_gradients(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, _np_params(m), (32, 1),
                                                   fit_charges=True)
    near_only, _ = nn_ref.energies_and_gradients(b.X, b.Y, b.Z, b.A, b.MOs, b.MACs, _np_params(m), (32, 1), need_grad=False)
    assert np.max(np.abs(want_e - near_only)) > 1e-6         # the charge term is really there
    got_e = np.array(m.predict(ds))
    assert np.max(np.abs(got_e - want_e)) <= 1e-10 * np.max(np.abs(want_e))
    got_g = np.concatenate(list(m.coordinate_gradients(ds)), axis=0)
    assert np.max(np.abs(got_g - want_g)) <= 1e-10 * max(1.0, np.max(np.abs(want_g)))
    # and the oracle's gradient is the derivative of the oracle's energy
    h = 1e-5
    for (atom, axis) in [(0, 1), (b.n_atoms - 1, 0)]:
        P = [b.X.astype(np.float64).copy(), b.Y.astype(np.float64).copy(), b.Z.astype(np.float64).copy()]
        M = [v.copy() for v in P]
        P[axis][atom] += h
        M[axis][atom] -= h
        ep, _ = nn_ref.energies_and_gradients(*P, b.A, b.MOs, b.MACs, _np_params(m), (32, 1), need_grad=False, fit_charges=True)
        em, _ = nn_ref.energies_and_gradients(*M, b.A, b.MOs, b.MACs, _np_params(m), (32, 1), need_grad=False, fit_charges=True)
        fd = (ep.sum() - em.sum()) / (2 * h)
        assert abs(want_g[atom, axis] - fd) <= 1e-6 * max(1.0, abs(fd)), (atom, axis)


@pytest.mark.gpu
def test_gradient_is_the_derivative_of_the_energy():
    _, mols = _molecules(n_mols=1, first=40)
    m = _gpu_model(torch.float64, seed=3)
    X0 = mols[0]
    g = list(m.coordinate_gradients(RawDataset([X0], [0.0])))[0]
    h = 1e-5
    for (atom, axis) in [(0, 0), (1, 2), (X0.shape[0] - 1, 1)]:
        Xp, Xm = X0.copy(), X0.copy()
        Xp[atom, 1 + axis] += h
        Xm[atom, 1 + axis] -= h
        fd = (m.predict(RawDataset([Xp], [0.0]))[0] - m.predict(RawDataset([Xm], [0.0]))[0]) / (2 * h)
        assert abs(g[atom, axis] - fd) <= 1e-7 * max(1.0, abs(fd)), (atom, axis)


@pytest.mark.gpu
@pytest.mark.parametrize("activation", ["celu", "none"])
def test_first_dense_layer_kernel_matches_the_oracle(activation):
    """khan_dense_first_f32 (the first layer of the four atomic networks on the featurizer's buckets, matrix cores,
    one launch) against oracle/nn_ref.py's layer 1 in float64 (khan/model/nn.py:38-68), on real feature rows:
    row counts on and off the 128-row tile size, an empty type, and the float32 library product beside it."""
    from khan_amd import ops
    b, _ = _molecules(n_mols=300, first=3)
    dev = "cuda:0"
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    A = b.A.copy()
    A[A == 2] = 1                                   # no nitrogen: an empty bucket
    macs, mos = ops.mol_offsets(d(b.mol_idxs), b.n_mols)
    sc, ga, ac = ops.ani_sort(d(A))
    acs = ac.cpu()
    feats = ops.featurize(d(b.X), d(b.Y), d(b.Z), d(A), mos, macs, sc, acs)
    assert acs.tolist()[2] == 0 and min(acs.tolist()[:2]) > 128
    rng = np.random.default_rng(4)
    Ws = [rng.standard_normal((384, 128)) * (2.0 / 512) ** 0.5 for _ in range(4)]
    bs = [rng.standard_normal(128) * 0.1 for _ in range(4)]
    wt = [d(W.T.astype(np.float32)) for W in Ws]
    bt = [d(v.astype(np.float32)) for v in bs]
    act = ops.ACT_CELU if activation == "celu" else ops.ACT_NONE
    outs = ops.dense_first(feats, acs, wt, bt, activation=act, alpha=0.1)
    for t in range(4):
        rows = feats[t].reshape(-1, 384).cpu().numpy().astype(np.float64)
        z = rows @ Ws[t].astype(np.float32).astype(np.float64) + bs[t].astype(np.float32).astype(np.float64)
        want = nn_ref._celu(z) if activation == "celu" else z
        got = outs[t].cpu().numpy().astype(np.float64)
        assert got.shape == want.shape
        if want.size == 0:
            continue
        # float32 products summed over 384 terms: the bound scales with the sum of the terms' magnitudes
        mag = np.abs(rows) @ np.abs(Ws[t]) + np.abs(bs[t])
        assert np.all(np.abs(got - want) <= 1e-6 * mag + 1e-7), (t, np.abs(got - want).max())
        lib = torch.addmm(bt[t], feats[t].reshape(-1, 384), wt[t].t())
        lib = torch.nn.functional.celu(lib, 0.1) if activation == "celu" else lib
        assert np.all(np.abs(lib.cpu().numpy() - want) <= 1e-6 * mag + 1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("k,n_out", [(128, 128), (128, 64), (64, 128), (128, 384), (384, 128)])
def test_dense_kernel_shapes_forward_and_data_gradient(k, n_out):
    """khan_dense_f32 for every (input width, output width) the default network 384-128-128-64-1 needs, forward
    (bias + CELU) and as the data gradient of a layer (rows times CELU' taken from saved activations, weights read the
    other way round): against float64 numpy, row counts on and off the 128-row tile, an empty type."""
    from khan_amd import ops
    dev = "cuda:0"
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a.astype(np.float32))).to(dev)
    rng = np.random.default_rng(k * 1000 + n_out)
    ns = [0, 1, 128, 300]
    xs = [rng.standard_normal((n, k)) for n in ns]
    hs = [rng.standard_normal((n, k)) * 0.2 for n in ns]           # activations the derivative is taken from
    Wt = [rng.standard_normal((n_out, k)) * (2.0 / (k + n_out)) ** 0.5 for _ in range(4)]
    bs = [rng.standard_normal(n_out) * 0.1 for _ in range(4)]
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    fwd = ops.dense([d(x) for x in xs], [d(w) for w in Wt], [d(v) for v in bs], ops.ACT_CELU, 0.1)
    lin = ops.dense([d(x) for x in xs], [d(w) for w in Wt], None, ops.ACT_NONE, 0.1)
    bwd = ops.dense([d(x) for x in xs], [d(w) for w in Wt], None, ops.ACT_NONE, 0.1, deriv_of=[d(h) for h in hs])
    for t in range(4):
        x, h, w, b_ = f32(xs[t]), f32(hs[t]), f32(Wt[t]), f32(bs[t])
        mag = np.abs(x) @ np.abs(w.T) + np.abs(b_)
        for name, got, want in (("forward", fwd[t], nn_ref._celu(x @ w.T + b_)), ("plain", lin[t], x @ w.T),
                                ("data gradient", bwd[t], (x * np.where(h >= 0, 1.0, h / 0.1 + 1.0)) @ w.T)):
            got = got.cpu().numpy().astype(np.float64)
            assert got.shape == want.shape == (ns[t], n_out), (name, t)
            if want.size:
                assert np.all(np.isfinite(got)) and np.all(np.abs(got - want) <= 2e-6 * mag + 1e-7), (name, t, np.abs(got - want).max())


@pytest.mark.gpu
@pytest.mark.parametrize("k", [128, 192, 64])
def test_output_layer_folded_into_the_last_hidden_layer(k):
    """khan_dense_head_f32 / khan_dense_head_grad_f32 (the 64 -> 1 output layer inside the launch of the 64-wide layer
    before it, both ways) against float64 numpy: row counts on and off the 128-row tile, an empty type, with and
    without the output layer's bias, and no activation in the hidden layer."""
    from khan_amd import ops
    dev = "cuda:0"
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a.astype(np.float32))).to(dev)
    rng = np.random.default_rng(7000 + k)
    ns = [300, 0, 129, 1]
    xs = [rng.standard_normal((n, k)) for n in ns]
    Wt = [rng.standard_normal((64, k)) * (2.0 / (k + 64)) ** 0.5 for _ in range(4)]
    bs = [rng.standard_normal(64) * 0.1 for _ in range(4)]
    hw = [rng.standard_normal(64) * 0.2 for _ in range(4)]
    hb = [rng.standard_normal(1) for _ in range(4)]
    f32 = lambda a: a.astype(np.float32).astype(np.float64)
    for act, with_hb in ((ops.ACT_CELU, True), (ops.ACT_CELU, False), (ops.ACT_NONE, True)):
        outs, heads = ops.dense_head([d(x) for x in xs], [d(w) for w in Wt], [d(v) for v in bs], [d(v) for v in hw],
                                     [d(v) for v in hb] if with_hb else None, act, 0.1)
        plain = ops.dense([d(x) for x in xs], [d(w) for w in Wt], [d(v) for v in bs], act, 0.1)
        for t in range(4):
            x, w, b_, v, c = f32(xs[t]), f32(Wt[t]), f32(bs[t]), f32(hw[t]), f32(hb[t])
            z = x @ w.T + b_
            h = nn_ref._celu(z) if act == ops.ACT_CELU else z
            want = h @ v + (c[0] if with_hb else 0.0)
            assert torch.equal(outs[t], plain[t]), t                      # the hidden activations are the plain layer's
            got = heads[t].cpu().numpy().astype(np.float64)
            assert got.shape == (ns[t],)
            if ns[t]:
                mag = (np.abs(x) @ np.abs(w.T) + np.abs(b_)) @ np.abs(v) + abs(c[0])
                assert np.all(np.isfinite(got)) and np.all(np.abs(got - want) <= 2e-6 * mag + 1e-7), (t, np.abs(got - want).max())
    # the way back: scale[r] * head_w[c] * CELU'(h[r, c]), times the hidden layer's weights as stored ([n_in, 64])
    n_in = 128
    Wst = [rng.standard_normal((n_in, 64)) * (2.0 / (n_in + 64)) ** 0.5 for _ in range(4)]
    hs = [rng.standard_normal((n, 64)) * 0.2 for n in ns]
    sc = [rng.standard_normal(n) for n in ns]
    got4 = ops.dense_head_grad([d(v) for v in sc], [d(v) for v in hw], [d(w) for w in Wst], [d(h) for h in hs], 0.1)
    two_step = ops.dense([d(sc[t][:, None] * hw[t][None, :]) for t in range(4)], [d(w) for w in Wst], None, ops.ACT_NONE, 0.1,
                         deriv_of=[d(h) for h in hs])
    for t in range(4):
        s_, v, h, w = f32(sc[t]), f32(hw[t]), f32(hs[t]), f32(Wst[t])
        up = s_[:, None] * v[None, :] * np.where(h >= 0, 1.0, h / 0.1 + 1.0)
        want = up @ w.T
        got = got4[t].cpu().numpy().astype(np.float64)
        assert got.shape == (ns[t], n_in)
        if ns[t]:
            mag = np.abs(up) @ np.abs(w.T)
            assert np.all(np.isfinite(got)) and np.all(np.abs(got - want) <= 2e-6 * mag + 1e-7), (t, np.abs(got - want).max())
            assert np.all(np.abs(got - two_step[t].cpu().numpy()) <= 2e-6 * mag + 1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_molecule_sums_of_the_type_outputs_and_the_way_back(dtype):
    """khan_mol_energy / khan_mol_energy_grad (the gather to atom order + segment sum by molecule of nn.py:165-177 in one
    launch) against numpy: organic molecules with an empty molecule in the middle and a type outside 0..3 (counted as O,
    as the sort does); the sums are the same bits on every call, and the autograd wiring returns the way back."""
    from khan_amd import ops, autograd, datagen
    dev = "cuda:0"
    tdt = getattr(torch, dtype)
    b = datagen.make_batch("organic", 300)
    A = b.A.copy()
    A[7] = 9                                         # out of range: the O bucket
    mol_idxs = b.mol_idxs.copy()
    mol_idxs[mol_idxs >= 150] += 1                   # molecule 150 is empty
    n_mols = b.n_mols + 1
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    macs, mos = ops.mol_offsets(d(mol_idxs), n_mols)
    sc, ga, ac = ops.ani_sort(d(A))
    acs = [int(v) for v in ac.cpu().tolist()]
    rng = np.random.default_rng(5)
    outs = [rng.standard_normal(c) for c in acs]
    t_of = np.minimum(np.where(A < 0, 3, A), 3)
    sis = sc.cpu().numpy()
    per_atom = np.array([outs[t_of[g]][sis[g]] for g in range(len(A))])
    want = np.zeros(n_mols)
    np.add.at(want, mol_idxs, per_atom)
    touts = [d(o).to(tdt) for o in outs]
    e = ops.mol_energy(touts, d(A), sc, mos, macs)
    tol = 1e-5 if dtype == "float32" else 1e-13
    mag = np.zeros(n_mols)
    np.add.at(mag, mol_idxs, np.abs(per_atom))
    assert e.shape == (n_mols,) and np.all(np.abs(e.cpu().numpy() - want) <= tol * mag + 1e-30)
    assert float(e[150]) == 0.0
    assert torch.equal(e, ops.mol_energy(touts, d(A), sc, mos, macs))             # fixed summation order
    ge = rng.standard_normal(n_mols)
    gs = ops.mol_energy_grad(d(ge).to(tdt), d(A), sc, mos, macs, acs)
    for t in range(4):
        wg = np.zeros(acs[t])
        sel = t_of == t
        wg[sis[sel]] = ge[mol_idxs[sel]]
        assert np.array_equal(gs[t].cpu().numpy(), wg.astype(getattr(np, dtype)))
    leaves = [o.clone().requires_grad_(True) for o in touts]
    (autograd.mol_energy(leaves, d(A), sc, mos, macs) * d(ge).to(tdt)).sum().backward()
    for t in range(4):
        assert torch.equal(leaves[t].grad, gs[t])


@pytest.mark.gpu
def test_kernel_layers_agree_with_library_layers_in_energy_and_gradient():
    """The float32 model with its CELU layers in khan_dense_f32 against the same model with every layer a library
    product: energies and coordinate gradients of 200 molecules."""
    b, mols = _molecules(n_mols=200, first=40)
    ys = [0.0] * len(mols)
    res = []
    for kernel in (True, False):
        m = model.AniModel(model.DEFAULT_LAYERS, model.celu, torch.float32, "cuda:0", seed=9, first_layer_kernel=kernel)
        assert m.near.kernel_layers() == (3 if kernel else 0)
        rd = RawDataset(mols, ys)
        res.append((np.asarray(m.predict(rd, batch_size=64)), np.concatenate(list(m.coordinate_gradients(rd, batch_size=64)), axis=0)))
    (e1, g1), (e0, g0) = res
    assert np.abs(e1 - e0).max() <= 2e-5 * max(1.0, np.abs(e0).max())
    assert np.abs(g1 - g0).max() <= 2e-4 * max(1e-3, np.abs(g0).max())


@pytest.mark.gpu
def test_kernel_layers_give_the_library_layers_weight_gradients():
    """Training through the kernel layers (`weights_need_grad`): d sum(energies) / d every weight and bias against
    the same model with library layers, on one batch; a network of other widths (384-192-64-1) goes through the plain kernel."""
    from khan_amd.batching import DeviceBatch
    b, _ = _molecules(n_mols=120, first=7)
    dev = "cuda:0"
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    batch = DeviceBatch.from_device_arrays(d(b.X), d(b.Y), d(b.Z), d(b.A), d(b.mol_idxs), b.n_mols)
    for layers in (model.DEFAULT_LAYERS, (192, 64, 1)):
        grads = []
        for kernel in (True, False):
            m = model.AniModel(layers, model.celu, torch.float32, dev, seed=3, first_layer_kernel=kernel)
            m.near.weights_need_grad = True
            assert m.near.kernel_layers() == ((len(layers) - 1) if kernel else 0)
            names = sorted(m.near.params)
            feats = autograd.featurize(batch.xs, batch.ys, batch.zs, batch.atom_types, batch.mol_offsets,
                                       batch.mol_atom_counts, batch.scatter_idxs, batch.host_counts()[0])
            atom_e = m.near.atom_outputs(feats, batch.gather_idxs)
            gs = torch.autograd.grad(atom_e.sum(), [m.near.params[k] for k in names])
            grads.append([g.cpu().numpy().astype(np.float64) for g in gs])
        for name, g1, g0 in zip(names, grads[0], grads[1]):
            assert np.abs(g1 - g0).max() <= 2e-4 * max(1e-6, np.abs(g0).max()), (layers, name, np.abs(g1 - g0).max())


@pytest.mark.gpu
def test_energy_server_round_trip_over_a_socket():
    b, mols = _molecules(n_mols=2, first=11)
    m = _gpu_model(torch.float64, seed=5)
    listening = server.connect_socket("127.0.0.1", 0, server=True)        # port 0: the system picks a free one
    port = listening.getsockname()[1]
    th = threading.Thread(target=server.serve_on, args=(listening, m, 1), daemon=True)
    th.start()
    c = server.connect_socket("127.0.0.1", port, server=False)
    try:
        for k, X in enumerate(mols):
            server.send(c, json.dumps({"X": X.tolist()}))
            doc = json.loads(server.receive(c))
            s = slice(b.MOs[k], b.MOs[k] + b.MACs[k])
            want_e, want_g = nn_ref.energies_and_gradients(b.X[s], b.Y[s], b.Z[s], b.A[s], np.array([0], dtype=np.int32),
                                                           b.MACs[k:k + 1], _np_params(m), model.DEFAULT_LAYERS)
            # the reference adds the float32 table entries up in float32, atom after atom (energy_server.py:159-162)
            self_e = np.float32(0)
            for t in b.A[s]:
                self_e = np.float32(self_e + server.SELF_INTERACTION[int(t)])
            e_ref = want_e[0] + float(self_e)
            assert abs(doc["energy"] - e_ref) <= 1e-9 * abs(e_ref)
            got = np.array(doc["gradient"]).reshape(-1, 3)
            assert np.max(np.abs(got - want_g * server.BOHR)) <= 1e-10 * max(1.0, np.max(np.abs(want_g)))
        server.send(c, '{"X": []}')
        assert "error" in json.loads(server.receive(c))
    finally:
        server.close_connection(c)
    th.join(30)
    assert not th.is_alive()


@pytest.mark.gpu
def test_force_loss_reaches_the_weights_through_the_kernel_layers():
    """A loss on forces (the coordinate gradient of the energy, taken with create_graph) differentiated with respect to
    every weight and bias -- what force training does (khan/training/trainer_multi_tower.py:418-430) -- through the
    kernel layers against the same model with library layers.  The kernel layers' own way back records no graph; asked
    for one, they form the layer from library operations, and the force term must arrive in the weight gradients."""
    from khan_amd.batching import DeviceBatch
    b, _ = _molecules(n_mols=60, first=11)
    dev = "cuda:0"
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    batch = DeviceBatch.from_device_arrays(d(b.X), d(b.Y), d(b.Z), d(b.A), d(b.mol_idxs), b.n_mols)
    target = torch.from_numpy(np.random.default_rng(5).standard_normal((b.n_atoms, 3)).astype(np.float32)).to(dev)
    grads, force_only = [], []
    for kernel in (True, False):
        m = model.AniModel(model.DEFAULT_LAYERS, model.celu, torch.float32, dev, seed=4, first_layer_kernel=kernel)
        m.near.weights_need_grad = True
        assert m.near.kernel_layers() == (3 if kernel else 0)
        names = sorted(m.near.params)
        xs, ys, zs = (t.detach().clone().requires_grad_(True) for t in (batch.xs, batch.ys, batch.zs))
        feats = autograd.featurize(xs, ys, zs, batch.atom_types, batch.mol_offsets, batch.mol_atom_counts,
                                   batch.scatter_idxs, batch.host_counts()[0])
        energies = autograd.mol_energy(m.near.type_outputs(feats), batch.atom_types, batch.scatter_idxs,
                                       batch.mol_offsets, batch.mol_atom_counts)
        gx, gy, gz = torch.autograd.grad(energies.sum(), (xs, ys, zs), create_graph=True)
        assert gx.requires_grad                               # the forces carry a graph back to the weights
        force_loss = ((torch.stack((gx, gy, gz), dim=1) - target) ** 2).sum()
        params = [m.near.params[k] for k in names]
        gf = torch.autograd.grad(force_loss, params, retain_graph=True, allow_unused=True)
        gs = torch.autograd.grad(energies.sum() + 0.1 * force_loss, params)
        force_only.append([None if g is None else g.cpu().numpy().astype(np.float64) for g in gf])
        grads.append([g.cpu().numpy().astype(np.float64) for g in gs])
    for name, g1, g0, f1, f0 in zip(names, grads[0], grads[1], force_only[0], force_only[1]):
        # the output layer's bias does not move the forces; every other parameter does
        if f0 is None or np.abs(f0).max() == 0.0:
            assert f1 is None or np.abs(f1).max() == 0.0, name
        else:
            assert f1 is not None and np.abs(f1 - f0).max() <= 5e-4 * np.abs(f0).max(), (name, np.abs(f1 - f0).max(), np.abs(f0).max())
        assert np.abs(g1 - g0).max() <= 5e-4 * max(1e-6, np.abs(g0).max()), (name, np.abs(g1 - g0).max())


def _network_f64(x, Ws, bs, w4, b4, scale, alpha=0.1):
    """The 384-128-128-64-1 CELU network and its gradient with respect to the rows in float64 numpy."""
    acts, a = [], x
    for W, b_ in zip(Ws, bs):
        a = nn_ref._celu(a @ W + b_)
        acts.append(a)
    value = a @ w4 + b4
    g = (scale[:, None] * w4[None, :]) * np.where(acts[2] >= 0, 1.0, acts[2] / alpha + 1.0)
    g = (g @ Ws[2].T) * np.where(acts[1] >= 0, 1.0, acts[1] / alpha + 1.0)
    g = (g @ Ws[1].T) * np.where(acts[0] >= 0, 1.0, acts[0] / alpha + 1.0)
    return value, g @ Ws[0].T


@pytest.mark.gpu
@pytest.mark.parametrize("with_scale", [False, True])
def test_whole_network_in_one_launch_matches_float64(with_scale):
    """khan_atomic_networks_f32 (the three CELU layers and the output layer of the four types in one launch, the
    hidden activations never leaving the compute unit, and the gradient back to the rows in the same launch) against
    float64 numpy on the same float32 operands: row counts on and off the 128-row tile, an empty type, one row; values
    only (no gradient asked for) must equal the values of the launch that also forms the gradient."""
    from khan_amd import ops
    dev = "cuda:0"
    f32 = lambda a: np.ascontiguousarray(a.astype(np.float32))
    d = lambda a: torch.from_numpy(f32(a)).to(dev)
    rng = np.random.default_rng(11)
    ns = [0, 1, 300, 1024 + 77]
    widths = (384, 128, 128, 64)
    xs = [np.abs(rng.standard_normal((n, 384))) * 0.5 for n in ns]          # feature rows are non-negative
    Ws = [[rng.standard_normal((widths[l], widths[l + 1])) * (2.0 / (widths[l] + widths[l + 1])) ** 0.5 for l in range(3)] for _ in range(4)]
    bs = [[rng.standard_normal(widths[l + 1]) * 0.1 for l in range(3)] for _ in range(4)]
    w4 = [rng.standard_normal(64) * 0.2 for _ in range(4)]
    b4 = [rng.standard_normal(1) for _ in range(4)]
    scales = [rng.standard_normal(n) for n in ns]
    weights = [[d(Ws[t][l]) for t in range(4)] for l in range(3)]
    weights_t = [[d(Ws[t][l].T) for t in range(4)] for l in range(3)]
    biases = [[d(bs[t][l]) for t in range(4)] for l in range(3)]
    rows = [d(x) for x in xs]
    vals, grads = ops.atomic_networks(rows, weights_t, biases, [d(w) for w in w4], [d(b_) for b_ in b4], weights=weights,
                                      scales=[d(sc) for sc in scales] if with_scale else None, want_grad=True)
    vals_only, none = ops.atomic_networks(rows, weights_t, biases, [d(w) for w in w4], [d(b_) for b_ in b4])
    assert none is None
    # the weights split once beforehand: the same bits out
    packed = ops.pack_network_weights(weights_t, weights)
    vals_p, grads_p = ops.atomic_networks(rows, None, biases, [d(w) for w in w4], [d(b_) for b_ in b4], packed=packed,
                                          scales=[d(sc) for sc in scales] if with_scale else None, want_grad=True)
    for t in range(4):
        assert torch.equal(vals_p[t], vals[t]) and torch.equal(grads_p[t], grads[t])
    for t in range(4):
        up = lambda a: f32(a).astype(np.float64)
        sc = up(scales[t]) if with_scale else np.ones(ns[t])
        want_v, want_g = _network_f64(up(xs[t]), [up(W) for W in Ws[t]], [up(b_) for b_ in bs[t]], up(w4[t]), up(b4[t])[0], sc)
        got_v, got_g = vals[t].cpu().numpy().astype(np.float64), grads[t].cpu().numpy().astype(np.float64)
        assert got_v.shape == (ns[t],) and got_g.shape == (ns[t], 384)
        assert torch.equal(vals[t], vals_only[t])
        if ns[t] == 0:
            continue
        # float32 products through four layers: relative to the size of the values / of the largest gradient entry of the row
        vscale = np.abs(want_v).max() + 1.0
        assert np.all(np.isfinite(got_v)) and np.abs(got_v - want_v).max() <= 2e-5 * vscale, (t, np.abs(got_v - want_v).max(), vscale)
        gscale = np.abs(want_g).max(axis=1, keepdims=True) + 1e-6
        assert np.all(np.isfinite(got_g)) and np.all(np.abs(got_g - want_g) <= 5e-5 * gscale), (t, (np.abs(got_g - want_g) / gscale).max())


@pytest.mark.gpu
def test_whole_network_operand_range():
    """khan_atomic_networks_f32 forms its products from two half-precision parts per float32 operand.  Pinned here: the
    accuracy does not depend on the size of the upstream factors (1e-8, 1e+6: the gradient is carried for a unit factor
    and scaled when it is stored) nor degrade for small feature rows (1e-4), and a feature beyond half precision's
    range (1e5 > 65,504) turns that row's value and gradient into NaN -- no wrong finite number -- and no other row's."""
    from khan_amd import ops
    dev = "cuda:0"
    f32 = lambda a: np.ascontiguousarray(a.astype(np.float32))
    d = lambda a: torch.from_numpy(f32(a)).to(dev)
    up = lambda a: f32(a).astype(np.float64)
    rng = np.random.default_rng(5)
    widths = (384, 128, 128, 64)
    n = 700
    Ws = [rng.standard_normal((widths[l], widths[l + 1])) * (2.0 / (widths[l] + widths[l + 1])) ** 0.5 for l in range(3)]
    bs = [rng.standard_normal(widths[l + 1]) * 0.1 for l in range(3)]
    w4, b4 = rng.standard_normal(64) * 0.2, rng.standard_normal(1)
    empty = torch.zeros((0, 384), device=dev)
    none = torch.zeros(0, device=dev)
    wt = [[d(Ws[l].T)] * 4 for l in range(3)]
    w = [[d(Ws[l])] * 4 for l in range(3)]
    bi = [[d(bs[l])] * 4 for l in range(3)]

    def launch(x, sc):
        vals, grads = ops.atomic_networks([empty, d(x), empty, empty], wt, bi, [d(w4)] * 4, [d(b4)] * 4, weights=w,
                                          scales=[none, d(sc), none, none], want_grad=True)
        return vals[1].cpu().numpy().astype(np.float64), grads[1].cpu().numpy().astype(np.float64)

    worst = {}
    for name, xscale, sscale in (("ordinary", 0.5, 1.0), ("features 1e-4", 1e-4, 1.0), ("upstream 1e-8", 0.5, 1e-8), ("upstream 1e+6", 0.5, 1e6)):
        x = np.abs(rng.standard_normal((n, 384))) * xscale
        sc = rng.standard_normal(n) * sscale
        want_v, want_g = _network_f64(up(x), [up(W) for W in Ws], [up(b_) for b_ in bs], up(w4), up(b4)[0], up(sc))
        got_v, got_g = launch(x, sc)
        ev = np.abs(got_v - want_v).max() / (np.abs(want_v).max() + 1.0)
        eg = (np.abs(got_g - want_g) / (np.abs(want_g).max(axis=1, keepdims=True) + 1e-300)).max()
        worst[name] = (ev, eg)
        assert np.isfinite(got_v).all() and np.isfinite(got_g).all(), name
        assert ev <= 5e-6 and eg <= 2e-5, (name, ev, eg)
    print("\none-launch networks, worst value / gradient error relative to the largest value / the row's largest entry:", worst)
    # the same relative accuracy whatever the upstream factors' size
    assert worst["upstream 1e-8"][1] <= 1.5 * worst["ordinary"][1] + 1e-6 and worst["upstream 1e+6"][1] <= 1.5 * worst["ordinary"][1] + 1e-6

    x = np.abs(rng.standard_normal((n, 384))) * 0.5
    sc = np.ones(n)
    clean_v, clean_g = launch(x, sc)
    x[300, 17] = 1.0e5
    got_v, got_g = launch(x, sc)
    assert not np.isfinite(got_v[300]) and not np.isfinite(got_g[300]).any()
    keep = np.arange(n) != 300
    assert np.array_equal(got_v[keep], clean_v[keep]) and np.array_equal(got_g[keep], clean_g[keep])
