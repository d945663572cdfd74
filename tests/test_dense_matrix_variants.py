"""The dense-layer kernels form their float32 products either on the bfloat16 matrix instructions, every operand split
exactly into three bfloat16 parts (the default), or on the float32 matrix instructions (KHAN_DENSE_MATRIX=f32, read once
per process by libkhan_aev.so, so each form runs in a child process).  Both are checked against a float64 product of
the same float32 inputs, forward with bias and CELU and as a layer's data gradient, at one bound: 2e-6 of
sum |x| |w| -- and the split form has to be as close to float64 as the float32 instructions are."""
import os
import subprocess
import sys

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
import numpy as np, torch
sys.path.insert(0, sys.argv[1])
from khan_amd import ops
z = np.load(sys.argv[2])
d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
out = {}
for tag in ("a", "b"):
    xs = [d(z["%s_x%d" % (tag, t)]) for t in range(4)]
    ws = [d(z["%s_w%d" % (tag, t)]) for t in range(4)]
    bs = [d(z["%s_b%d" % (tag, t)]) for t in range(4)]
    hs = [d(z["%s_h%d" % (tag, t)]) for t in range(4)]
    gw = [d(z["%s_gw%d" % (tag, t)]) for t in range(4)]
    f = ops.dense(xs, ws, bs, ops.ACT_CELU, 0.1)
    g = ops.dense(hs, gw, None, ops.ACT_NONE, 0.1, deriv_of=[d(z["%s_act%d" % (tag, t)]) for t in range(4)])
    for t in range(4):
        out["%s_f%d" % (tag, t)] = f[t].cpu().numpy()
        out["%s_g%d" % (tag, t)] = g[t].cpu().numpy()
torch.cuda.synchronize()
np.savez(sys.argv[3], **out)
"""


def _celu(z, alpha=0.1):
    return np.where(z >= 0, z, alpha * np.expm1(np.minimum(z, 0) / alpha))


def test_both_forms_of_the_products_agree_with_float64(tmp_path):
    rng = np.random.default_rng(99)
    data = {}
    shapes = {"a": (384, 128), "b": (128, 64)}           # (summed width, output width): both tile widths
    ns = [700, 0, 129, 5]
    for tag, (k, n_out) in shapes.items():
        for t in range(4):
            x = rng.standard_normal((ns[t], k)) * np.exp(rng.uniform(-6, 2, (ns[t], k)))      # magnitudes over orders
            data["%s_x%d" % (tag, t)] = x.astype(np.float32)
            data["%s_w%d" % (tag, t)] = (rng.standard_normal((n_out, k)) * (2.0 / (k + n_out)) ** 0.5).astype(np.float32)
            data["%s_b%d" % (tag, t)] = (rng.standard_normal(n_out) * 0.1).astype(np.float32)
            # the way back through a layer of width k with n_out inputs: gradient rows [n, k], weights as stored [n_out, k]
            data["%s_h%d" % (tag, t)] = rng.standard_normal((ns[t], k)).astype(np.float32)
            data["%s_act%d" % (tag, t)] = (rng.standard_normal((ns[t], k)) * 0.2).astype(np.float32)
            data["%s_gw%d" % (tag, t)] = (rng.standard_normal((n_out, k)) * (2.0 / (k + n_out)) ** 0.5).astype(np.float32)
    inp = str(tmp_path / "in.npz")
    np.savez(inp, **data)
    results = {}
    for mode in ("bf16x3", "f32"):
        env = dict(os.environ)
        env.pop("KHAN_DENSE_MATRIX", None)
        if mode == "f32":
            env["KHAN_DENSE_MATRIX"] = "f32"
        out = str(tmp_path / (mode + ".npz"))
        print("child: dense products %s" % mode, flush=True)
        subprocess.run([sys.executable, "-c", CHILD, ROOT, inp, out], env=env, check=True, timeout=300)
        results[mode] = np.load(out)
    worst = {"bf16x3": 0.0, "f32": 0.0}
    for tag in shapes:
        for t in range(4):
            if ns[t] == 0:
                continue
            x, w, b = (data["%s_%s%d" % (tag, v, t)].astype(np.float64) for v in ("x", "w", "b"))
            want_f = _celu(x @ w.T + b)
            mag_f = np.abs(x) @ np.abs(w.T) + np.abs(b)
            h, act, gw = (data["%s_%s%d" % (tag, v, t)].astype(np.float64) for v in ("h", "act", "gw"))
            up = h * np.where(act >= 0, 1.0, act / 0.1 + 1.0)
            want_g = up @ gw.T
            mag_g = np.abs(up) @ np.abs(gw.T)
            for mode, r in results.items():
                for name, want, mag in (("f", want_f, mag_f), ("g", want_g, mag_g)):
                    got = r["%s_%s%d" % (tag, name, t)].astype(np.float64)
                    assert got.shape == want.shape and np.all(np.isfinite(got)), (mode, tag, name, t)
                    ratio = float((np.abs(got - want) / (2e-6 * mag + 1e-7)).max())
                    worst[mode] = max(worst[mode], ratio)
                    assert ratio <= 1.0, (mode, tag, name, t, ratio)
    print("   worst error / bound: split bfloat16 products %.3f, float32 matrix instructions %.3f" % (worst["bf16x3"], worst["f32"]), flush=True)
    # the split products lose nothing against the float32 instructions (both are dominated by the float32 accumulation)
    assert worst["bf16x3"] <= 1.5 * worst["f32"] + 0.05
