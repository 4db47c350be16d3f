"""Backward passes of the layer Functions against closed forms evaluated independently in numpy float64.

Nothing here calls a helper of bgemm_linear.py: every expected gradient is written out from the reference's
backward methods (tests/python/bgemm_linear.py:28-42 matmul, :64-86 attention matmul, :149-165 linear,
:186-219 Bi-Real surrogate 2 - 2|x|, :277-347 elastic with 2 exp(-t^2), :382-457 elastic with 2 / cosh^2,
:519-535 scale gradients; the reference calls the last with three arguments where four are required, the
four-argument form is what is evaluated).

Tolerances.  The straight-through products (grad @ sign(W), sign(X)^T @ grad) run in fp16 like the
reference's (the saved tensors are halves); the upstream gradients are drawn from {-1, -1/2, 0, 1/2, 1}, so every
sum is a small multiple of 1/2, exact in fp16: those gradients must be EQUAL.  The Bi-Real factor is one fp16
multiply: one fp16 ulp (2^-10 relative).  The elastic layers run in fp32 with device reductions (means) whose
summation order differs from numpy's: 1e-4 of the largest magnitude.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import bgemm_linear as bl

DEV = "cuda:0"


def halves(rng, *shape):
    """fp32 values that survive a round trip through fp16, with exact zeros of both signs mixed in."""
    a = rng.standard_normal(shape).astype(np.float16)
    z = rng.random(shape) < 0.03
    a[z] = np.float16(0.0)
    a[z & (rng.random(shape) < 0.5)] = np.float16(-0.0)
    return a.astype(np.float32)


def upstream(rng, *shape):
    return rng.choice(np.array([-1.0, -0.5, 0.0, 0.5, 1.0], dtype=np.float32), size=shape)


def run(fn, g, *inputs):
    """fn(*tensors) -> out; returns the gradients of sum(out * g) with respect to every input, as float64 arrays."""
    ts = [torch.from_numpy(np.ascontiguousarray(a)).to(DEV).requires_grad_(True) for a in inputs]
    out = fn(*ts)
    (out.float() * torch.from_numpy(g).to(DEV)).sum().backward()
    return [t.grad.double().cpu().numpy() for t in ts]


def test_linear_straight_through_gradients_are_exact():
    rng = np.random.default_rng(1)
    x, w, g = halves(rng, 32, 128), halves(rng, 16, 128), upstream(rng, 32, 16)
    gx, gw = run(lambda a, b: bl.bgemm_linear.apply(a, b), g, x, w)
    xs, ws = np.sign(x.astype(np.float64)), np.sign(w.astype(np.float64))        # torch.sign: 0 -> 0
    assert (gx == g.astype(np.float64) @ ws).all()                                # feat_grad = grad @ sign(W)
    assert (gw == g.astype(np.float64).T @ xs).all()                              # weight_grad = (sign(X)^T @ grad)^T
    # leading batch dimensions fold into the rows
    x3, g3 = halves(rng, 4, 8, 128), upstream(rng, 4, 8, 16)
    gx3, gw3 = run(lambda a, b: bl.bgemm_linear.apply(a, b), g3, x3, w)
    assert (gx3 == g3.astype(np.float64) @ ws).all()
    assert (gw3 == np.einsum("bnm,bnk->mk", g3.astype(np.float64), np.sign(x3.astype(np.float64)))).all()


def test_bireal_surrogate_gradient():
    rng = np.random.default_rng(2)
    x, w, g = 1.5 * halves(rng, 32, 128), halves(rng, 16, 128), upstream(rng, 32, 16)
    x = x.astype(np.float16).astype(np.float32)
    gx, gw = run(lambda a, b: bl.bgemm_linear_bireal.apply(a, b), g, x, w)
    ws, xs = np.sign(w.astype(np.float64)), np.sign(x.astype(np.float64))
    dx = 2.0 - 2.0 * np.minimum(np.abs(x.astype(np.float64)), 1.0)                # 2 + 2x on (-1, 0), 2 - 2x on (0, 1), else 0
    want = (g.astype(np.float64) @ ws) * dx
    assert np.abs(gx - want).max() <= 2.0 ** -10 * np.abs(want).max()             # one fp16 multiply
    assert (gx[np.abs(x) >= 1] == 0).all() and (np.abs(x) >= 1).any()             # the surrogate vanishes outside (-1, 1)
    assert (gw == g.astype(np.float64).T @ xs).all()                              # the weight gradient is plain straight-through


def test_matmul_gradients_2d_and_batched():
    rng = np.random.default_rng(3)
    a, b, g = halves(rng, 32, 64), halves(rng, 64, 48), upstream(rng, 32, 48)
    ga, gb = run(lambda p, q: bl.bgemm_matmul.apply(p, q), g, a, b)
    sa_, sb = np.sign(a.astype(np.float64)), np.sign(b.astype(np.float64))
    assert (ga == g.astype(np.float64) @ sb.T).all()                              # matA_grad = grad @ sign(B)^T
    assert (gb == sa_.T @ g.astype(np.float64)).all()                             # matB_grad = sign(A)^T @ grad
    q, kt, g4 = halves(rng, 2, 3, 32, 64), halves(rng, 2, 3, 64, 32), upstream(rng, 2, 3, 32, 32)
    gq, gk = run(lambda p, r: bl.bgemm_matmul.apply(p, r), g4, q, kt)
    assert (gq == g4.astype(np.float64) @ np.swapaxes(np.sign(kt.astype(np.float64)), -1, -2)).all()
    assert (gk == np.swapaxes(np.sign(q.astype(np.float64)), -1, -2) @ g4.astype(np.float64)).all()


def test_attention_matmul_gradients():
    rng = np.random.default_rng(4)
    attn, v, g = halves(rng, 32, 64), halves(rng, 64, 16), upstream(rng, 32, 16)
    ga, gv = run(lambda p, q: bl.bgemm_attn_matmul.apply(p, q), g, attn, v)
    a01 = (np.sign(attn.astype(np.float64)) + 1) / 2                              # {-1, 0, 1} -> {0, 1/2, 1} ...
    a01[a01 == 0] = 1                                                             # ... and the reference's where(== 0 -> 1) (:70-71)
    assert (ga == g.astype(np.float64) @ np.sign(v.astype(np.float64)).T / 2).all()
    assert (gv == a01.T @ g.astype(np.float64)).all()


@pytest.mark.parametrize("name", ["bgemm_linear_elastic_signed", "nn_linear_elastic_signed"])
def test_elastic_gradients_including_the_scales(name):
    fn = getattr(bl, name)
    surrogate, clip = ((lambda t: 2.0 / np.cosh(t) ** 2), 4.0) if name == "bgemm_linear_elastic_signed" else ((lambda t: 2.0 * np.exp(-t ** 2)), 1.0)
    rng = np.random.default_rng(5)
    N, K, M = 32, 128, 16
    inp = rng.standard_normal((N, K)).astype(np.float32) * 1.7 + 0.3              # values beyond +-1 after the scaling, a mean to remove
    wt = rng.standard_normal((M, K)).astype(np.float32) * 0.05 + 0.01
    g = upstream(rng, N, M)
    sa, sw = np.float32(0.9), rng.uniform(0.01, 0.03, M).astype(np.float32)
    grad_scale = 1.0 / np.sqrt(N * K)
    ginp, gwt, gsa, gsw = run(lambda a, b, c, d: fn.apply(a, b, c, d, grad_scale), g, inp, wt, np.asarray(sa), sw)

    x = (inp.astype(np.float64) - inp.astype(np.float64).mean()) / sa             # forward: x = (input - mean) / sa, w = weight - mean
    w = wt.astype(np.float64) - wt.astype(np.float64).mean()
    # out = (ternary(x) @ ternary(w)^T) * sa * sw: the Function sees d(loss)/d(out) = g and returns gradients for
    # its four inputs from the straight-through products of that g
    feat = g.astype(np.float64) @ np.sign(w)                                      # feat_grad = grad @ ternary(W)
    wgrad = g.astype(np.float64).T @ np.sign(x)                                   # weight_grad = (ternary(X)^T @ grad)^T
    small, big = (x < -1).astype(np.float64), (x > 1).astype(np.float64)
    inner = big - small + (1 - small - big) * (np.sign(x) - x)                    # Qn = -1, Qp = 1
    want_sa = (inner * feat * grad_scale).sum()                                   # summed over the row, then to sa's shape
    want_sw = (np.sign(w) * wgrad * grad_scale).sum(-1)
    want_inp = feat * surrogate(np.minimum(np.abs(x), clip))
    want_wt = wgrad * surrogate(np.minimum(np.abs(w), clip))
    tol = lambda want: 1e-4 * max(np.abs(want).max(), 1e-6)
    assert np.abs(ginp - want_inp).max() <= tol(want_inp)
    assert np.abs(gwt - want_wt).max() <= tol(want_wt)
    assert abs(float(np.asarray(gsa).sum()) - want_sa) <= 1e-4 * max(abs(want_sa), np.abs(inner * feat * grad_scale).sum() * 1e-2)
    assert np.abs(gsw - want_sw).max() <= tol(want_sw)
    assert (big.sum() > 0) and (small.sum() > 0)                                  # all three branches of the scale gradient are hit


def test_module_gradients_reach_the_scales_with_these_values():
    """The modules hand the Functions x - zpa and w - zpw (linear, Bi-Real) resp. the raw tensors and the learned
    scales (elastic): the parameter gradients are the Function gradients above times the module's own factors."""
    rng = np.random.default_rng(6)
    N, K, M = 32, 128, 16
    x = halves(rng, N, K)
    lin = bl.BGEMMLinear(K, M, bias=True).to(DEV)
    xt = torch.from_numpy(x).to(DEV)
    y = lin(xt)                                               # initialises sw, sa, zpw, zpa from this batch
    g = upstream(rng, N, M)
    (y.float() * torch.from_numpy(g).to(DEV)).sum().backward()
    w = lin.weight.detach().double().cpu().numpy()
    sw, sa = lin.sw.detach().double().cpu().numpy(), float(lin.sa.detach())
    zpw, zpa = float(lin.zpw), float(lin.zpa)
    xs = np.sign((x.astype(np.float32) - np.float32(zpa)).astype(np.float16).astype(np.float64))
    ws = np.sign((w.astype(np.float32) - np.float32(zpw)).astype(np.float16).astype(np.float64))
    acc = xs @ ws.T                                            # what the kernel returned (as fp16, exact: |acc| <= 128)
    gout = g.astype(np.float64) * sw[None, :] * sa            # d loss / d kernel output
    assert np.abs(lin.weight.grad.double().cpu().numpy() - gout.T @ xs).max() <= 2.0 ** -9 * np.abs(gout.T @ xs).max()
    assert np.abs(lin.sw.grad.double().cpu().numpy() - (g * acc * sa).sum(0)).max() <= 1e-4 * np.abs((g * acc * sa).sum(0)).max()
    assert abs(float(lin.sa.grad) - (g * acc * sw[None, :]).sum()) <= 1e-4 * np.abs(g * acc * sw[None, :]).sum()
    assert np.abs(lin.bias.grad.double().cpu().numpy() - g.sum(0)).max() == 0
