"""Pins of the AMP discriminator-loss oracle (CPU): closed forms, brute-force input gradients, finite differences."""
import numpy as np

from oracle import amp as oamp

ACTS = {"elu": lambda z: np.where(z > 0, z, np.expm1(np.minimum(z, 0))), "tanh": np.tanh, "relu": lambda z: np.maximum(z, 0),
        "none": lambda z: z}


def _net(x, ws, bs, act):
    h = x
    for i, (w, b) in enumerate(zip(ws, bs)):
        h = h @ w.T + b
        if i + 1 < len(ws):
            h = ACTS[act](h)
    return h[..., 0]


def _loss_numpy(ws, bs, real, sim, coef, act, eps=1e-6):
    """The loss with the input gradient taken by central differences, one input coordinate at a time."""
    total = 0.5 * ((_net(real, ws, bs, act) - 1) ** 2).sum() + 0.5 * ((_net(sim, ws, bs, act) + 1) ** 2).sum()
    B, T, F = real.shape
    sq = np.zeros(B)
    for f in range(F):
        e = np.zeros(F); e[f] = eps
        d = (_net(real + e, ws, bs, act) - _net(real - e, ws, bs, act)) / (2 * eps)   # (B, T): d logit[b, t] / d x[b, t, f]
        sq += (d ** 2).sum(axis=1)
    return total + coef / 2 * sq.mean()


def _random(dims, B, T, B2, T2, seed):
    rng = np.random.default_rng(seed)
    ws = [rng.normal(size=(o, i)) / np.sqrt(i) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.normal(size=o) * 0.1 for o in dims[1:]]
    return ws, bs, rng.normal(size=(B, T, dims[0])), rng.normal(size=(B2, T2, dims[0]))


def test_linear_discriminator_closed_forms():
    """D(x) = w.x + b: the input gradient is w for every frame, so the penalty is coef / 2 * T |w|^2 and its gradient
    coef * T * w; the squared-error parts are ordinary least squares."""
    ws, bs, real, sim = _random([5, 1], B=3, T=4, B2=2, T2=6, seed=1)
    coef = 0.7
    losses, grads = oamp.disc_loss_and_grads(ws, bs, real, sim, coef, act="elu")
    w, b = ws[0][0], bs[0][0]
    er, es = real @ w + b - 1, sim @ w + b + 1
    np.testing.assert_allclose(losses, [0.5 * (er ** 2).sum(), 0.5 * (es ** 2).sum(), coef / 2 * 4 * (w @ w)], rtol=1e-12)
    dw = np.einsum("bt,btf->f", er, real) + np.einsum("bt,btf->f", es, sim) + coef * 4 * w
    np.testing.assert_allclose(grads[0][0][0], dw, rtol=1e-12)
    np.testing.assert_allclose(grads[0][1][0], er.sum() + es.sum(), rtol=1e-12)


def test_loss_against_brute_force_input_gradients_and_parameter_differences():
    for act in ("elu", "tanh"):
        dims = [3, 6, 5, 1]
        ws, bs, real, sim = _random(dims, B=2, T=3, B2=3, T2=2, seed=7)
        coef = 1.3
        losses, grads = oamp.disc_loss_and_grads(ws, bs, real, sim, coef, act=act)
        assert losses[2] > 1e-3
        np.testing.assert_allclose(losses.sum(), _loss_numpy(ws, bs, real, sim, coef, act), rtol=1e-8)
        # the penalty averages over motions, not frames: doubling T by repeating the frames doubles it
        l2, _ = oamp.disc_loss_and_grads(ws, bs, np.concatenate([real, real], axis=1), sim, coef, act=act)
        np.testing.assert_allclose(l2[2], 2 * losses[2], rtol=1e-12)
        # single parameters by central differences of the (autograd-free) numpy loss
        rng = np.random.default_rng(3)
        for _ in range(12):
            l = int(rng.integers(len(ws)))
            o, i = int(rng.integers(ws[l].shape[0])), int(rng.integers(ws[l].shape[1]))
            h = 1e-4
            wp = [w.copy() for w in ws]; wm = [w.copy() for w in ws]
            wp[l][o, i] += h; wm[l][o, i] -= h
            fd = (_loss_numpy(wp, bs, real, sim, coef, act) - _loss_numpy(wm, bs, real, sim, coef, act)) / (2 * h)
            np.testing.assert_allclose(grads[l][0][o, i], fd, rtol=2e-5, atol=1e-7)
            bp = [b.copy() for b in bs]; bm = [b.copy() for b in bs]
            bp[l][o] += h; bm[l][o] -= h
            fd = (_loss_numpy(ws, bp, real, sim, coef, act) - _loss_numpy(ws, bm, real, sim, coef, act)) / (2 * h)
            np.testing.assert_allclose(grads[l][1][o], fd, rtol=2e-5, atol=1e-7)


def test_relu_has_no_second_derivative_term():
    """With ReLU the input gradient is piecewise constant in the biases: the penalty's gradient with respect to the hidden
    biases is zero, so those gradients equal the ones without a penalty."""
    ws, bs, real, sim = _random([4, 8, 1], B=2, T=5, B2=2, T2=5, seed=11)
    _, g0 = oamp.disc_loss_and_grads(ws, bs, real, sim, 0.0, act="relu")
    _, g1 = oamp.disc_loss_and_grads(ws, bs, real, sim, 2.0, act="relu")
    np.testing.assert_allclose(g0[0][1], g1[0][1], rtol=1e-12)
    assert np.abs(g0[0][0] - g1[0][0]).max() > 1e-3


def test_disc_loss_terms_on_a_constant_discriminator():
    """`disc_loss` itself: a discriminator with zero weights answers its bias b everywhere, so the real term is
    B T (b - 1)^2 / 2, the simulated term B2 T2 (b + 1)^2 / 2, and the gradient penalty zero."""
    import torch

    ws = [torch.zeros(1, 5, dtype=torch.float64)]
    bs = [torch.tensor([0.25], dtype=torch.float64)]
    real, sim = torch.randn(3, 4, 5, dtype=torch.float64), torch.randn(2, 6, 5, dtype=torch.float64)
    total, lr, ls, gp = (t.detach() for t in oamp.disc_loss(ws, bs, real, sim, 0.7, act="elu"))
    assert float(lr) == 12 * 0.75 ** 2 / 2 and float(ls) == 12 * 1.25 ** 2 / 2 and float(gp) == 0.0
    assert float(total) == float(lr) + float(ls)
