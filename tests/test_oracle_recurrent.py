"""Pins the recurrent-network oracle (CPU): the GRU cell against torch's library cell and limits, GELU against torch."""
import numpy as np
import pytest
import torch

from oracle import recurrent as orec


def test_gru_cell_matches_the_library_cell_and_limits():
    rng = np.random.default_rng(0)
    N, I, H = 5, 7, 6
    wi, wh = rng.normal(size=(3 * H, I)), rng.normal(size=(3 * H, H))
    b, bn = rng.normal(size=3 * H), rng.normal(size=H)
    x, h = rng.normal(size=(N, I)), rng.normal(size=(N, H))
    cell = torch.nn.GRUCell(I, H).double()
    with torch.no_grad():
        cell.weight_ih.copy_(torch.from_numpy(wi)); cell.weight_hh.copy_(torch.from_numpy(wh))
        cell.bias_ih.copy_(torch.from_numpy(b))
        cell.bias_hh.copy_(torch.from_numpy(np.concatenate([np.zeros(2 * H), bn])))
        want = cell(torch.from_numpy(x), torch.from_numpy(h)).numpy()
    np.testing.assert_allclose(orec.gru_cell(x, h, wi, wh, b, bn), want, rtol=1e-12, atol=1e-12)
    # update gate saturated open (z -> 1): the state is kept; saturated shut with zero recurrent weights: tanh(W_n x)
    big = np.zeros(3 * H); big[H:2 * H] = 50.0
    np.testing.assert_allclose(orec.gru_cell(x, h, 0 * wi, 0 * wh, big, None), h, atol=1e-12)
    wn = np.zeros_like(wi); wn[2 * H:] = wi[2 * H:]
    np.testing.assert_allclose(orec.gru_cell(x, h, wn, 0 * wh, -big, None), np.tanh(x @ wi[2 * H:].T), atol=1e-12)


def test_gelu_and_network_composition():
    x = np.linspace(-4, 4, 41)
    want = torch.nn.functional.gelu(torch.from_numpy(x), approximate="tanh").numpy()
    np.testing.assert_allclose(orec.gelu(x), want, rtol=1e-12, atol=1e-14)
    rng = np.random.default_rng(1)
    N, I, H, O = 4, 5, 6, 3
    proj = (rng.normal(size=(H, I)), rng.normal(size=H))
    cells = [(rng.normal(size=(3 * H, H)), rng.normal(size=(3 * H, H)), rng.normal(size=3 * H), rng.normal(size=H)) for _ in range(2)]
    ow, ob_ = [rng.normal(size=(H, H)), rng.normal(size=(O, H))], [rng.normal(size=H), np.zeros(O)]
    obs, carry = rng.normal(size=(N, I)), rng.normal(size=(2, N, H))
    fresh = np.array([0, 1, 0, 0], bool)
    out, new = orec.recurrent_network(obs, carry, fresh, proj, cells, ow, ob_)
    # by hand: layer by layer with the fresh env's carry zeroed
    c0 = carry.copy(); c0[:, 1] = 0.0
    x0 = obs @ proj[0].T + proj[1]
    h0 = orec.gru_cell(x0, c0[0], *cells[0]); h1 = orec.gru_cell(h0, c0[1], *cells[1])
    np.testing.assert_allclose(new, np.stack([h0, h1]))
    np.testing.assert_allclose(out, orec.gelu(h1 @ ow[0].T + ob_[0]) @ ow[1].T)


def test_lstm_cell_matches_the_library_cell():
    rng = np.random.default_rng(2)
    N, I, H = 5, 7, 6
    wi, wh, b = rng.normal(size=(4 * H, I)), rng.normal(size=(4 * H, H)), rng.normal(size=4 * H)
    x, h, c = rng.normal(size=(N, I)), rng.normal(size=(N, H)), rng.normal(size=(N, H))
    cell = torch.nn.LSTMCell(I, H).double()
    with torch.no_grad():
        cell.weight_ih.copy_(torch.from_numpy(wi)); cell.weight_hh.copy_(torch.from_numpy(wh))
        cell.bias_ih.copy_(torch.from_numpy(b)); cell.bias_hh.zero_()
        hw, cw = cell(torch.from_numpy(x), (torch.from_numpy(h), torch.from_numpy(c)))
    hn, cn = orec.lstm_cell(x, h, c, wi, wh, b)
    np.testing.assert_allclose(hn, hw.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(cn, cw.numpy(), rtol=1e-12, atol=1e-12)
    # forget gate saturated open, input gate shut: the cell state is kept and h = sigmoid(o) tanh(c)
    big = np.zeros(4 * H); big[:H] = -50.0; big[H:2 * H] = 50.0
    hn, cn = orec.lstm_cell(x, h, c, 0 * wi, 0 * wh, big)
    np.testing.assert_allclose(cn, c, atol=1e-12)
    np.testing.assert_allclose(hn, 0.5 * np.tanh(c), atol=1e-12)


def _small_net(rng, I=5, H=6, O=3, depth=2):
    proj = (rng.normal(size=(H, I)) * 0.5, rng.normal(size=H) * 0.1)
    cells = [(rng.normal(size=(3 * H, H)) * 0.5, rng.normal(size=(3 * H, H)) * 0.5, rng.normal(size=3 * H) * 0.1,
              rng.normal(size=H) * 0.1) for _ in range(depth)]
    ow, ob_ = [rng.normal(size=(H, H)) * 0.5, rng.normal(size=(O, H)) * 0.5], [rng.normal(size=H) * 0.1, rng.normal(size=O) * 0.1]
    return proj, cells, ow, ob_


def test_sequence_gradients_against_central_differences():
    """The backward pass through time: forward value equal to the step-by-step numpy network, gradient entries equal to
    central differences of that network, no gradient across an episode boundary."""
    rng = np.random.default_rng(2)
    T, N, I, H, O = 6, 3, 5, 6, 3
    proj, cells, ow, ob_ = _small_net(rng, I, H, O)
    obs, carry0 = rng.normal(size=(T, N, I)), rng.normal(size=(2, N, H))
    fresh = np.zeros((T, N), bool); fresh[3, 1] = True; fresh[0, 2] = True
    d_out = rng.normal(size=(T, N, O))
    out, g = orec.recurrent_sequence_gradients(obs, carry0, fresh, proj, cells, ow, ob_, d_out)
    np.testing.assert_allclose(out, orec.recurrent_sequence(obs, carry0, fresh, proj, cells, ow, ob_), rtol=1e-12, atol=1e-12)

    def loss(proj_, cells_, ow_, ob2_):
        return float((orec.recurrent_sequence(obs, carry0, fresh, proj_, cells_, ow_, ob2_) * d_out).sum())

    eps = 1e-6
    def fd(get, idx):  # central difference on one entry of one parameter array
        vals = []
        for s in (+eps, -eps):
            p2, c2, w2, b2 = (proj[0].copy(), proj[1].copy()), [tuple(a.copy() for a in c) for c in cells], [w.copy() for w in ow], [b.copy() for b in ob_]
            get(p2, c2, w2, b2)[idx] += s
            vals.append(loss(p2, c2, w2, b2))
        return (vals[0] - vals[1]) / (2 * eps)

    checks = [(lambda p, c, w, b: p[0], (2, 3), g["input_proj"][0]), (lambda p, c, w, b: p[1], (4,), g["input_proj"][1]),
              (lambda p, c, w, b: c[0][0], (7, 2), g["cells"][0][0]), (lambda p, c, w, b: c[0][1], (13, 5), g["cells"][0][1]),
              (lambda p, c, w, b: c[1][1], (1, 1), g["cells"][1][1]), (lambda p, c, w, b: c[1][2], (9,), g["cells"][1][2]),
              (lambda p, c, w, b: c[0][3], (2,), g["cells"][0][3]), (lambda p, c, w, b: c[1][3], (5,), g["cells"][1][3]),
              (lambda p, c, w, b: w[0], (3, 3), g["out"][0][0]), (lambda p, c, w, b: b[1], (1,), g["out"][1][1])]
    for get, idx, grad in checks:
        assert grad[idx] == pytest.approx(fd(get, idx), rel=1e-6, abs=1e-8)
    # an env that starts an episode at step 3 takes nothing from its earlier carry: outputs from step 3 on do not
    # depend on carry0 of that env, and with d_out zero before step 3 the first-step observation gets no say either
    c2 = carry0.copy(); c2[:, 1] += 1.0
    o1 = orec.recurrent_sequence(obs, carry0, fresh, proj, cells, ow, ob_)
    o2 = orec.recurrent_sequence(obs, c2, fresh, proj, cells, ow, ob_)
    assert np.array_equal(o2[3:, 1], o1[3:, 1]) and not np.allclose(o2[:3, 1], o1[:3, 1])


def test_lstm_sequence_gradients_against_central_differences():
    rng = np.random.default_rng(3)
    T, N, I, H, O = 5, 3, 4, 6, 2
    proj = (rng.normal(size=(H, I)) * 0.5, rng.normal(size=H) * 0.1)
    cells = [(rng.normal(size=(4 * H, H)) * 0.5, rng.normal(size=(4 * H, H)) * 0.5, rng.normal(size=4 * H) * 0.1) for _ in range(2)]
    ow, ob_ = [rng.normal(size=(H, H)) * 0.5, rng.normal(size=(O, H)) * 0.5], [rng.normal(size=H) * 0.1, rng.normal(size=O) * 0.1]
    obs, carry0 = rng.normal(size=(T, N, I)), rng.normal(size=(2, 2, N, H))
    fresh = np.zeros((T, N), bool); fresh[2, 1] = True
    d_out = rng.normal(size=(T, N, O))
    out, g = orec.recurrent_sequence_gradients(obs, carry0, fresh, proj, cells, ow, ob_, d_out)
    np.testing.assert_allclose(out, orec.recurrent_sequence(obs, carry0, fresh, proj, cells, ow, ob_), rtol=1e-12, atol=1e-12)
    eps = 1e-6
    for layer, k, idx in [(0, 0, (3, 2)), (0, 1, (20, 4)), (1, 1, (7, 0)), (1, 2, (13,)), (0, 2, (1,)), (1, 0, (23, 5))]:
        vals = []
        for s in (+eps, -eps):
            c2 = [tuple(a.copy() for a in c) for c in cells]
            c2[layer][k][idx] += s
            vals.append(float((orec.recurrent_sequence(obs, carry0, fresh, proj, c2, ow, ob_) * d_out).sum()))
        assert g["cells"][layer][k][idx] == pytest.approx((vals[0] - vals[1]) / (2 * eps), rel=1e-6, abs=1e-8)
