"""Pins the recurrent-network oracle (CPU): the GRU cell against torch's library cell and limits, GELU against torch."""
import numpy as np
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
