"""GRU cell and recurrent policy networks on the GPU against the float64 oracle."""
import numpy as np
import pytest
import torch

from oracle import recurrent as orec

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t32(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=DEV).contiguous()


def _bf16(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32).bfloat16().double().numpy()


def _cell_params(rng, I, H):
    s = 1.0 / np.sqrt(H)
    return (rng.uniform(-s, s, (3 * H, I)), rng.uniform(-s, s, (3 * H, H)), rng.uniform(-s, s, 3 * H), rng.uniform(-s, s, H))


@pytest.mark.parametrize("N,I,H", [(33, 20, 24), (512, 128, 128), (8192, 256, 256)])
def test_gru_cell_f32_and_bf16(N, I, H):
    from ksim_amd.recurrent import GRUCell

    rng = np.random.default_rng(N)
    wi, wh, b, bn = _cell_params(rng, I, H)
    x, h = rng.normal(size=(N, I)), rng.normal(size=(N, H)) * 0.5
    fresh = rng.random(N) < 0.2
    h_eff = np.where(fresh[:, None], 0.0, h)
    want = orec.gru_cell(x, h_eff, wi, wh, b, bn)
    mask = torch.from_numpy(fresh.astype(np.uint8)).to(DEV)
    got = GRUCell(wi, wh, b, bn, dtype="f32")(t32(x), t32(h), mask).cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)  # fp32 projections vs float64
    # bf16 projections: operands of the two matrix products rounded to bf16, everything else fp32
    gi = _bf16(x) @ _bf16(wi).T + b
    gh = _bf16(h) @ _bf16(wh).T
    gh = np.where(fresh[:, None], 0.0, gh)
    r = orec.sigmoid(gi[:, :H] + gh[:, :H]); z = orec.sigmoid(gi[:, H:2 * H] + gh[:, H:2 * H])
    n = np.tanh(gi[:, 2 * H:] + r * (gh[:, 2 * H:] + bn))
    want16 = n + z * (h_eff - n)
    cell = GRUCell(wi, wh, b, bn, dtype="bf16")
    hin = t32(h)
    got16 = cell(t32(x), hin, mask, out=hin).cpu().numpy()  # in place on the carry
    np.testing.assert_allclose(got16, want16, rtol=2e-4, atol=2e-4)
    assert np.abs(got16 - want).max() < 3e-2  # and close to the unrounded cell
    # no bias, no mask
    got0 = GRUCell(wi, wh, dtype="f32")(t32(x), t32(h)).cpu().numpy()
    np.testing.assert_allclose(got0, orec.gru_cell(x, h, wi, wh), rtol=2e-5, atol=2e-5)


def test_recurrent_network_over_an_episode_with_restarts():
    """Input projection, two GRU layers and a GELU output MLP stepped ten times; some envs restart along the way."""
    from ksim_amd.mlp import MLP
    from ksim_amd.recurrent import GRUCell, RecurrentNetwork

    rng = np.random.default_rng(5)
    N, I, H, O, depth = 96, 43, 64, 60, 2
    proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
    cells = [_cell_params(rng, H, H) for _ in range(depth)]
    ow = [rng.normal(size=(H, H)) / np.sqrt(H), rng.normal(size=(O, H)) / np.sqrt(H)]
    ob_ = [rng.normal(size=H) * 0.1, np.zeros(O)]  # use_final_bias=False (walking.py:98-106)
    net = RecurrentNetwork(proj, [GRUCell(*c, dtype="f32") for c in cells], MLP(ow, ob_, activation="gelu", dtype="f32"), dtype="f32")
    carry = net.initial_carry(N, DEV)
    want_carry = np.zeros((depth, N, H))
    for k in range(10):
        obs = rng.normal(size=(N, I))
        fresh = rng.random(N) < (0.0 if k == 0 else 0.15)
        out = net(t32(obs), carry, torch.from_numpy(fresh.astype(np.uint8)).to(DEV))
        want, want_carry = orec.recurrent_network(obs, want_carry, fresh, proj, cells, ow, ob_)
        np.testing.assert_allclose(out.cpu().numpy(), want, rtol=1e-4, atol=1e-4)
        np.testing.assert_allclose(carry.cpu().numpy(), want_carry, rtol=1e-4, atol=1e-4)
    with pytest.raises(Exception, match="carry"):
        net(t32(obs), carry[:1])


def test_gelu_mlp_bf16():
    from ksim_amd.mlp import MLP

    rng = np.random.default_rng(6)
    dims = (64, 256, 256, 40)
    ws = [rng.normal(size=(o, i)) / np.sqrt(i) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.normal(size=o) * 0.1 for o in dims[1:]]
    for M in (100, 40000):  # the per-layer and the whole-network kernels
        x = rng.normal(size=(M, dims[0]))
        got = MLP(ws, bs, activation="gelu", dtype="bf16")(t32(x)).cpu().numpy()
        h = _bf16(x)
        for i, (w, b) in enumerate(zip(ws, bs)):
            h = h @ _bf16(w).T + b
            if i + 1 < len(ws):
                h = _bf16(orec.gelu(h))
        assert np.abs(got - h).max() < 6e-3 * max(1.0, np.abs(h).max())
        got32 = MLP(ws, bs, activation="gelu", dtype="f32")(t32(x)).cpu().numpy()
        np.testing.assert_allclose(got32, orec.mlp(x, ws, bs, orec.gelu), rtol=2e-5, atol=2e-5)
    m = MLP(ws, bs, activation="gelu", dtype="f32")
    with pytest.raises(Exception, match="GELU"):
        m.train_init()


@pytest.mark.parametrize("N,I,H", [(40, 12, 16), (4096, 128, 128)])
def test_lstm_cell_and_network(N, I, H):
    from ksim_amd.mlp import MLP
    from ksim_amd.recurrent import LSTMCell, RecurrentNetwork

    rng = np.random.default_rng(N + 1)
    s = 1.0 / np.sqrt(H)
    def params(i):
        return (rng.uniform(-s, s, (4 * H, i)), rng.uniform(-s, s, (4 * H, H)), rng.uniform(-s, s, 4 * H))
    wi, wh, b = params(I)
    x, h, c = rng.normal(size=(N, I)), rng.normal(size=(N, H)) * 0.5, rng.normal(size=(N, H))
    fresh = rng.random(N) < 0.25
    keep = ~fresh[:, None]
    hw, cw = orec.lstm_cell(x, h * keep, c * keep, wi, wh, b)
    mask = torch.from_numpy(fresh.astype(np.uint8)).to(DEV)
    hg, cg = LSTMCell(wi, wh, b, dtype="f32")(t32(x), t32(h), t32(c), mask)
    np.testing.assert_allclose(hg.cpu().numpy(), hw, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(cg.cpu().numpy(), cw, rtol=2e-5, atol=2e-5)
    hg, cg = LSTMCell(wi, wh, b, dtype="bf16")(t32(x), t32(h), t32(c), mask)
    assert np.abs(hg.cpu().numpy() - hw).max() < 3e-2 and np.abs(cg.cpu().numpy() - cw).max() < 5e-2
    # the K-Bot actor's shape: projection, two LSTM layers, ELU output MLP; carry (depth, 2, N, H) advanced in place
    proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
    cells = [params(H) for _ in range(2)]
    ow, ob_ = [rng.normal(size=(H, H)) / np.sqrt(H), rng.normal(size=(40, H)) / np.sqrt(H)], [rng.normal(size=H) * 0.1, np.zeros(40)]
    net = RecurrentNetwork(proj, [LSTMCell(*p, dtype="f32") for p in cells], MLP(ow, ob_, activation="elu", dtype="f32"), dtype="f32")
    carry = net.initial_carry(N, DEV)
    assert tuple(carry.shape) == (2, 2, N, H)
    want_carry = np.zeros((2, 2, N, H))
    elu = lambda v: np.where(v > 0, v, np.expm1(v))  # noqa: E731
    for k in range(6):
        obs = rng.normal(size=(N, I))
        fr = rng.random(N) < (0.0 if k == 0 else 0.2)
        out = net(t32(obs), carry, torch.from_numpy(fr.astype(np.uint8)).to(DEV))
        want, want_carry = orec.recurrent_network(obs, want_carry, fr, proj, cells, ow, ob_, act=elu)
        np.testing.assert_allclose(out.cpu().numpy(), want, rtol=2e-4, atol=2e-4)
        np.testing.assert_allclose(carry.cpu().numpy(), want_carry, rtol=2e-4, atol=2e-4)
