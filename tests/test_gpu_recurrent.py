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


@pytest.mark.parametrize("dtype,tol,act", [("f32", 2e-4, "elu"), ("bf16", 6e-2, "elu"), ("f32", 2e-4, "gelu")])
def test_backward_through_time_matches_the_oracle(dtype, tol, act):
    """Gradients of a GRU actor over a trajectory (input projection, two GRU layers, ELU or GELU output network) with episode
    starts inside it, against torch float64 reverse-mode differentiation of the oracle network; then one optimiser step.
    Tolerances are relative to the largest entry of each gradient array: fp32 accumulation only for f32; for bf16 the
    activations and the gradients between layers are rounded to bf16 at every one of the T steps."""
    from ksim_amd import _lib_terms as T
    from ksim_amd.mlp import MLP
    from ksim_amd.recurrent import GRUCell, RecurrentNetwork

    rng = np.random.default_rng(41)
    Tn, N, I, H, O = 12, 96, 37, 64, 10
    proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
    cells = [(rng.normal(size=(3 * H, H)) / np.sqrt(H), rng.normal(size=(3 * H, H)) / np.sqrt(H), rng.normal(size=3 * H) * 0.1,
              rng.normal(size=H) * 0.1) for _ in range(2)]
    ow = [rng.normal(size=(H, H)) / np.sqrt(H), rng.normal(size=(O, H)) / np.sqrt(H)]
    ob = [rng.normal(size=H) * 0.1, rng.normal(size=O) * 0.1]
    obs, carry0 = rng.normal(size=(Tn, N, I)), rng.normal(size=(2, N, H)) * 0.5
    fresh = rng.random((Tn, N)) < 0.08
    d_out = rng.normal(size=(Tn, N, O))
    if dtype == "bf16":  # both sides start from bf16-representable weights
        rb = lambda a: torch.tensor(a, dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy()  # noqa: E731
        proj = (rb(proj[0]), proj[1]); ow = [rb(w) for w in ow]
        cells = [(rb(c[0]), rb(c[1]), c[2], c[3]) for c in cells]
    want_out, want = orec.recurrent_sequence_gradients(obs, carry0, fresh, proj, cells, ow, ob, d_out, act=act)

    net = RecurrentNetwork(proj, [GRUCell(*c, dtype=dtype) for c in cells], MLP(ow, ob, activation=act, dtype=dtype), dtype=dtype)
    net.train_init()
    out = net.train_forward(t32(obs), t32(carry0), torch.tensor(fresh, dtype=torch.uint8, device=DEV))
    scale = np.abs(want_out).max()
    assert np.abs(out.cpu().numpy() - want_out).max() <= (1e-4 if dtype == "f32" else 3e-2) * scale
    net.backward(t32(d_out))
    got = {"input_proj.W": net.input_proj.parameters(True)[0][0], "input_proj.b": net.input_proj.parameters(True)[0][1]}
    ref = {"input_proj.W": want["input_proj"][0], "input_proj.b": want["input_proj"][1]}
    for i, c in enumerate(net.cells):
        g = c.parameters(True)
        for k, j in (("weight_ih", 0), ("weight_hh", 1), ("bias", 2), ("bias_n", 3)):
            got[f"cell{i}.{k}"], ref[f"cell{i}.{k}"] = g[k], want["cells"][i][j]
    for l, (w, b) in enumerate(net.output_proj.parameters(True)):
        got[f"out{l}.W"], ref[f"out{l}.W"], got[f"out{l}.b"], ref[f"out{l}.b"] = w, want["out"][l][0], b, want["out"][l][1]
    for k in ref:
        err = np.abs(got[k].cpu().numpy() - ref[k]).max() / np.abs(ref[k]).max()
        assert err <= tol, f"{k}: {err:.2e} > {tol}"
    # the hidden projection has no reset / update bias of its own: those entries stay out of the update
    before = [c.parameters() for c in net.cells]
    acc = torch.zeros(1, dtype=torch.float64, device=DEV)
    net.grad_sqnorm(acc)
    total = sum(float((np.asarray(v) ** 2).sum()) for v in ref.values())
    assert acc.item() == pytest.approx(total, rel=2e-3 if dtype == "f32" else 0.15)
    params = T.KsAdamParams(1e-3, 0.9, 0.999, 1e-8, 0.0, 0.0, 1)
    net.adam_step(params, None)
    for c, b0 in zip(net.cells, before):
        p = c.parameters()
        (_, bh), = c.proj_h.parameters()
        assert torch.equal(bh[:2 * H], torch.zeros(2 * H, device=DEV))
        # first Adam step: every parameter with a gradient moves by lr against the gradient's sign
        moved = (p["bias_n"] - b0["bias_n"]).cpu().numpy()
        gn = c.parameters(True)["bias_n"].cpu().numpy()
        big = np.abs(gn) > 1e-4
        np.testing.assert_allclose(moved[big], -1e-3 * np.sign(gn[big]), rtol=1e-3)
    # the forward pass of the rollout sees the updated b_n also for envs that start an episode
    h1 = net.cells[0](t32(rng.normal(size=(N, H))), t32(np.zeros((N, H))), torch.ones(N, dtype=torch.uint8, device=DEV))
    assert torch.isfinite(h1).all()


@pytest.mark.parametrize("dtype,tol,H,N", [("f32", 2e-4, 64, 80), ("bf16", 6e-2, 64, 80), ("f32", 2e-4, 128, 77), ("f32", 2e-4, 128, 16)])
def test_lstm_backward_through_time_matches_the_oracle(dtype, tol, H, N):
    """The same for an LSTM stack (the K-Bot example's actor shape: projection, LSTM layers, linear output).  Hidden size
    128 in fp32 is the K-Bot cell itself and runs through the one-launch-per-trajectory kernels (`ks_lstm_sequence_*`),
    with a row count that does not fill the last 16-row workgroup."""
    from ksim_amd import _lib_terms as T
    from ksim_amd.mlp import MLP
    from ksim_amd.recurrent import LSTMCell, RecurrentNetwork

    rng = np.random.default_rng(43)
    Tn, I, O = 10, 29, 12
    proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
    cells = [(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=4 * H) * 0.1)
             for _ in range(2)]
    ow, ob = [rng.normal(size=(O, H)) / np.sqrt(H)], [rng.normal(size=O) * 0.1]
    obs, carry0 = rng.normal(size=(Tn, N, I)), rng.normal(size=(2, 2, N, H)) * 0.5
    fresh = rng.random((Tn, N)) < 0.08
    d_out = rng.normal(size=(Tn, N, O))
    if dtype == "bf16":
        proj = (_bf16(proj[0]), proj[1]); ow = [_bf16(w) for w in ow]
        cells = [(_bf16(c[0]), _bf16(c[1]), c[2]) for c in cells]
    want_out, want = orec.recurrent_sequence_gradients(obs, carry0, fresh, proj, cells, ow, ob, d_out)
    net = RecurrentNetwork(proj, [LSTMCell(*c, dtype=dtype) for c in cells], MLP(ow, ob, activation="none", dtype=dtype), dtype=dtype)
    net.train_init()
    assert all(c.sequence_supported == (dtype == "f32" and H == 128) for c in net.cells)
    out = net.train_forward(t32(obs), t32(carry0), torch.tensor(fresh, dtype=torch.uint8, device=DEV))
    assert np.abs(out.cpu().numpy() - want_out).max() <= (1e-4 if dtype == "f32" else 3e-2) * np.abs(want_out).max()
    net.backward(t32(d_out))
    got = {"input_proj.W": net.input_proj.parameters(True)[0][0], "input_proj.b": net.input_proj.parameters(True)[0][1],
           "out.W": net.output_proj.parameters(True)[0][0], "out.b": net.output_proj.parameters(True)[0][1]}
    ref = {"input_proj.W": want["input_proj"][0], "input_proj.b": want["input_proj"][1], "out.W": want["out"][0][0], "out.b": want["out"][0][1]}
    for i, c in enumerate(net.cells):
        g = c.parameters(True)
        for k, j in (("weight_ih", 0), ("weight_hh", 1), ("bias", 2)):
            got[f"cell{i}.{k}"], ref[f"cell{i}.{k}"] = g[k], want["cells"][i][j]
    for k in ref:
        err = np.abs(got[k].cpu().numpy() - ref[k]).max() / np.abs(ref[k]).max()
        assert err <= tol, f"{k}: {err:.2e} > {tol}"
    net.adam_step(T.KsAdamParams(1e-3, 0.9, 0.999, 1e-8, 0.0, 0.0, 1), None)
    for c in net.cells:  # the hidden projection carries no bias of its own, before and after the update
        (_, bh), = c.proj_h.parameters()
        assert torch.equal(bh, torch.zeros(4 * H, device=DEV))


def test_lstm_sequence_kernels_agree_with_the_step_by_step_entry_points():
    """One launch over the trajectory against T calls of the per-step entry points on the same cell (which, for such a cell,
    are that launch with T = 1): states, saved activations and gate gradients bit for bit; the carry of the hidden-state
    gradient, which the per-step path forms with a separate product, to rounding.  In place with T = 1, as the rollout
    advances its carry."""
    from ksim_amd import _lib
    from ksim_amd.recurrent import LSTMCell

    rng = np.random.default_rng(47)
    Tn, M, H = 7, 45, 128
    cell = LSTMCell(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=4 * H) * 0.1, dtype="f32")
    cell.train_init()
    assert cell.sequence_supported
    x, h0, c0 = t32(rng.normal(size=(Tn, M, H))), t32(rng.normal(size=(M, H)) * 0.5), t32(rng.normal(size=(M, H)) * 0.5)
    fresh = torch.tensor(rng.random((Tn, M)) < 0.1, dtype=torch.uint8, device=DEV)
    z = lambda *s: torch.zeros(*s, device=DEV)  # noqa: E731
    hs, cs, sv = z(Tn, M, H), z(Tn, M, H), z(Tn, M, 7 * H)
    cell.sequence_forward(x, h0, c0, fresh, hs, cs, sv)
    hs1, cs1, sv1 = z(Tn, M, H), z(Tn, M, H), z(Tn, M, 7 * H)
    for t in range(Tn):
        cell.train_forward(x[t], h0 if t == 0 else hs1[t - 1], c0 if t == 0 else cs1[t - 1], fresh[t], hs1[t], cs1[t], sv1[t])
    assert torch.equal(hs, hs1) and torch.equal(cs, cs1) and torch.equal(sv, sv1)
    h, c = h0.clone(), c0.clone()  # the rollout's step: the carry advanced in place
    for t in range(Tn):
        cell(x[t], h, c, fresh[t], out=(h, c))
    assert torch.equal(h, hs[-1]) and torch.equal(c, cs[-1])
    dH = t32(rng.normal(size=(Tn, M, H)))
    d_g = z(Tn, M, 4 * H)
    cell.sequence_backward(dH, sv, fresh, d_g)
    d_g1, carry, ccarry = z(Tn, M, 4 * H), z(2, M, H), z(2, M, H)
    dH1 = dH.clone()
    for t in range(Tn - 1, -1, -1):
        dH1[t] += carry[t & 1]
        cell.backward_step(dH1[t], ccarry[t & 1], sv[t], fresh[t], d_g1[t], carry[(t + 1) & 1], ccarry[(t + 1) & 1])
    err = (d_g - d_g1).abs().max().item() / d_g1.abs().max().item()
    assert err < 1e-5, err
    assert torch.equal(d_g[-1], d_g1[-1])  # the last step has no carried gradient yet: the same arithmetic
    lib = _lib.load()  # shapes the kernels do not cover are refused, not approximated
    small = LSTMCell(rng.normal(size=(4 * 64, 64)), rng.normal(size=(4 * 64, 64)), None, dtype="f32")
    assert not small.sequence_supported
    assert lib.ks_lstm_sequence_forward(small._handle, _lib.current_stream(), 1, 4, _lib.ptr(z(4, 256)), _lib.ptr(z(4, 64)), _lib.ptr(z(4, 64)),
                                        None, _lib.ptr(z(4, 64)), None, None) != 0
    assert lib.ks_lstm_sequence_forward(cell._handle, _lib.current_stream(), 2, M, _lib.ptr(z(2, M, 4 * H)), _lib.ptr(h0), _lib.ptr(c0),
                                        None, _lib.ptr(h0), None, None) != 0  # aliasing is for T = 1 only


def test_lstm_sequence_forward_over_many_rows_equals_the_same_rows_in_small_calls():
    """A short call over thousands of rows lets each workgroup take several 4-row sets in turn (the rollout's single step over all
    envs): the rows must come out exactly as when they are given in calls small enough for one set per workgroup, including a
    last set that is not full, in place as the rollout calls it, and with the episode starts honoured."""
    from ksim_amd.recurrent import LSTMCell

    rng = np.random.default_rng(53)
    M, H = 2102, 128
    cell = LSTMCell(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=4 * H) * 0.1, dtype="f32")
    cell.train_init()
    z = lambda *s: torch.zeros(*s, device=DEV)  # noqa: E731
    for Tn in (1, 3):
        x, h0, c0 = t32(rng.normal(size=(Tn, M, H))), t32(rng.normal(size=(M, H)) * 0.5), t32(rng.normal(size=(M, H)) * 0.5)
        fresh = torch.tensor(rng.random((Tn, M)) < 0.1, dtype=torch.uint8, device=DEV)
        hs, cs, sv = z(Tn, M, H), z(Tn, M, H), z(Tn, M, 7 * H)
        cell.sequence_forward(x, h0, c0, fresh, hs, cs, sv)
        for lo in range(0, M, 700):
            hi = min(M, lo + 700)
            n = hi - lo
            hs1, cs1, sv1 = z(Tn, n, H), z(Tn, n, H), z(Tn, n, 7 * H)
            cell.sequence_forward(x[:, lo:hi].contiguous(), h0[lo:hi].contiguous(), c0[lo:hi].contiguous(), fresh[:, lo:hi].contiguous(),
                                  hs1, cs1, sv1)
            assert torch.equal(hs[:, lo:hi], hs1) and torch.equal(cs[:, lo:hi], cs1) and torch.equal(sv[:, lo:hi], sv1), (Tn, lo)
    h, c = h0.clone(), c0.clone()  # one step in place over all rows, as the rollout advances its carry
    cell(x[0], h, c, fresh[0], out=(h, c))
    hs1, cs1, sv1 = z(1, M, H), z(1, M, H), z(1, M, 7 * H)
    cell.sequence_forward(x[:1].contiguous(), h0, c0, fresh[:1].contiguous(), hs1, cs1, sv1)
    assert torch.equal(h, hs1[0]) and torch.equal(c, cs1[0])
