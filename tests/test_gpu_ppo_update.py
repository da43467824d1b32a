"""Policy update (gradients through the Gaussian head, the PPO loss and the MLPs; optimiser chain; minibatch loop)
through the C ABI against the float64 autograd oracle."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import ppo_update as ou

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CFG = dict(gamma=0.99, lam=0.95, normalize_advantages=True, monte_carlo_returns=False, clip_param=0.2, value_loss_coef=0.5,
           entropy_coef=0.008, kl_coef=1e-3, log_clip_value=5.0, use_clipped_value_loss=True, learning_rate=3e-4,
           adam_b1=0.9, adam_b2=0.999, adam_eps=1e-8, adam_weight_decay=0.01, grad_clip=2.0, batch_size=8, num_passes=2)


def t32(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=DEV).contiguous()


def rel(got, want):
    want = np.asarray(want, np.float64)
    return np.abs(np.asarray(got, np.float64) - want).max() / max(np.abs(want).max(), 1e-30)


@pytest.mark.parametrize("dims,dtype,act,M,tol", [
    ((71, 256, 256, 21), "f32", "elu", 300, 2e-4),     # fp32 path: accumulation-order error only
    ((68, 512, 512, 512, 20), "bf16", "elu", 1000, 3e-2),  # bf16 operands, fp32 accumulate
    ((33, 130, 2), "f32", "tanh", 77, 2e-4), ((40, 64, 64, 1), "f32", "relu", 129, 2e-4),
    # GELU (the walking example's output networks): the pre-activations are kept for the derivative
    ((64, 128, 128, 36), "f32", "gelu", 257, 2e-4), ((256, 256, 256, 256, 60), "bf16", "gelu", 1000, 3e-2),
])
def test_mlp_backward_matches_autograd(dims, dtype, act, M, tol):
    from ksim_amd.mlp import MLP

    rng = np.random.default_rng(sum(dims))
    ws = [rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.normal(scale=0.1, size=o).astype(np.float32) for o in dims[1:]]
    x = rng.normal(size=(M, dims[0])).astype(np.float32)
    dy = rng.normal(size=(M, dims[-1])).astype(np.float32)
    net = MLP(ws, bs, activation=act, dtype=dtype)
    net.train_init()
    xd = t32(x)
    y = net.train_forward(xd)
    net.backward(xd, t32(dy))
    tw = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in ws]
    tb = [torch.tensor(b, dtype=torch.float64, requires_grad=True) for b in bs]
    yo = ou.mlp(torch.tensor(x, dtype=torch.float64), tw, tb, act)
    (yo * torch.tensor(dy, dtype=torch.float64)).sum().backward()
    assert rel(y.cpu().numpy(), yo.detach().numpy()) < (2e-5 if dtype == "f32" else 1e-2)
    for (gw, gb), w, b in zip(net.parameters(gradients=True), tw, tb):
        assert rel(gw.cpu().numpy(), w.grad.numpy()) < tol
        assert rel(gb.cpu().numpy(), b.grad.numpy()) < tol
    for (pw, pb), w, b in zip(net.parameters(), ws, bs):  # master copy is the caller's fp32 parameters, bit for bit
        assert np.array_equal(pw.cpu().numpy(), w) and np.array_equal(pb.cpu().numpy(), b)
    y2 = net(xd)  # the inference path still reads the same weights
    assert rel(y2.cpu().numpy(), yo.detach().numpy()) < (2e-5 if dtype == "f32" else 1e-2)


def test_ppo_loss_gradient_kernel_matches_autograd():
    from ksim_amd import _lib

    lib = _lib.load()
    rng = np.random.default_rng(3)
    M, A = 5000, 20
    mean, ls, act = rng.normal(size=(M, A)), rng.normal(size=A) * 0.2 - 1.0, rng.normal(size=(M, A))
    act = mean + np.exp(ls) * act                        # actions the policy plausibly took
    on_lp = ou.gaussian(torch.tensor(mean + rng.normal(size=(M, A)) * 0.02), torch.tensor(ls), torch.tensor(act))[0].numpy()
    adv, tgt, on_v, v = rng.normal(size=M), rng.normal(size=M), rng.normal(size=M), rng.normal(size=M)
    v = on_v + rng.normal(size=M) * 0.3                  # both sides of the value clip
    tm = torch.tensor(mean, requires_grad=True); tl = torch.tensor(ls, requires_grad=True); tv = torch.tensor(v, requires_grad=True)
    lp, ent = ou.gaussian(tm, tl, torch.tensor(act))
    loss, _ = ou.ppo_loss_torch(torch.tensor(adv), torch.tensor(tgt), torch.tensor(on_lp), torch.tensor(on_v), lp, tv, ent, CFG, 1.3)
    loss.backward()
    p = _lib.KsPpoLossParams(0.2, 0.5, 0.008, 1e-3, 5.0, 1.3, 1)
    d_mean, d_value, d_ls = torch.empty(M, A, device=DEV), torch.empty(M, device=DEV), torch.empty(A, device=DEV)
    ws = torch.empty(256 * A, device=DEV)
    args = [t32(a) for a in (mean, ls, act, on_lp, adv, tgt, on_v, v)]
    _lib.check(lib.ks_ppo_loss_grad(_lib.current_stream(), M, A, ctypes.byref(p), *[_lib.ptr(a) for a in args],
                                    _lib.ptr(d_mean), _lib.ptr(d_value), _lib.ptr(d_ls), _lib.ptr(ws)))
    assert rel(d_mean.cpu().numpy(), tm.grad.numpy()) < 1e-4
    assert rel(d_value.cpu().numpy(), tv.grad.numpy()) < 1e-5
    assert rel(d_ls.cpu().numpy(), tl.grad.numpy()) < 1e-4
    lp_k, ent_k = torch.empty(M, A, device=DEV), torch.empty(M, A, device=DEV)
    _lib.check(lib.ks_gaussian_log_prob(_lib.current_stream(), M, A, _lib.ptr(args[0]), _lib.ptr(args[1]), _lib.ptr(args[2]),
                                        _lib.ptr(lp_k), _lib.ptr(ent_k)))
    np.testing.assert_allclose(lp_k.cpu().numpy(), lp.detach().numpy(), rtol=1e-5, atol=1e-5)   # GAE/returns class tolerance
    np.testing.assert_allclose(ent_k.cpu().numpy(), ent.detach().numpy(), rtol=1e-6, atol=1e-6)


def test_ppo_loss_gradient_for_the_deviation_head_matches_autograd():
    """d loss / d (mean | raw deviation) for a network that emits its own deviations, against float64 autograd of the
    oracle loss; rows with a capped deviation get no deviation gradient."""
    from ksim_amd import _lib, _lib_terms as T

    lib = _lib.load()
    rng = np.random.default_rng(13)
    M, A = 4000, 20
    raw = rng.normal(size=(M, 2 * A))
    raw[:50, A:] = 6.0  # (softplus + 0.01) * 0.5 above the cap of 1.5
    bias = rng.normal(size=A) * 0.1
    hd = dict(min_std=0.01, max_std=1.5, var_scale=0.5)
    tr = torch.tensor(raw, requires_grad=True)
    with torch.no_grad():
        sd = torch.clamp((torch.nn.functional.softplus(tr[:, A:]) + 0.01) * 0.5, max=1.5).numpy()
    act = raw[:, :A] + bias + sd * rng.normal(size=(M, A))
    on_lp = ou.gaussian_head(torch.tensor(raw + rng.normal(size=raw.shape) * 0.02), torch.tensor(act), mean_bias=torch.tensor(bias), **hd)[0].numpy()
    adv, tgt, on_v = rng.normal(size=M), rng.normal(size=M), rng.normal(size=M)
    v = on_v + rng.normal(size=M) * 0.3
    tv = torch.tensor(v, requires_grad=True)
    lp, ent = ou.gaussian_head(tr, torch.tensor(act), mean_bias=torch.tensor(bias), **hd)
    loss, _ = ou.ppo_loss_torch(torch.tensor(adv), torch.tensor(tgt), torch.tensor(on_lp), torch.tensor(on_v), lp, tv, ent, CFG, 1.3)
    loss.backward()
    p = _lib.KsPpoLossParams(0.2, 0.5, 0.008, 1e-3, 5.0, 1.3, 1)
    bias_d = t32(bias)
    head = T.KsGaussianHead(0.01, 1.5, 0.5, 0, _lib.ptr(bias_d).value)
    d_raw, d_value = torch.empty(M, 2 * A, device=DEV), torch.empty(M, device=DEV)
    args = [t32(a) for a in (raw, act, on_lp, adv, tgt, on_v, v)]
    _lib.check(lib.ks_ppo_loss_grad_head(_lib.current_stream(), M, A, ctypes.byref(p), ctypes.byref(head), *[_lib.ptr(a) for a in args],
                                         _lib.ptr(d_raw), _lib.ptr(d_value)))
    g = tr.grad.numpy()
    assert rel(d_raw[:, :A].cpu().numpy(), g[:, :A]) < 1e-4
    assert rel(d_raw[:, A:].cpu().numpy(), g[:, A:]) < 1e-4
    assert rel(d_value.cpu().numpy(), tv.grad.numpy()) < 1e-5
    assert (d_raw[:50, A:] == 0).all() and (g[:50, A:] == 0).all()


def test_adam_chain_kernel_matches_optax_restatement():
    from ksim_amd import _lib, _lib_terms as T

    lib = _lib.load()
    rng = np.random.default_rng(4)
    n = 3000
    p0, g = rng.normal(size=n), rng.normal(size=n) * 0.1
    g[5] = np.nan
    p, m1, m2 = t32(p0), torch.zeros(n, device=DEV), torch.zeros(n, device=DEV)
    po, o1, o2 = [p0.astype(np.float32).astype(np.float64)], [np.zeros(n)], [np.zeros(n)]
    for step in (1, 2, 3):
        gs = g * step
        sq = torch.zeros(1, dtype=torch.float64, device=DEV)
        gd = t32(gs)
        _lib.check(lib.ks_grad_sqnorm(_lib.current_stream(), n, _lib.ptr(gd), _lib.ptr(sq)))
        ap = T.KsAdamParams(3e-4, 0.9, 0.999, 1e-8, 0.01, 2.0, step)
        _lib.check(lib.ks_adam_step(_lib.current_stream(), n, _lib.ptr(p), _lib.ptr(gd), _lib.ptr(m1), _lib.ptr(m2),
                                    ctypes.byref(ap), _lib.ptr(sq)))
        po, o1, o2, norm = ou.optax_chain_step(po, [gs.astype(np.float32).astype(np.float64)], o1, o2, step, CFG)
        assert abs(float(sq.sqrt().item()) - norm) < 1e-5 * norm
    np.testing.assert_allclose(p.cpu().numpy(), po[0], rtol=0, atol=2e-6)
    np.testing.assert_allclose(m1.cpu().numpy(), o1[0], rtol=1e-5, atol=1e-8)


@pytest.mark.parametrize("dims,act,M", [((68, 512, 512, 512, 20), "elu", 33000), ((40, 128, 256, 1), "tanh", 32768),
                                        ((68, 512, 512, 20), "relu", 40001)])
def test_whole_network_backward_pass_at_large_batches(dims, act, M):
    """Batches of 32768 rows and more of a bf16 network go through the whole-network backward kernel (hidden-layer gradients in
    one launch, activations kept in accumulator order and transposed).  Its gradients against float64 reverse-mode
    differentiation, and against the layer-by-layer pass, which the same call takes when the input gradient is asked for
    (it rebuilds the row-major activations from the transposed copies); batch sizes that are not multiples of the tile."""
    from ksim_amd.mlp import MLP

    rng = np.random.default_rng(sum(dims) + M)
    ws = [rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.normal(scale=0.1, size=o).astype(np.float32) for o in dims[1:]]
    x = rng.normal(size=(M, dims[0])).astype(np.float32)
    dy = (rng.normal(size=(M, dims[-1])) / M).astype(np.float32)
    net = MLP(ws, bs, activation=act, dtype="bf16")
    net.train_init()
    xd, dyd = t32(x), t32(dy)
    y = net.train_forward(xd)
    net.backward(xd, dyd)
    chain = [(w.clone(), b.clone()) for w, b in net.parameters(gradients=True)]
    tw = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in ws]
    tb = [torch.tensor(b, dtype=torch.float64, requires_grad=True) for b in bs]
    yo = ou.mlp(torch.tensor(x, dtype=torch.float64), tw, tb, act)
    (yo * torch.tensor(dy, dtype=torch.float64)).sum().backward()
    assert rel(y.cpu().numpy(), yo.detach().numpy()) < 1e-2
    tol = 1e-1 if act == "relu" else 3e-2  # a bf16-rounded pre-activation next to zero switches the step of a ReLU's derivative
    for (gw, gb), w, b in zip(chain, tw, tb):
        assert rel(gw.cpu().numpy(), w.grad.numpy()) < tol
        assert rel(gb.cpu().numpy(), b.grad.numpy()) < tol
    # the layer-by-layer pass on the same stored activations
    y2 = net.train_forward(xd)
    assert torch.equal(y, y2)
    dx = torch.zeros_like(xd)
    net.backward_dx(xd, dyd, dx)
    for (gw, gb), (cw, cb) in zip(net.parameters(gradients=True), chain):
        assert rel(gw.cpu().numpy(), cw.cpu().numpy().astype(np.float64)) < 1e-2
        assert rel(gb.cpu().numpy(), cb.cpu().numpy().astype(np.float64)) < 1e-2
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    (ou.mlp(tx, [w.detach() for w in tw], [b.detach() for b in tb], act) * torch.tensor(dy, dtype=torch.float64)).sum().backward()
    if act != "relu":  # a single row's input gradient has no sum over the batch to average a switched step out
        assert rel(dx.cpu().numpy(), tx.grad.numpy()) < tol


@pytest.mark.parametrize("dims,dtype", [((68, 512, 512, 20), "bf16"), ((71, 256, 21), "f32"), ((30, 64, 1), "bf16")])
def test_optimiser_step_refreshes_every_working_copy(dims, dtype):
    """After an optimiser step both forward paths (the whole-network kernel with its fragment-ordered weights, the training
    forward over the per-layer copies) and the input gradient (the transposed copies) are those of a network built afresh
    from the updated master parameters, bit for bit; widths that are not multiples of the kernels' tiles included."""
    from ksim_amd import _lib_terms as T
    from ksim_amd.mlp import MLP, random_mlp

    rng = np.random.default_rng(6)
    net, _, _ = random_mlp(dims, 3, dtype=dtype)
    net.train_init()
    M = 300
    x, dy = t32(rng.normal(size=(M, dims[0]))), t32(rng.normal(size=(M, dims[-1])))
    for step in (1, 2):
        net.train_forward(x)
        net.backward(x, dy)
        net.adam_step(T.KsAdamParams(1e-2, 0.9, 0.999, 1e-8, 0.01, 0.0, step), None)
    fresh = MLP([w for w, _ in net.parameters()], [b for _, b in net.parameters()], dtype=dtype)
    fresh.train_init()
    assert all((b != 0).any() for _, b in net.parameters())  # the biases moved too
    assert torch.equal(net(x), fresh(x))
    assert torch.equal(net.train_forward(x), fresh.train_forward(x))
    dx_a, dx_b = torch.zeros_like(x), torch.zeros_like(x)
    net.backward_dx(x, dy, dx_a, weight_gradients=False)
    fresh.backward_dx(x, dy, dx_b, weight_gradients=False)
    assert torch.equal(dx_a, dx_b)


def _setup(seed, Tn, N, od, A, hidden):
    from ksim_amd.mlp import MLP
    from ksim_amd.ppo_update import GaussianMlpPolicy

    rng = np.random.default_rng(seed)
    ad, cd = (od, hidden, hidden, A), (od, hidden, 1)
    mk = lambda dims: ([rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])],  # noqa: E731
                       [rng.normal(scale=0.05, size=o).astype(np.float32) for o in dims[1:]])
    (aw, ab), (cw, cb) = mk(ad), mk(cd)
    ls = (rng.normal(size=A) * 0.1 - 0.7).astype(np.float32)
    rollout = dict(actor_obs=rng.normal(size=(Tn, N, od)).astype(np.float32), critic_obs=rng.normal(size=(Tn, N, od)).astype(np.float32),
                   rewards=rng.normal(size=(Tn, N)).astype(np.float32), done=rng.random((Tn, N)) < 0.05,
                   success=np.zeros((Tn, N), bool))
    mean = ou.mlp(torch.tensor(rollout["actor_obs"], dtype=torch.float64), [torch.tensor(w, dtype=torch.float64) for w in aw],
                  [torch.tensor(b, dtype=torch.float64) for b in ab]).numpy()
    rollout["action"] = (mean + np.exp(ls) * rng.normal(size=mean.shape)).astype(np.float32)
    pol = GaussianMlpPolicy(actor=MLP(aw, ab, dtype="f32"), critic=MLP(cw, cb, dtype="f32"), log_std=t32(ls))
    params = dict(actor_w=aw, actor_b=ab, critic_w=cw, critic_b=cb, log_std=ls)
    return pol, params, rollout, rng


def test_single_step_gradients_match_oracle():
    from ksim_amd.ppo_update import PPOUpdateConfig, get_ppo_variables, single_step

    Tn, N, od, A = 16, 8, 30, 6
    pol, params, ro, rng = _setup(7, Tn, N, od, A, 64)
    pol.train_init()
    cfg = PPOUpdateConfig(**{k: v for k, v in CFG.items() if k != "adam_weight_decay"}, adam_weight_decay=0.01)
    d = {k: (torch.tensor(v, device=DEV) if v.dtype == bool else t32(v)) for k, v in ro.items()}
    rows = Tn * N
    on_lp, on_v, _, _ = get_ppo_variables(pol, d["actor_obs"].reshape(rows, od), d["critic_obs"].reshape(rows, od), d["action"].reshape(rows, A))
    on_lp, on_v = on_lp.view(Tn, N, A).clone() - 0.05, on_v.view(Tn, N).clone() + 0.1   # a previous policy, slightly off
    batch = dict(ro, on_log_probs=on_lp.cpu().numpy(), on_values=on_v.cpu().numpy())
    loss, grads, aux = ou.loss_and_grads(params, batch, CFG)
    met = single_step(pol, cfg, d["actor_obs"], d["critic_obs"], d["action"], d["rewards"], d["done"], d["success"], on_lp, on_v)
    assert rel(met["advantages"].cpu().numpy(), aux["advantages"]) < 1e-4
    for (gw, gb), w, b in zip(pol.actor.parameters(gradients=True), grads["actor_w"], grads["actor_b"]):
        assert rel(gw.cpu().numpy(), w) < 5e-4 and rel(gb.cpu().numpy(), b) < 5e-4
    for (gw, gb), w, b in zip(pol.critic.parameters(gradients=True), grads["critic_w"], grads["critic_b"]):
        assert rel(gw.cpu().numpy(), w) < 5e-4 and rel(gb.cpu().numpy(), b) < 5e-4
    assert rel(met["d_log_std"].cpu().numpy(), grads["log_std"]) < 5e-4
    norm = np.sqrt(sum(float((np.asarray(g) ** 2).sum()) for g in ou.flat(grads)))
    assert abs(float(met["grad_norm"].item()) - norm) < 1e-3 * norm


def test_update_model_tracks_oracle():
    from ksim_amd.ppo_update import PPOUpdateConfig, update_model

    Tn, N, od, A = 12, 16, 24, 4
    pol, params, ro, rng = _setup(9, Tn, N, od, A, 64)
    cfg = PPOUpdateConfig(**CFG)
    perms = [rng.permutation(N) for _ in range(cfg.num_passes)]
    want, losses = ou.update_model(params, ro, CFG, perms)
    d = {k: (torch.tensor(v, device=DEV) if v.dtype == bool else t32(v)) for k, v in ro.items()}
    mets = update_model(pol, cfg, d["actor_obs"], d["critic_obs"], d["action"], d["rewards"], d["done"], d["success"],
                        permutations=[torch.tensor(p, device=DEV) for p in perms])
    steps = cfg.num_passes * (N // cfg.batch_size)
    assert len(mets) == steps and pol.opt_step == steps
    # Adam's first steps move a coordinate by about lr whatever the size of its gradient, so a coordinate whose
    # gradient is at rounding level may go the other way: the bound is a few lr, the typical error far below
    bound = 2.5 * cfg.learning_rate * steps
    errs = []
    for (pw, pb), w, b in zip(pol.actor.parameters() + pol.critic.parameters(), want["actor_w"] + want["critic_w"], want["actor_b"] + want["critic_b"]):
        for got, ref in ((pw, w), (pb, b)):
            e = np.abs(got.cpu().numpy() - ref)
            assert e.max() <= bound
            errs.append(e.ravel())
    assert np.abs(pol.log_std.cpu().numpy() - want["log_std"]).max() <= bound
    assert np.median(np.concatenate(errs)) < 2e-6, "typical parameter error after the update"
    moved = np.abs(pol.actor.parameters()[0][0].cpu().numpy() - params["actor_w"][0]).max()
    assert moved > 0.5 * cfg.learning_rate, "the update did not move the parameters"


def test_recurrent_single_step_gradients_match_oracle():
    """One minibatch step of a K-Bot-shaped policy (LSTM actor emitting means | raw deviations, LSTM critic; projection,
    two LSTM layers, linear output) over a (T, b) slice with episode starts: gradients of every parameter against float64
    reverse-mode differentiation of the whole loss (scan over time, head, GAE as a constant, PPO objective)."""
    from ksim_amd import ppo_update as pu
    from ksim_amd.mlp import MLP
    from ksim_amd.recurrent import LSTMCell, RecurrentNetwork

    rng = np.random.default_rng(51)
    Tn, b, I, H, nu = 8, 64, 23, 64, 6

    def make(out_dim):
        proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
        cells = [(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=4 * H) * 0.1)
                 for _ in range(2)]
        ow, ob = [rng.normal(size=(out_dim, H)) / np.sqrt(H)], [rng.normal(size=out_dim) * 0.1]
        carry0 = rng.normal(size=(2, 2, b, H)) * 0.3
        net = RecurrentNetwork(proj, [LSTMCell(*c, dtype="f32") for c in cells], MLP(ow, ob, activation="none", dtype="f32"), dtype="f32")
        return dict(input_proj=proj, cells=cells, out_w=ow, out_b=ob, carry0=carry0), net

    oa, actor = make(2 * nu)
    oc, critic = make(1)
    head = dict(min_std=0.01, max_std=1.0, var_scale=0.5, mean_bias=rng.normal(size=nu) * 0.1)
    obs = rng.normal(size=(Tn, b, I))
    fresh = rng.random((Tn, b)) < 0.08
    done = np.roll(fresh, -1, axis=0); done[-1] = False   # an env restarts at the step after it finished
    batch = dict(actor_obs=obs + rng.normal(size=obs.shape) * 0.01, critic_obs=obs, fresh=fresh, done=done,
                 success=np.zeros((Tn, b), bool), rewards=rng.normal(size=(Tn, b)))
    # the old policy: the same networks a little perturbed, so that ratios differ from one on both sides of the clip
    _, _, _, aux0 = ou.recurrent_loss_and_grads(oa, oc, dict(batch, action=np.zeros((Tn, b, nu)), on_log_probs=np.zeros((Tn, b, nu)),
                                                             on_values=np.zeros((Tn, b))), CFG, head)
    raw0 = aux0["raw"] + rng.normal(size=aux0["raw"].shape) * 0.05
    sd0 = np.minimum((np.logaddexp(0, raw0[..., nu:]) + 0.01) * 0.5, 1.0)
    batch["action"] = raw0[..., :nu] + head["mean_bias"] + sd0 * rng.normal(size=sd0.shape)
    batch["on_log_probs"] = ou.gaussian_head(torch.tensor(raw0), torch.tensor(batch["action"]), 0.01, 1.0, 0.5,
                                             torch.tensor(head["mean_bias"]))[0].numpy()
    batch["on_values"] = aux0["values"] + rng.normal(size=(Tn, b)) * 0.2
    loss, ga, gc, aux = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head)

    policy = pu.RecurrentHeadPolicy(actor, critic, 0.01, 1.0, 0.5, t32(head["mean_bias"]))
    policy.train_init()
    cfg = pu.PPOUpdateConfig(**{k: v for k, v in CFG.items() if k not in ("batch_size", "num_passes")}, batch_size=b)
    u8 = lambda a: torch.tensor(a, dtype=torch.uint8, device=DEV)  # noqa: E731
    m = pu.single_step_recurrent(policy, cfg, t32(batch["actor_obs"]), t32(batch["critic_obs"]), t32(batch["action"]),
                                 t32(batch["rewards"]), u8(done), u8(batch["success"]), t32(batch["on_log_probs"]),
                                 t32(batch["on_values"]), t32(oa["carry0"]), t32(oc["carry0"]), u8(fresh))
    assert rel(m["raw"].cpu().numpy(), aux["raw"]) < 1e-4 and rel(m["values"].cpu().numpy()[..., 0], aux["values"]) < 1e-4
    # gradients were taken before the optimiser step moved the parameters
    for net, want in ((actor, ga), (critic, gc)):
        got = {"proj.W": net.input_proj.parameters(True)[0][0], "proj.b": net.input_proj.parameters(True)[0][1],
               "out.W": net.output_proj.parameters(True)[0][0], "out.b": net.output_proj.parameters(True)[0][1]}
        ref = {"proj.W": want["input_proj"][0], "proj.b": want["input_proj"][1], "out.W": want["out"][0][0], "out.b": want["out"][0][1]}
        for i, c in enumerate(net.cells):
            g = c.parameters(True)
            for k, j in (("weight_ih", 0), ("weight_hh", 1), ("bias", 2)):
                got[f"cell{i}.{k}"], ref[f"cell{i}.{k}"] = g[k], want["cells"][i][j]
        for k in ref:
            assert rel(got[k].cpu().numpy(), ref[k]) < 2e-3, k
    total = sum(float((np.asarray(v) ** 2).sum()) for g in (ga, gc) for v in (g["input_proj"] + tuple(x for c in g["cells"] for x in c) + tuple(x for o in g["out"] for x in o)))
    assert m["grad_norm"].item() == pytest.approx(np.sqrt(total), rel=2e-3)


def test_lowpass_scan_kernels_match_the_oracle():
    """The filter threaded through a trajectory and its reverse sweep, through the C ABI, against the numpy restatement
    (itself pinned by closed forms and central differences): rows of 2 nu floats whose second half travels unchanged, a
    bias per joint, an observation-dependent bias on some joints, restarts inside the slice, and the T = 1 in-place form
    the rollout uses."""
    from ksim_amd import _lib
    from oracle import terms as ot

    lib = _lib.load()
    rng = np.random.default_rng(77)
    Tn, M, nu, I = 11, 37, 6, 9
    dt, fc = 0.02, 6.0
    raw, obs = rng.normal(size=(Tn, M, 2 * nu)), rng.normal(size=(Tn, M, I))
    bias, y0 = rng.normal(size=nu) * 0.2, rng.normal(size=(M, nu))
    fresh = rng.random((Tn, M)) < 0.15
    col0, a0, cnt = 5, 3, 2
    x = raw[..., :nu] + bias
    x[..., a0:a0 + cnt] += obs[..., col0:col0 + cnt]
    want, want_last = ot.lowpass_scan(x, dt, fc, y0, fresh)
    d_raw, d_obs, d_f = t32(raw), t32(obs), torch.tensor(fresh, dtype=torch.uint8, device=DEV)
    out, last = torch.empty_like(d_raw), torch.empty(M, nu, device=DEV)
    d_bias, d_y0in = t32(bias), t32(y0)  # named, so that they outlive the launches that read them
    add = ctypes.c_void_p(d_obs.data_ptr() + 4 * col0)
    _lib.check(lib.ks_lowpass_scan(_lib.current_stream(), Tn, M, nu, 2 * nu, dt, fc, _lib.ptr(d_raw), _lib.ptr(d_bias), add, I, a0, cnt,
                                   _lib.ptr(d_y0in), _lib.ptr(d_f), _lib.ptr(out), _lib.ptr(last)))
    got = out.cpu().numpy()
    np.testing.assert_allclose(got[..., :nu], want, rtol=2e-5, atol=2e-6)
    assert np.array_equal(got[..., nu:], raw[..., nu:].astype(np.float32))
    np.testing.assert_allclose(last.cpu().numpy(), want_last, rtol=2e-5, atol=2e-6)
    # reverse sweep, in place on the first nu columns
    g = rng.normal(size=(Tn, M, 2 * nu))
    want_dx, want_dy0 = ot.lowpass_scan_backward(g[..., :nu], dt, fc, fresh)
    d_g, d_y0 = t32(g), torch.empty(M, nu, device=DEV)
    _lib.check(lib.ks_lowpass_scan_backward(_lib.current_stream(), Tn, M, nu, 2 * nu, dt, fc, _lib.ptr(d_f), _lib.ptr(d_g), _lib.ptr(d_y0)))
    np.testing.assert_allclose(d_g.cpu().numpy()[..., :nu], want_dx, rtol=2e-5, atol=2e-6)
    assert np.array_equal(d_g.cpu().numpy()[..., nu:], g[..., nu:].astype(np.float32))
    np.testing.assert_allclose(d_y0.cpu().numpy(), want_dy0, rtol=2e-5, atol=2e-6)
    # one step in place, the state advanced in its own buffer: bit-equal to step 0 of the scan
    state, step0 = t32(y0), t32(raw[0])
    f0 = d_f[0].contiguous()
    _lib.check(lib.ks_lowpass_scan(_lib.current_stream(), 1, M, nu, 2 * nu, dt, fc, _lib.ptr(step0), _lib.ptr(d_bias), add, I, a0, cnt,
                                   _lib.ptr(state), _lib.ptr(f0), _lib.ptr(step0), _lib.ptr(state)))
    assert torch.equal(step0, out[0]) and torch.equal(state, out[0][:, :nu])
    assert lib.ks_lowpass_scan(_lib.current_stream(), Tn, M, nu, nu - 1, dt, fc, _lib.ptr(d_raw), None, None, 0, 0, 0, None, None, _lib.ptr(out), None) != 0
    assert lib.ks_lowpass_scan(_lib.current_stream(), Tn, M, nu, 2 * nu, dt, fc, _lib.ptr(d_raw), None, add, I, nu - 1, 2, None, None, _lib.ptr(out), None) != 0


@pytest.mark.parametrize("symmetric", [False, True])
def test_kbot_training_step_with_filter_and_mirror_carries_matches_oracle(symmetric):
    """The K-Bot task's minibatch step as shipped (examples/kbot/train.py:903-934, 1439-1533): LSTM actor whose biased means
    (bias vector + command columns of the observation) pass the one-pole low-pass with its state in the carry, LSTM
    critic, and the mirrored second pass of both from their own carries with the two mirror losses.  Every parameter's
    gradient against float64 reverse-mode differentiation of that loss.  `symmetric`: the mirror map is the identity and
    the mirrored carries equal the first pass's, so both mirror losses must vanish and leave the gradients alone."""
    from ksim_amd import ppo_update as pu
    from ksim_amd.actions import LowPass
    from ksim_amd.mlp import MLP
    from ksim_amd.recurrent import LSTMCell, RecurrentNetwork

    rng = np.random.default_rng(61)
    Tn, b, I, H, nu = 8, 48, 26, 64, 10

    def make(out_dim):
        proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
        cells = [(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=4 * H) * 0.1)
                 for _ in range(2)]
        ow, ob = [rng.normal(size=(out_dim, H)) / np.sqrt(H)], [rng.normal(size=out_dim) * 0.1]
        carry0 = rng.normal(size=(2, 2, b, H)) * 0.3
        net = RecurrentNetwork(proj, [LSTMCell(*c, dtype="f32") for c in cells], MLP(ow, ob, activation="none", dtype="f32"), dtype="f32")
        return dict(input_proj=proj, cells=cells, out_w=ow, out_b=ob, carry0=carry0), net

    oa, actor = make(2 * nu)
    oc, critic = make(1)
    head = dict(min_std=0.01, max_std=1.0, var_scale=0.5, mean_bias=rng.normal(size=nu) * 0.1)
    obs = rng.normal(size=(Tn, b, I))
    fresh = rng.random((Tn, b)) < 0.1
    done = np.roll(fresh, -1, axis=0); done[-1] = False
    batch = dict(actor_obs=obs + rng.normal(size=obs.shape) * 0.01, critic_obs=obs, fresh=fresh, done=done,
                 success=np.zeros((Tn, b), bool), rewards=rng.normal(size=(Tn, b)))
    lowpass = dict(ctrl_dt=0.02, cutoff=10.0, y0=rng.normal(size=(b, nu)) * 0.2, obs_bias=(I - 4, nu - 4, 4))
    if symmetric:
        operm, osign, aperm, asign = np.arange(I), np.ones(I), np.arange(nu), np.ones(nu)
        mirror = dict(actor_carry0=oa["carry0"], critic_carry0=oc["carry0"], y0=lowpass["y0"])
    else:  # legs and arms swap, every joint negated; the observation entries reorder and change sign likewise
        aperm, asign = np.r_[np.arange(3, 6), np.arange(0, 3), np.arange(6, 10)], -np.ones(nu)
        operm, osign = rng.permutation(I), rng.choice([-1.0, 1.0], I)
        mirror = dict(actor_carry0=rng.normal(size=(2, 2, b, H)) * 0.3, critic_carry0=rng.normal(size=(2, 2, b, H)) * 0.3,
                      y0=rng.normal(size=(b, nu)) * 0.2)
    mirror.update(actor_obs=(operm, osign), critic_obs=(operm, osign), action=(aperm, asign), actor_scale=0.8, critic_scale=0.4)
    # the old policy: the same networks a little perturbed, so that ratios differ from one on both sides of the clip
    zero = dict(batch, action=np.zeros((Tn, b, nu)), on_log_probs=np.zeros((Tn, b, nu)), on_values=np.zeros((Tn, b)))
    aux0 = ou.recurrent_loss_and_grads(oa, oc, zero, CFG, head, lowpass=lowpass)[3]
    raw0 = aux0["raw"] + rng.normal(size=aux0["raw"].shape) * 0.05
    sd0 = np.minimum((np.logaddexp(0, raw0[..., nu:]) + 0.01) * 0.5, 1.0)
    batch["action"] = raw0[..., :nu] + sd0 * rng.normal(size=sd0.shape)
    batch["on_log_probs"] = ou.gaussian_head(torch.tensor(raw0), torch.tensor(batch["action"]), 0.01, 1.0, 0.5)[0].numpy()
    batch["on_values"] = aux0["values"] + rng.normal(size=(Tn, b)) * 0.2
    loss, ga, gc, aux = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass, mirror=mirror)
    loss_plain, ga_plain, _, _ = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass)

    spec = pu.MirrorSpec(list(operm), list(osign), list(operm), list(osign), list(aperm), list(asign))
    policy = pu.RecurrentHeadPolicy(actor, critic, 0.01, 1.0, 0.5, t32(head["mean_bias"]), mirror=spec,
                                    lowpass=LowPass(0.02, 10.0, obs_bias=lowpass["obs_bias"]))
    policy.train_init()
    cfg = pu.PPOUpdateConfig(**{k: v for k, v in CFG.items() if k not in ("batch_size", "num_passes")}, batch_size=b,
                             actor_mirror_loss_scale=0.8, critic_mirror_loss_scale=0.4)
    u8 = lambda a: torch.tensor(a, dtype=torch.uint8, device=DEV)  # noqa: E731
    m = pu.single_step_recurrent(policy, cfg, t32(batch["actor_obs"]), t32(batch["critic_obs"]), t32(batch["action"]),
                                 t32(batch["rewards"]), u8(done), u8(batch["success"]), t32(batch["on_log_probs"]),
                                 t32(batch["on_values"]), t32(oa["carry0"]), t32(oc["carry0"]), u8(fresh), t32(lowpass["y0"]),
                                 pu.MirrorCarries(t32(mirror["actor_carry0"]), t32(mirror["critic_carry0"]), t32(mirror["y0"])))
    assert rel(m["raw"].cpu().numpy(), aux["raw"]) < 1e-4 and rel(m["values"].cpu().numpy()[..., 0], aux["values"]) < 1e-4
    if symmetric:
        assert m["action_mirror_loss"].abs().max().item() == 0.0 and m["value_mirror_loss"].abs().max().item() == 0.0
        # (float64 matrix products of the library differ in the last bit between the two passes: 1e-32, not 0)
        assert np.abs(aux["action_mirror_loss"]).max() < 1e-25 and loss == pytest.approx(loss_plain, rel=1e-13)
    else:
        assert rel(m["action_mirror_loss"].cpu().numpy(), aux["action_mirror_loss"]) < 1e-3
        assert rel(m["value_mirror_loss"].cpu().numpy(), aux["value_mirror_loss"]) < 1e-3
        assert aux["action_mirror_loss"].mean() > 1e-3  # the term is there, and it changes the gradient
        assert rel(ga["out"][0][0], ga_plain["out"][0][0]) > 1e-2
    for net, want in ((actor, ga), (critic, gc)):
        got = {"proj.W": net.input_proj.parameters(True)[0][0], "proj.b": net.input_proj.parameters(True)[0][1],
               "out.W": net.output_proj.parameters(True)[0][0], "out.b": net.output_proj.parameters(True)[0][1]}
        ref = {"proj.W": want["input_proj"][0], "proj.b": want["input_proj"][1], "out.W": want["out"][0][0], "out.b": want["out"][0][1]}
        for i, c in enumerate(net.cells):
            g = c.parameters(True)
            for k, j in (("weight_ih", 0), ("weight_hh", 1), ("bias", 2)):
                got[f"cell{i}.{k}"], ref[f"cell{i}.{k}"] = g[k], want["cells"][i][j]
        for k in ref:
            assert rel(got[k].cpu().numpy(), ref[k]) < 2e-3, k
    # the deviation half of the mirrored pass enters no loss: the raw-deviation rows of the output layer see the first pass only
    total = sum(float((np.asarray(v) ** 2).sum()) for g in (ga, gc) for v in (g["input_proj"] + tuple(x for c in g["cells"] for x in c) + tuple(x for o in g["out"] for x in o)))
    assert m["grad_norm"].item() == pytest.approx(np.sqrt(total), rel=2e-3)


def test_ppo_loss_gradient_for_the_mixture_head_matches_autograd():
    """d loss / d (means | raw deviations | logits) for the mixture head against float64 autograd of the oracle loss (policy
    and KL terms through the exact mixture log-density, entropy term through the stated upper bound); clipped means and
    capped deviations get no gradient."""
    from ksim_amd import _lib, _lib_terms as T
    from oracle import terms as ot

    lib = _lib.load()
    rng = np.random.default_rng(23)
    M, A, K = 1500, 6, 10
    raw = rng.normal(size=(M, 3 * A * K))
    raw[:40, A * K:2 * A * K] = 6.0          # capped deviations
    raw[40:80, :A * K] = 3.0                 # means beyond the clip range
    bias = rng.normal(size=A) * 0.1
    lo, hi = -np.ones(A) * 1.5, np.ones(A) * 1.8
    hd = dict(min_std=0.01, max_std=1.2, var_scale=0.5)
    act, _, _ = ot.mixture_head(raw, K, uniform=rng.random((M, A)), normal=rng.normal(size=(M, A)), mean_bias=bias, clip_lo=lo,
                                clip_hi=hi, **hd)
    tb, tlo, thi = torch.tensor(bias), torch.tensor(lo), torch.tensor(hi)
    on_lp = ou.mixture_head(torch.tensor(raw + rng.normal(size=raw.shape) * 0.02), torch.tensor(act), K, mean_bias=tb, clip_lo=tlo,
                            clip_hi=thi, **hd)[0].numpy()
    adv, tgt, on_v = rng.normal(size=M), rng.normal(size=M), rng.normal(size=M)
    v = on_v + rng.normal(size=M) * 0.3
    tr, tv = torch.tensor(raw, requires_grad=True), torch.tensor(v, requires_grad=True)
    lp, ent = ou.mixture_head(tr, torch.tensor(act), K, mean_bias=tb, clip_lo=tlo, clip_hi=thi, **hd)
    loss, _ = ou.ppo_loss_torch(torch.tensor(adv), torch.tensor(tgt), torch.tensor(on_lp), torch.tensor(on_v), lp, tv, ent, CFG, 1.3)
    loss.backward()
    p = _lib.KsPpoLossParams(0.2, 0.5, 0.008, 1e-3, 5.0, 1.3, 1)
    dev = [t32(a) for a in (bias, lo, hi)]
    head = T.KsMixtureHead(K, 0.01, 1.2, 0.5, 0, *[_lib.ptr(t).value for t in dev])
    d_raw, d_value = torch.empty(M, 3 * A * K, device=DEV), torch.empty(M, device=DEV)
    args = [t32(a) for a in (raw, act, on_lp, adv, tgt, on_v, v)]
    _lib.check(lib.ks_ppo_loss_grad_mixture(_lib.current_stream(), M, A, ctypes.byref(p), ctypes.byref(head), *[_lib.ptr(a) for a in args],
                                            _lib.ptr(d_raw), _lib.ptr(d_value)))
    g, got = tr.grad.numpy(), d_raw.cpu().numpy()
    for name, sl in (("means", slice(0, A * K)), ("deviations", slice(A * K, 2 * A * K)), ("logits", slice(2 * A * K, None))):
        assert rel(got[:, sl], g[:, sl]) < 2e-4, name
    assert rel(d_value.cpu().numpy(), tv.grad.numpy()) < 1e-5
    assert (got[:40, A * K:2 * A * K] == 0).all() and (got[40:80, :A * K] == 0).all() and (g[40:80, :A * K] == 0).all()
    # the kernel that drew the actions reports the log-density this gradient starts from
    from ksim_amd.env_terms import sample_action_mixture
    _, lp_k, _ = sample_action_mixture(args[0], K, mean_bias=dev[0], clip_lo=dev[1], clip_hi=dev[2], uniform=t32(rng.random((M, A))),
                                       noise=t32(rng.normal(size=(M, A))), want_stats=True, **hd)
    assert torch.isfinite(lp_k).all()


def test_adaptive_kl_coefficient_is_updated_on_the_device():
    """ppo.py:546-563: the coefficient grows by 1.5 above 1.5 x desired, shrinks by 1.5 below desired / 1.5, stays inside the
    band and is clipped to [1e-8, 1e2].  Expected values below are worked out by hand from the mean of the row sums."""
    from ksim_amd import _lib

    lib = _lib.load()
    rows, A, kl_coef = 1000, 5, 1e-3
    rng = np.random.default_rng(3)
    lp = rng.normal(size=(rows, A)).astype(np.float32)
    ws = torch.empty(256, device=DEV)

    def run(diff_per_element, scale0, desired):
        on_lp = lp + np.float32(diff_per_element)  # mean over rows of sum over actions = A * diff
        s = torch.tensor([scale0], dtype=torch.float32, device=DEV)
        a, b = t32(on_lp), t32(lp)
        _lib.check(lib.ks_ppo_adapt_kl(_lib.current_stream(), rows, A, _lib.ptr(a), _lib.ptr(b), kl_coef, desired,
                                       _lib.ptr(s), _lib.ptr(ws)))
        return float(s.item())

    # kl_mean = 5 * 0.4 * 1e-3 * 2 = 4e-3
    assert run(0.4, 2.0, 0.002) == pytest.approx(3.0, rel=1e-5)       # 4e-3 > 3e-3: x 1.5
    assert run(0.4, 2.0, 0.01) == pytest.approx(2.0 / 1.5, rel=1e-5)  # 4e-3 < 6.67e-3: / 1.5
    assert run(0.4, 2.0, 0.004) == pytest.approx(2.0, rel=1e-6)       # inside the band
    assert run(0.4, 9e4, 1e-6) == pytest.approx(1e5, rel=1e-5)        # 90 x 1.5 = 135 is clipped to 1e2 = 1e5 x kl_coef
    assert run(-0.4, 1.2e-5, 1.0) == pytest.approx(1e-5, rel=1e-5)    # 1.2e-8 / 1.5 is clipped to 1e-8


def test_adaptive_kl_in_single_step_follows_the_host_rule_without_a_sync():
    from ksim_amd.ppo_update import PPOUpdateConfig, get_ppo_variables, single_step

    Tn, N, od, A = 16, 8, 30, 6
    pol, params, ro, rng = _setup(11, Tn, N, od, A, 64)
    pol.train_init()
    cfg = PPOUpdateConfig(**dict(CFG, learning_rate=3e-3), adaptive_kl=True, desired_kl=2e-4)
    d = {k: (torch.tensor(v, device=DEV) if v.dtype == bool else t32(v)) for k, v in ro.items()}
    rows = Tn * N
    on_lp, on_v, _, _ = get_ppo_variables(pol, d["actor_obs"].reshape(rows, od), d["critic_obs"].reshape(rows, od), d["action"].reshape(rows, A))
    on_lp, on_v = on_lp.view(Tn, N, A).clone(), on_v.view(Tn, N).clone()
    coef, seen = cfg.kl_coef, set()
    for _ in range(8):
        met = single_step(pol, cfg, d["actor_obs"], d["critic_obs"], d["action"], d["rewards"], d["done"], d["success"], on_lp, on_v)
        kl_mean = float((on_lp.reshape(rows, A).double() - met["log_probs"].double()).sum(-1).mean().item()) * coef
        new = coef * 1.5 if kl_mean > cfg.desired_kl * 1.5 else coef
        new = new / 1.5 if kl_mean < cfg.desired_kl / 1.5 else new
        seen.add("up" if new > coef else "down" if new < coef else "same")
        coef = min(max(new, 1e-8), 1e2)
        assert pol.kl_coef(cfg) == pytest.approx(coef, rel=1e-5)
    assert {"up", "down"} <= seen, f"the test drove the coefficient only {seen}"


def test_gradient_norm_and_update_are_bit_reproducible():
    """The global norm behind clip_by_global_norm is summed in a fixed order: two updates from the same state are the same bits."""
    from ksim_amd.ppo_update import PPOUpdateConfig, update_model

    outs = []
    for _ in range(2):
        Tn, N, od, A = 12, 64, 24, 4
        pol, params, ro, rng = _setup(13, Tn, N, od, A, 512)
        cfg = PPOUpdateConfig(**dict(CFG, grad_clip=0.05, batch_size=16))
        d = {k: (torch.tensor(v, device=DEV) if v.dtype == bool else t32(v)) for k, v in ro.items()}
        perms = [torch.tensor(np.random.default_rng(p).permutation(N), device=DEV) for p in range(cfg.num_passes)]
        mets = update_model(pol, cfg, d["actor_obs"], d["critic_obs"], d["action"], d["rewards"], d["done"], d["success"], permutations=perms)
        outs.append([m["grad_norm"].clone() for m in mets] + [p.clone() for pair in pol.actor.parameters() + pol.critic.parameters() for p in pair])
    assert float(outs[0][0].item()) > 0.05, "the clip is not active"
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_mirror_losses_match_autograd_and_vanish_for_a_symmetric_policy():
    """Mirror losses of the K-Bot task (examples/kbot/train.py:1458-1477) inside the minibatch step: per-transition loss values
    and every parameter gradient against float64 autograd of the same terms added to the PPO loss; a policy that already
    commutes with the mirror maps has zero mirror loss and the gradients of plain PPO."""
    from ksim_amd.mlp import MLP
    from ksim_amd.ppo_update import GaussianMlpPolicy, MirrorSpec, PPOUpdateConfig, get_ppo_variables, kbot_mirror_joints, single_step

    Tn, N, od, A = 8, 8, 26, 20
    pol, params, ro, rng = _setup(17, Tn, N, od, A, 64)
    aperm, asign = kbot_mirror_joints()
    assert aperm[:10] == [5, 6, 7, 8, 9, 0, 1, 2, 3, 4] and aperm[10:] == list(range(10, 20)) and set(asign) == {-1.0}
    operm = list(rng.permutation(od))
    osign = list(rng.choice([-1.0, 1.0], od))
    cperm = list(rng.permutation(od))
    csign = list(rng.choice([-1.0, 1.0], od))
    pol.mirror = MirrorSpec(operm, osign, cperm, csign, aperm, asign)
    pol.train_init()
    cfgd = dict(CFG, batch_size=N)
    cfg = PPOUpdateConfig(**cfgd, actor_mirror_loss_scale=0.7, critic_mirror_loss_scale=0.3)
    d = {k: (torch.tensor(v, device=DEV) if v.dtype == bool else t32(v)) for k, v in ro.items()}
    rows = Tn * N
    on_lp, on_v, _, _ = get_ppo_variables(pol, d["actor_obs"].reshape(rows, od), d["critic_obs"].reshape(rows, od), d["action"].reshape(rows, A))
    on_lp, on_v = on_lp.view(Tn, N, A).clone() - 0.03, on_v.view(Tn, N).clone() + 0.05
    batch = dict(ro, on_log_probs=on_lp.cpu().numpy(), on_values=on_v.cpu().numpy())
    mirror = dict(actor_obs=(operm, osign), critic_obs=(cperm, csign), action=(aperm, asign), actor_scale=0.7, critic_scale=0.3)
    loss, grads, aux = ou.loss_and_grads(params, batch, cfgd, mirror=mirror)
    plain = ou.loss_and_grads(params, batch, cfgd)[1]
    assert rel(grads["actor_w"][0], plain["actor_w"][0]) > 0.05, "the mirror terms do not matter in this test"
    met = single_step(pol, cfg, d["actor_obs"], d["critic_obs"], d["action"], d["rewards"], d["done"], d["success"], on_lp, on_v)
    assert rel(met["action_mirror_loss"].cpu().numpy(), aux["terms"]["action_mirror_loss"].reshape(-1)) < 1e-4
    assert rel(met["value_mirror_loss"].cpu().numpy(), aux["terms"]["value_mirror_loss"].reshape(-1)) < 1e-4
    for net, kw, kb in ((pol.actor, "actor_w", "actor_b"), (pol.critic, "critic_w", "critic_b")):
        for (gw, gb), w, b in zip(net.parameters(gradients=True), grads[kw], grads[kb]):
            assert rel(gw.cpu().numpy(), w) < 5e-4 and rel(gb.cpu().numpy(), b) < 5e-4
    assert rel(met["d_log_std"].cpu().numpy(), grads["log_std"]) < 5e-4

    # a linear actor W with W = P_a W P_o^T (and a critic row w = w P_c^T) is mirror-symmetric: zero loss, PPO's gradients
    def sym(perm_out, sign_out, perm_in, sign_in, w):
        po = np.zeros((len(perm_out), len(perm_out)))
        po[np.arange(len(perm_out)), perm_out] = sign_out   # mirrored[j] = sign[j] x[perm[j]]
        pi = np.zeros((len(perm_in), len(perm_in)))
        pi[np.arange(len(perm_in)), perm_in] = sign_in
        return (0.5 * (w + po @ w @ np.linalg.inv(pi))).astype(np.float32)  # average over the two-element group generated by a pair of involutions

    # the K-Bot joint mirror is an involution; give the observation an involution too
    oinv = list(range(od)); oinv[0], oinv[1] = 1, 0; oinv[4], oinv[9] = 9, 4
    osg = [1.0] * od; osg[2] = -1.0; osg[4] = osg[9] = -1.0
    wa = sym(aperm, asign, oinv, osg, rng.normal(size=(A, od)) * 0.2)
    wc = sym([0], [1.0], oinv, osg, rng.normal(size=(1, od)) * 0.2)
    pol2 = GaussianMlpPolicy(actor=MLP([wa], [np.zeros(A, np.float32)], dtype="f32"), critic=MLP([wc], [np.zeros(1, np.float32)], dtype="f32"),
                             log_std=pol.log_std.clone(), mirror=MirrorSpec(oinv, osg, oinv, osg, aperm, asign))
    pol3 = GaussianMlpPolicy(actor=MLP([wa], [np.zeros(A, np.float32)], dtype="f32"), critic=MLP([wc], [np.zeros(1, np.float32)], dtype="f32"),
                             log_std=pol.log_std.clone())
    pol2.train_init(); pol3.train_init()
    m2 = single_step(pol2, cfg, d["actor_obs"], d["critic_obs"], d["action"], d["rewards"], d["done"], d["success"], on_lp, on_v)
    single_step(pol3, PPOUpdateConfig(**cfgd), d["actor_obs"], d["critic_obs"], d["action"], d["rewards"], d["done"], d["success"], on_lp, on_v)
    assert float(m2["action_mirror_loss"].abs().max()) < 1e-10 and float(m2["value_mirror_loss"].abs().max()) < 1e-10
    for a, b in zip(pol2.actor.parameters(gradients=True) + pol2.critic.parameters(gradients=True),
                    pol3.actor.parameters(gradients=True) + pol3.critic.parameters(gradients=True)):
        assert rel(a[0].cpu().numpy(), b[0].cpu().numpy()) < 1e-5 and rel(a[1].cpu().numpy(), b[1].cpu().numpy()) < 1e-5
