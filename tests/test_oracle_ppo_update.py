"""Pins the torch restatement of the PPO loss (used for autograd) and the optimiser chain of oracle/ppo_update.py."""
import math

import numpy as np
import pytest
import torch

from oracle import ppo as oppo
from oracle import ppo_update as ou

CFG = dict(gamma=0.99, lam=0.95, normalize_advantages=True, monte_carlo_returns=False, clip_param=0.2, value_loss_coef=0.5,
           entropy_coef=0.008, kl_coef=1e-3, log_clip_value=5.0, use_clipped_value_loss=True, learning_rate=3e-4,
           adam_b1=0.9, adam_b2=0.999, adam_eps=1e-8, adam_weight_decay=0.01, grad_clip=2.0, batch_size=4)


def test_torch_loss_equals_numpy_restatement():
    rng = np.random.default_rng(0)
    B, Tn, A = 7, 9, 3
    adv, tgt = rng.normal(size=(B, Tn)), rng.normal(size=(B, Tn))
    on_lp, lp = rng.normal(size=(B, Tn, A)), rng.normal(size=(B, Tn, A)) * 0.3
    lp = on_lp + lp  # ratios on both sides of the clip range
    on_v, v, ent = rng.normal(size=(B, Tn)), rng.normal(size=(B, Tn)), rng.normal(size=(B, Tn, A))
    want = oppo.compute_ppo_loss(adv, tgt, on_lp, on_v, lp, v, ent, kl_scale=1.7)
    t = lambda a: torch.tensor(a)  # noqa: E731
    loss, terms = ou.ppo_loss_torch(t(adv), t(tgt), t(on_lp), t(on_v), t(lp), t(v), t(ent), CFG, kl_scale=1.7)
    assert abs(float(loss) - want["total"]) < 1e-14
    for k in ("policy", "value", "kl", "entropy"):
        np.testing.assert_allclose(terms[k].numpy(), want[k], rtol=1e-13, atol=1e-15)


def test_gaussian_head_against_scipy_and_finite_differences():
    from scipy.stats import norm

    rng = np.random.default_rng(1)
    mean, ls, a = rng.normal(size=(5, 4)), rng.normal(size=4) * 0.3, rng.normal(size=(5, 4))
    lp, ent = ou.gaussian(torch.tensor(mean), torch.tensor(ls), torch.tensor(a))
    np.testing.assert_allclose(lp.numpy(), norm.logpdf(a, mean, np.exp(ls)), rtol=1e-12)
    np.testing.assert_allclose(ent.numpy()[0], norm.entropy(0, np.exp(ls)), rtol=1e-12)


def test_autograd_gradient_against_finite_differences():
    rng = np.random.default_rng(2)
    Tn, b, od, A = 6, 4, 5, 2
    params = dict(actor_w=[rng.normal(size=(8, od)) * 0.4, rng.normal(size=(A, 8)) * 0.4], actor_b=[np.zeros(8), np.zeros(A)],
                  critic_w=[rng.normal(size=(8, od)) * 0.4, rng.normal(size=(1, 8)) * 0.4], critic_b=[np.zeros(8), np.zeros(1)],
                  log_std=rng.normal(size=A) * 0.1 - 0.5)
    batch = dict(actor_obs=rng.normal(size=(Tn, b, od)), critic_obs=rng.normal(size=(Tn, b, od)), action=rng.normal(size=(Tn, b, A)),
                 rewards=rng.normal(size=(Tn, b)), done=rng.random((Tn, b)) < 0.1, success=np.zeros((Tn, b), bool),
                 on_log_probs=rng.normal(size=(Tn, b, A)) - 1.0, on_values=rng.normal(size=(Tn, b)))
    cfg = dict(CFG, normalize_advantages=False)
    loss, grads, aux = ou.loss_and_grads(params, batch, cfg)
    # finite differences with the advantages frozen (they are a constant of the loss)
    t = torch.tensor

    def f(p):
        mean = ou.mlp(t(batch["actor_obs"]), [t(x) for x in p["actor_w"]], [t(x) for x in p["actor_b"]])
        v = ou.mlp(t(batch["critic_obs"]), [t(x) for x in p["critic_w"]], [t(x) for x in p["critic_b"]])[..., 0]
        lp, ent = ou.gaussian(mean, t(p["log_std"]), t(batch["action"]))
        return float(ou.ppo_loss_torch(t(aux["advantages"]), t(aux["value_targets"]), t(batch["on_log_probs"]),
                                       t(batch["on_values"]), lp, v, ent, cfg)[0])

    assert abs(f(params) - loss) < 1e-12
    for key, idx in [("actor_w", (0, (3, 2))), ("critic_w", (1, (0, 5))), ("actor_b", (1, (1,)))]:
        l, ij = idx
        for eps in (1e-6,):
            p2 = {k: ([x.copy() for x in v] if isinstance(v, list) else v.copy()) for k, v in params.items()}
            p2[key][l][ij] += eps
            p3 = {k: ([x.copy() for x in v] if isinstance(v, list) else v.copy()) for k, v in params.items()}
            p3[key][l][ij] -= eps
            fd = (f(p2) - f(p3)) / (2 * eps)
            assert abs(fd - grads[key][l][ij]) < 1e-6 * max(1.0, abs(fd)), (key, fd, grads[key][l][ij])
    p2 = dict(params, log_std=params["log_std"] + np.array([1e-6, 0.0]))
    p3 = dict(params, log_std=params["log_std"] - np.array([1e-6, 0.0]))
    assert abs((f(p2) - f(p3)) / 2e-6 - grads["log_std"][0]) < 1e-6


def test_optimiser_chain_known_answers():
    cfg = dict(CFG, adam_weight_decay=0.0, grad_clip=0.0)
    # first Adam step moves every coordinate by lr * sign(g) (bias-corrected moments: m/sqrt(v) = +-1)
    p, m1, m2, norm = ou.optax_chain_step([np.array([1.0, -2.0, 3.0])], [np.array([0.5, -4.0, np.nan])], [np.zeros(3)], [np.zeros(3)], 1, cfg)
    np.testing.assert_allclose(p[0], [1.0 - 3e-4, -2.0 + 3e-4, 3.0], rtol=0, atol=1e-10)  # the NaN gradient is zeroed
    assert abs(norm - math.sqrt(0.25 + 16)) < 1e-12
    # clipping: gradient of norm 5 clipped to norm 2 keeps its direction
    cfg2 = dict(cfg, grad_clip=2.0, adam_b1=0.0, adam_b2=0.0, adam_eps=0.0)
    p, m1, _, _ = ou.optax_chain_step([np.zeros(2)], [np.array([3.0, 4.0])], [np.zeros(2)], [np.zeros(2)], 1, cfg2)
    np.testing.assert_allclose(m1[0], [1.2, 1.6])
    # weight decay enters the gradient before Adam
    cfg3 = dict(cfg, adam_weight_decay=0.1, adam_b1=0.0, adam_b2=0.0)
    _, m1, _, _ = ou.optax_chain_step([np.array([10.0])], [np.array([1.0])], [np.zeros(1)], [np.zeros(1)], 1, cfg3)
    np.testing.assert_allclose(m1[0], [2.0])


def test_mixture_head_in_torch_matches_the_numpy_oracle_and_bounds_the_entropy():
    """The differentiable mixture head used for the gradient check: its log-density equals the numpy oracle's (pinned by
    scipy), and its entropy term is an upper bound of the mixture's entropy (Monte-Carlo estimate on one mixture)."""
    from oracle import terms as ot

    rng = np.random.default_rng(5)
    M, A, K = 30, 4, 3
    raw = rng.normal(size=(M, 3 * A * K))
    bias = rng.normal(size=A) * 0.1
    lo, hi = -np.ones(A), np.ones(A) * 1.2
    hd = dict(min_std=0.02, max_std=0.8, var_scale=0.5)
    act, logp, _ = ot.mixture_head(raw, K, uniform=rng.random((M, A)), normal=rng.normal(size=(M, A)), mean_bias=bias, clip_lo=lo, clip_hi=hi, **hd)
    lp, ent = ou.mixture_head(torch.tensor(raw), torch.tensor(act), K, mean_bias=torch.tensor(bias), clip_lo=torch.tensor(lo),
                              clip_hi=torch.tensor(hi), **hd)
    np.testing.assert_allclose(lp.numpy(), logp, rtol=1e-10, atol=1e-10)
    # entropy of env 0, action 0 by sampling: -E[log p] <= sum_k pi_k H_k + H(pi)
    one = np.tile(raw[:1], (200000, 1))
    a, l, _ = ot.mixture_head(one, K, uniform=rng.random((200000, A)), normal=rng.normal(size=(200000, A)), mean_bias=bias, clip_lo=lo, clip_hi=hi, **hd)
    h_mc = -l[:, 0].mean()
    assert h_mc <= float(ent[0, 0]) + 0.01
    assert float(ent[0, 0]) - h_mc < np.log(K) + 0.01  # and within the mixing entropy of it


def _kbot_case(rng, Tn=6, b=5, I=12, H=8, nu=4):
    """A small K-Bot-shaped problem: LSTM actor (means | raw deviations) and critic, episode starts inside the slice, the
    last two observation columns feeding the bias of the last two action means."""
    def make(out_dim):
        proj = (rng.normal(size=(H, I)) / np.sqrt(I), rng.normal(size=H) * 0.1)
        cells = [(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=4 * H) * 0.1)
                 for _ in range(2)]
        return dict(input_proj=proj, cells=cells, out_w=[rng.normal(size=(out_dim, H)) / np.sqrt(H)], out_b=[rng.normal(size=out_dim) * 0.1],
                    carry0=rng.normal(size=(2, 2, b, H)) * 0.3)

    oa, oc = make(2 * nu), make(1)
    head = dict(min_std=0.01, max_std=1.0, var_scale=0.5, mean_bias=rng.normal(size=nu) * 0.1)
    obs = rng.normal(size=(Tn, b, I))
    fresh = rng.random((Tn, b)) < 0.25
    fresh[2, 0] = True
    done = np.roll(fresh, -1, axis=0); done[-1] = False
    batch = dict(actor_obs=obs + rng.normal(size=obs.shape) * 0.01, critic_obs=obs, fresh=fresh, done=done,
                 success=np.zeros((Tn, b), bool), rewards=rng.normal(size=(Tn, b)), action=rng.normal(size=(Tn, b, nu)) * 0.3,
                 on_log_probs=rng.normal(size=(Tn, b, nu)) * 0.1 - 0.5, on_values=rng.normal(size=(Tn, b)) * 0.3)
    lowpass = dict(ctrl_dt=0.02, cutoff=10.0, y0=rng.normal(size=(b, nu)) * 0.2, obs_bias=(I - 2, nu - 2, 2))
    # a mirror map that swaps and negates entries (a signed permutation, like mirror_joints / mirror_obs of the task)
    operm = rng.permutation(I); osign = rng.choice([-1.0, 1.0], I)
    aperm = rng.permutation(nu); asign = rng.choice([-1.0, 1.0], nu)
    mirror = dict(actor_obs=(operm, osign), critic_obs=(operm, osign), action=(aperm, asign), actor_scale=0.7, critic_scale=0.3,
                  actor_carry0=rng.normal(size=(2, 2, b, H)) * 0.3, critic_carry0=rng.normal(size=(2, 2, b, H)) * 0.3,
                  y0=rng.normal(size=(b, nu)) * 0.2)
    return oa, oc, head, batch, lowpass, mirror


def _bump(net, path, eps):
    """A copy of the network dict with one parameter entry moved by eps; path = (key, ..., index tuple)."""
    import copy

    out = copy.deepcopy(net)
    obj = out
    for k in path[:-2]:
        obj = obj[k]
    arr = np.array(obj[path[-2]], dtype=np.float64)
    arr[path[-1]] += eps
    if isinstance(obj, tuple):
        raise TypeError
    obj[path[-2]] = arr
    return out


def test_kbot_loss_with_filter_and_mirror_carries_against_central_differences():
    """The recurrent loss with the low-pass filter on the means (state carried through time, cut at episode starts) and the
    mirrored second pass of both networks.  GAE enters as a constant and depends on the critic only, so central differences
    of the whole loss in ACTOR parameters are the exact gradient; for the critic the mirror term alone is differenced."""
    rng = np.random.default_rng(7)
    oa, oc, head, batch, lowpass, mirror = _kbot_case(rng)
    for n in (oa, oc):  # lists, so that single entries can be moved
        n["cells"] = [list(c) for c in n["cells"]]
        n["input_proj"] = list(n["input_proj"])
    loss, ga, gc, aux = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass, mirror=mirror)
    loss0, ga0, gc0, aux0 = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass)
    # the auxiliary terms join the mean over (t, env) of the summed terms (ppo.py:241-244, 485-486)
    assert loss - loss0 == pytest.approx(aux["action_mirror_loss"].mean() + aux["value_mirror_loss"].mean(), rel=1e-12)
    assert aux["action_mirror_loss"].shape == batch["done"].shape and aux["action_mirror_loss"].min() > 0
    np.testing.assert_allclose(aux["raw"], aux0["raw"], atol=0)  # the first pass does not see the mirrored one
    eps = 1e-6
    f = lambda a, c: ou.recurrent_loss_and_grads(a, c, batch, CFG, head, lowpass=lowpass, mirror=mirror)  # noqa: E731
    for path, got in ((("input_proj", 0, (3, 5)), ga["input_proj"][0][3, 5]), (("input_proj", 1, (2,)), ga["input_proj"][1][2]),
                      (("cells", 0, 0, (7, 1)), ga["cells"][0][0][7, 1]), (("cells", 1, 1, (20, 3)), ga["cells"][1][1][20, 3]),
                      (("cells", 1, 2, (9,)), ga["cells"][1][2][9]), (("out_w", 0, (1, 4)), ga["out"][0][0][1, 4]),
                      (("out_w", 0, (6, 2)), ga["out"][0][0][6, 2]), (("out_b", 0, (3,)), ga["out"][0][1][3])):
        fd = (f(_bump(oa, path, eps), oc)[0] - f(_bump(oa, path, -eps), oc)[0]) / (2 * eps)
        assert got == pytest.approx(fd, rel=2e-5, abs=1e-9), path
    vm = lambda c: ou.recurrent_loss_and_grads(oa, c, batch, CFG, head, lowpass=lowpass, mirror=mirror)[3]["value_mirror_loss"].mean()  # noqa: E731
    for path, pick in ((("input_proj", 0, (1, 2)), lambda g: g["input_proj"][0][1, 2]), (("cells", 0, 1, (5, 5)), lambda g: g["cells"][0][1][5, 5]),
                       (("out_w", 0, (0, 3)), lambda g: g["out"][0][0][0, 3])):
        fd = (vm(_bump(oc, path, eps)) - vm(_bump(oc, path, -eps))) / (2 * eps)
        # the actor's mirror term does not touch the critic, so the difference of the two critic gradients is this term's
        assert pick(gc) - pick(gc0) == pytest.approx(fd, rel=2e-5, abs=1e-9), path


def test_kbot_filter_in_the_loss_is_the_numpy_scan_and_the_head_bias_moves_inside_it():
    from oracle import terms as ot

    rng = np.random.default_rng(8)
    oa, oc, head, batch, lowpass, _ = _kbot_case(rng)
    nu = batch["action"].shape[-1]
    _, _, _, plain = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head)
    _, _, _, filt = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass)
    col0, a0, cnt = lowpass["obs_bias"]
    x = plain["raw"][..., :nu] + head["mean_bias"]
    x[..., a0:a0 + cnt] += batch["actor_obs"][..., col0:col0 + cnt]
    want, _ = ot.lowpass_scan(x, lowpass["ctrl_dt"], lowpass["cutoff"], lowpass["y0"], batch["fresh"])
    np.testing.assert_allclose(filt["raw"][..., :nu], want, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(filt["raw"][..., nu:], plain["raw"][..., nu:], atol=0)


def test_mirror_terms_vanish_for_a_mirror_symmetric_recurrent_policy():
    """A policy that commutes with the mirror map (here: the map is the identity permutation with all signs +1, mirrored
    carries and filter state equal to the first pass's) must have zero mirror losses and contribute no gradient."""
    rng = np.random.default_rng(9)
    oa, oc, head, batch, lowpass, mirror = _kbot_case(rng)
    I, nu = batch["actor_obs"].shape[-1], batch["action"].shape[-1]
    ident = dict(mirror, actor_obs=(np.arange(I), np.ones(I)), critic_obs=(np.arange(I), np.ones(I)), action=(np.arange(nu), np.ones(nu)),
                 actor_carry0=oa["carry0"], critic_carry0=oc["carry0"], y0=lowpass["y0"])
    loss, ga, gc, aux = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass, mirror=ident)
    loss0, ga0, gc0, _ = ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass)
    assert np.abs(aux["action_mirror_loss"]).max() == 0 and np.abs(aux["value_mirror_loss"]).max() == 0 and loss == loss0
    np.testing.assert_allclose(ga["out"][0][0], ga0["out"][0][0], atol=1e-15)
    # and with different mirrored carries the same weights no longer agree: the carries do enter
    other = dict(ident, actor_carry0=mirror["actor_carry0"])
    assert ou.recurrent_loss_and_grads(oa, oc, batch, CFG, head, lowpass=lowpass, mirror=other)[3]["action_mirror_loss"].max() > 1e-6


def test_deviation_head_clipped_value_loss_and_filter_helpers_hand_computed():
    """The small restatements that the larger oracle functions are built from, each against numbers worked out by hand or a
    library routine."""
    from scipy.stats import norm

    # mean | raw deviation head: std = min((softplus(raw) + min_std) * var_scale, max_std), with the bias on the mean
    raw = np.array([[0.3, -0.2, 0.0, 5.0]])  # means 0.3, -0.2; raw deviations 0, 5
    a = np.array([[0.5, 0.1]])
    bias = np.array([0.1, -0.1])
    lp, ent = ou.gaussian_head(torch.tensor(raw), torch.tensor(a), 0.01, 1.0, 0.5, torch.tensor(bias))
    std = np.array([(math.log(2.0) + 0.01) * 0.5, 1.0])  # softplus(0) = ln 2; (softplus(5) + 0.01) / 2 = 2.5 capped at 1
    np.testing.assert_allclose(lp.numpy()[0], norm.logpdf(a[0], [0.4, -0.3], std), rtol=1e-12)
    np.testing.assert_allclose(ent.numpy()[0], norm.entropy(0, std), rtol=1e-12)
    # clipped value loss (ppo.py:124-135): the clip holds the new value within 0.2 of the old one before the error is taken
    got = oppo.clipped_value_loss(np.array([1.0, 1.0, 1.0]), np.array([1.5, 1.1, 0.0]), np.array([2.0, 2.0, 1.0]), 0.2)
    np.testing.assert_allclose(got, [max(0.5**2, 0.8**2), max(0.9**2, 0.9**2), max(1.0**2, 0.2**2)], rtol=1e-15)
    # the torch filter equals the closed form of a step response and restarts where flagged
    al = 0.02 / (1.0 / (2 * math.pi * 4.0) + 0.02)
    x = torch.ones(5, 1, 1, dtype=torch.float64)
    fresh = np.zeros((5, 1), bool); fresh[3] = True
    y = ou.lowpass_torch(x, 0.02, 4.0, np.zeros((1, 1)), fresh)
    y = (y[0] if isinstance(y, tuple) else y).numpy()[:, 0, 0]
    np.testing.assert_allclose(y, [1 - (1 - al) ** 1, 1 - (1 - al) ** 2, 1 - (1 - al) ** 3, al, 1 - (1 - al) ** 2], rtol=1e-13)
    # parameter lists survive the flat / unflat round trip in the optimiser's order
    p = dict(actor_w=[np.ones((2, 3))], actor_b=[np.zeros(2)], critic_w=[np.ones((1, 3)) * 2], critic_b=[np.ones(1)], log_std=np.zeros(2))
    q = ou.unflat(ou.flat(p), p)
    assert all(np.array_equal(x_, y_) for k in ("actor_w", "actor_b", "critic_w", "critic_b") for x_, y_ in zip(p[k], q[k]))
    assert np.array_equal(q["log_std"], p["log_std"])


def test_mirror_terms_of_the_mlp_policy_hand_computed():
    """A linear actor and critic on a two-entry observation that the mirror map swaps and negates: the mirrored mode and value
    follow by hand, and the terms vanish when the weights respect the symmetry."""
    obs = torch.tensor([[[1.0, 3.0]]])                       # (T = 1, b = 1, 2)
    mirror = dict(actor_obs=([1, 0], [-1.0, -1.0]), critic_obs=([1, 0], [-1.0, -1.0]), action=([1, 0], [-1.0, -1.0]),
                  actor_scale=2.0, critic_scale=0.5)
    tp = dict(actor_w=[torch.tensor([[1.0, 0.0], [0.0, 2.0]])], actor_b=[torch.zeros(2, dtype=torch.float64)],
              critic_w=[torch.tensor([[1.0, 1.0]])], critic_b=[torch.zeros(1, dtype=torch.float64)])
    tp = {k: [a.double() for a in v] for k, v in tp.items()}
    obs = obs.double()
    mean = obs @ tp["actor_w"][0].T                          # (1, 6)
    v = (obs @ tp["critic_w"][0].T)[..., 0]                  # 4
    out = ou.mirror_terms(mean, v, obs, obs, tp, mirror, "none")
    # mirrored obs (-3, -1) -> mode (-3, -2) -> mirrored back (2, 3); value of the mirrored obs -4
    np.testing.assert_allclose(out["action_mirror_loss"].numpy(), [[2.0 * ((1 - 2) ** 2 + (6 - 3) ** 2) / 2]], rtol=1e-15)
    np.testing.assert_allclose(out["value_mirror_loss"].numpy(), [[0.5 * (4 - (-4)) ** 2]], rtol=1e-15)
    tp["actor_w"] = [torch.tensor([[1.0, 0.5], [0.5, 1.0]], dtype=torch.float64)]   # commutes with the swap
    tp["critic_w"] = [torch.tensor([[1.0, -1.0]], dtype=torch.float64)]             # unchanged by swapping and negating the entries
    mean = obs @ tp["actor_w"][0].T
    v = (obs @ tp["critic_w"][0].T)[..., 0]
    out = ou.mirror_terms(mean, v, obs, obs, tp, mirror, "none")
    assert float(out["action_mirror_loss"].abs().max()) < 1e-28 and float(out["value_mirror_loss"].abs().max()) < 1e-28
