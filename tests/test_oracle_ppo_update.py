"""Pins the torch restatement of the PPO loss (used for autograd) and the optimiser chain of oracle/ppo_update.py."""
import math

import numpy as np
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
