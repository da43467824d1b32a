"""Pins oracle/ppo.py against brute force, closed forms and special cases (CPU only)."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from oracle import ppo


def brute_force_gae(v, r, done, succ, g, lam):
    """O(T^2) sums: A_t = sum_k (g*lam)^(k-t) prod_{j=t}^{k-1} mask_j delta_k; R_t likewise with g."""
    B, T = v.shape
    adv = np.zeros((B, T))
    ret = np.zeros((B, T))
    for b in range(B):
        rb = [(1 - g) * r[b, t] + (g * v[b, t] if succ[b, t] else 0.0) for t in range(T)]
        m = [0.0 if done[b, t] else 1.0 for t in range(T)]
        dl = [rb[t] + g * (v[b, t + 1] if t + 1 < T else v[b, T - 1]) * m[t] - v[b, t] for t in range(T)]
        for t in range(T):
            pa, pr, sa, sr = 1.0, 1.0, 0.0, 0.0
            for k in range(t, T):
                sa += pa * dl[k]
                sr += pr * rb[k]
                pa *= g * lam * m[k]
                pr *= g * m[k]
            adv[b, t], ret[b, t] = sa, sr
    return adv, ret


def _rand(seed, B=5, T=17, p_done=0.15, p_succ=0.5):
    rng = np.random.default_rng(seed)
    v = rng.normal(size=(B, T))
    r = rng.normal(size=(B, T))
    done = rng.random((B, T)) < p_done
    succ = done & (rng.random((B, T)) < p_succ)
    return v, r, done, succ


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_gae_matches_brute_force(seed):
    v, r, done, succ = _rand(seed)
    out = ppo.compute_ppo_inputs(v, r, done, succ, 0.99, 0.95)
    adv, ret = brute_force_gae(v, r, done, succ, 0.99, 0.95)
    np.testing.assert_allclose(out["gae"], adv, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(out["returns"], ret, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(out["value_targets"], adv + v, rtol=1e-12, atol=1e-12)


def test_closed_form_constant_reward():
    # done=0, V=0, r=c  =>  R_t = c (1 - g^(T-t)); A_t = (1-g) c (1-(g lam)^(T-t)) / (1 - g lam)
    T, c, g, lam = 40, 2.5, 0.9, 0.8
    z = np.zeros((1, T))
    out = ppo.compute_ppo_inputs(z, z + c, z.astype(bool), z.astype(bool), g, lam)
    n = T - np.arange(T)
    np.testing.assert_allclose(out["returns"][0], c * (1 - g**n), rtol=1e-12)
    np.testing.assert_allclose(out["gae"][0], (1 - g) * c * (1 - (g * lam) ** n) / (1 - g * lam), rtol=1e-12)


def test_done_cuts_the_scan_and_lambda_zero():
    v, r, done, succ = _rand(3)
    done[:, 6] = True
    succ[:, 6] = False
    out = ppo.compute_ppo_inputs(v, r, done, succ, 0.97, 0.9)
    rb6 = (1 - 0.97) * r[:, 6]
    np.testing.assert_allclose(out["returns"][:, 6], rb6, rtol=1e-12)
    np.testing.assert_allclose(out["gae"][:, 6], rb6 - v[:, 6], rtol=1e-12)
    out0 = ppo.compute_ppo_inputs(v, r, done, succ, 0.97, 0.0)
    vs = np.concatenate([v[:, 1:], v[:, -1:]], axis=1)
    delta = (1 - 0.97) * r + 0.97 * v * succ + 0.97 * vs * (~done) - v
    np.testing.assert_allclose(out0["gae"], delta, rtol=1e-12, atol=1e-14)


def test_success_bootstrap_term():
    # one step, done & success: r' = (1-g) r + g V  => A = r' - V
    v = np.array([[3.0]]); r = np.array([[2.0]])
    out = ppo.compute_ppo_inputs(v, r, np.array([[True]]), np.array([[True]]), 0.9, 0.95)
    assert out["returns"][0, 0] == pytest.approx(0.1 * 2.0 + 0.9 * 3.0)
    assert out["gae"][0, 0] == pytest.approx(0.1 * 2.0 + 0.9 * 3.0 - 3.0)


def test_monte_carlo_and_normalisation():
    v, r, done, succ = _rand(4)
    out = ppo.compute_ppo_inputs(v, r, done, succ, 0.99, 0.95, normalize_advantages=True, monte_carlo_returns=True)
    np.testing.assert_array_equal(out["value_targets"], out["returns"])
    a = out["advantages"]
    assert abs(a.mean()) < 1e-12 and abs(a.std() - 1.0) < 1e-12
    np.testing.assert_allclose(a, (out["gae"] - out["gae"].mean()) / out["gae"].std(), rtol=1e-12)
    # degenerate: all-equal advantages -> std clipped at 1e-6, result 0
    z = np.zeros((2, 3))
    o = ppo.compute_ppo_inputs(z, z, z.astype(bool), z.astype(bool), 0.9, 0.9, normalize_advantages=True)
    np.testing.assert_array_equal(o["advantages"], z)


@settings(max_examples=40, deadline=None)
@given(st.integers(0, 10_000), st.integers(1, 12))
def test_segment_independence(seed, cut):
    # values/rewards after a done do not change outputs at or before it.
    v, r, done, succ = _rand(seed, B=2, T=14)
    cut = min(cut, 12)
    done[:, cut] = True
    a = ppo.compute_ppo_inputs(v, r, done, succ, 0.95, 0.9)
    v2, r2 = v.copy(), r.copy()
    v2[:, cut + 1:] += 7.0
    r2[:, cut + 1:] -= 3.0
    b = ppo.compute_ppo_inputs(v2, r2, done, succ, 0.95, 0.9)
    np.testing.assert_array_equal(a["gae"][:, : cut + 1], b["gae"][:, : cut + 1])
    np.testing.assert_array_equal(a["returns"][:, : cut + 1], b["returns"][:, : cut + 1])


def test_ppo_loss_special_cases():
    rng = np.random.default_rng(0)
    B, T, A = 3, 5, 4
    lp = rng.normal(size=(B, T, A))
    adv = rng.normal(size=(B, T))
    v = rng.normal(size=(B, T))
    tgt = rng.normal(size=(B, T))
    # identical policies: ratio = 1 -> policy = -A, kl = 0; identical values: value = 0.25 (V - tgt)^2
    out = ppo.compute_ppo_loss(adv, tgt, lp, v, lp, v)
    np.testing.assert_allclose(out["policy"], -adv, rtol=1e-12)
    np.testing.assert_array_equal(out["kl"], np.zeros((B, T)))
    np.testing.assert_allclose(out["value"], 0.5 * 0.5 * (v - tgt) ** 2, rtol=1e-12)
    assert out["total"] == pytest.approx((out["policy"] + out["value"]).mean())
    # A > 0 and ratio > 1.2 -> clipped branch -1.2 A ; A < 0 and ratio > 1.2 -> unclipped -ratio A
    lp_new = lp.copy(); lp_new[..., 0] += 0.5
    out = ppo.compute_ppo_loss(np.abs(adv), tgt, lp, v, lp_new, v)
    np.testing.assert_allclose(out["policy"], -1.2 * np.abs(adv), rtol=1e-12)
    out = ppo.compute_ppo_loss(-np.abs(adv), tgt, lp, v, lp_new, v)
    np.testing.assert_allclose(out["policy"], np.exp(0.5) * np.abs(adv), rtol=1e-12)
    np.testing.assert_allclose(out["kl"], -0.5 * 1e-3 * np.ones((B, T)), rtol=1e-12)
    # log-ratio clip at +-5
    lp_big = lp.copy(); lp_big[..., 0] += 50.0
    out = ppo.compute_ppo_loss(-np.abs(adv), tgt, lp, v, lp_big, v)
    np.testing.assert_allclose(out["policy"], np.exp(5.0) * np.abs(adv), rtol=1e-12)
    # value clip: |V - V_old| <= clip -> plain squared error; beyond -> max of the two errors
    v_new = v + 0.1
    out = ppo.compute_ppo_loss(adv, tgt, lp, v, lp, v_new)
    np.testing.assert_allclose(out["value"], 0.25 * (v_new - tgt) ** 2, rtol=1e-12)
    v_new = v + 1.0
    out = ppo.compute_ppo_loss(adv, tgt, lp, v, lp, v_new)
    np.testing.assert_allclose(out["value"], 0.25 * np.maximum((v_new - tgt) ** 2, (v + 0.2 - tgt) ** 2), rtol=1e-12)
    # entropy term
    ent = rng.random((B, T, A))
    out = ppo.compute_ppo_loss(adv, tgt, lp, v, lp, v, ent)
    np.testing.assert_allclose(out["entropy"], -0.008 * ent.sum(-1), rtol=1e-12)
