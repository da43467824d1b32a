"""Parity of the HIP GAE / PPO-loss / reward kernels against the oracle (through the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import ppo as oppo
from oracle import terms as oterms

pytestmark = pytest.mark.gpu

GAE_TOL = 1e-5  # benchmark tolerance for GAE and returns (relative to the array's max magnitude)


def _inputs(seed, B, T, p_done=0.01, p_succ=0.3):
    rng = np.random.default_rng(seed)
    v = rng.normal(size=(B, T)).astype(np.float32)
    r = rng.normal(size=(B, T)).astype(np.float32)
    done = rng.random((B, T)) < p_done
    succ = done & (rng.random((B, T)) < p_succ)
    return v, r, done, succ


def _close(got, want, tol=GAE_TOL):
    want = np.asarray(want, dtype=np.float64)
    got = got.detach().cpu().numpy().astype(np.float64)
    scale = max(1.0, np.abs(want).max())
    err = np.abs(got - want).max() / scale
    assert err <= tol, f"max rel err {err:.3e} > {tol}"


@pytest.mark.parametrize("B,T", [(1, 1), (3, 5), (7, 63), (5, 64), (5, 65), (33, 128), (9, 200), (4096, 128)])
@pytest.mark.parametrize("time_major", [False, True])
def test_gae_parity(B, T, time_major):
    from ksim_amd import ppo

    v, r, done, succ = _inputs(B * 1000 + T, B, T, p_done=0.05 if B < 4096 else 0.01)
    want = oppo.compute_ppo_inputs(v, r, done, succ, 0.99, 0.95)
    tr = (lambda a: np.ascontiguousarray(a.T)) if time_major else (lambda a: a)
    dev = "cuda:0"
    out = ppo.compute_ppo_inputs(torch.from_numpy(tr(v)).to(dev), torch.from_numpy(tr(r)).to(dev),
                                 torch.from_numpy(tr(done)).to(dev), torch.from_numpy(tr(succ)).to(dev), 0.99, 0.95,
                                 time_major=time_major)
    back = (lambda t: t.T) if time_major else (lambda t: t)
    _close(back(out.gae_bt), want["gae"])
    _close(back(out.returns_bt), want["returns"])
    _close(back(out.value_targets_bt), want["value_targets"])


def test_gae_options_and_dtypes():
    from ksim_amd import ppo

    v, r, done, succ = _inputs(5, 64, 100, p_done=0.1)
    dev = "cuda:0"
    want = oppo.compute_ppo_inputs(v, r, done, succ, 0.97, 0.9, normalize_advantages=True, monte_carlo_returns=True)
    out = ppo.compute_ppo_inputs(torch.from_numpy(v).to(dev), torch.from_numpy(r).to(dev),
                                 torch.from_numpy(done.astype(np.int8)).to(dev),
                                 torch.from_numpy(succ.astype(np.uint8)).to(dev), 0.97, 0.9,
                                 normalize_advantages=True, monte_carlo_returns=True)
    _close(out.value_targets_bt, want["returns"])
    _close(out.advantages_bt, want["advantages"])
    # successes=None is all-false
    want = oppo.compute_ppo_inputs(v, r, done, np.zeros_like(done), 0.97, 0.9)
    out = ppo.compute_ppo_inputs(torch.from_numpy(v).to(dev), torch.from_numpy(r).to(dev),
                                 torch.from_numpy(done).to(dev), None, 0.97, 0.9)
    _close(out.gae_bt, want["gae"])


def test_gae_empty_and_errors():
    from ksim_amd import _lib, ppo

    dev = "cuda:0"
    e = torch.empty((0, 8), device=dev)
    out = ppo.compute_ppo_inputs(e, e, torch.empty((0, 8), dtype=torch.bool, device=dev), None, 0.9, 0.9)
    assert out.gae_bt.shape == (0, 8)
    with pytest.raises(_lib.KsError):
        ppo.compute_ppo_inputs(torch.zeros(4, 4), torch.zeros(4, 4), torch.zeros(4, 4, dtype=torch.bool), None, 0.9, 0.9)
    with pytest.raises(_lib.KsError):
        ppo.compute_ppo_inputs(torch.zeros(4, 4, device=dev), torch.zeros(4, 5, device=dev),
                               torch.zeros(4, 4, dtype=torch.bool, device=dev), None, 0.9, 0.9)


def test_gae_full_size_properties():
    """cfg-2 size: segment independence and the closed form, checked on device without the oracle."""
    from ksim_amd import ppo

    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(2)
    B, T = 4096, 128
    v = torch.randn(B, T, device=dev, generator=g)
    r = torch.randn(B, T, device=dev, generator=g)
    done = torch.rand(B, T, device=dev, generator=g) < 0.01
    done[:, 70] = True
    a = ppo.compute_ppo_inputs(v, r, done, None, 0.99, 0.95)
    v2, r2 = v.clone(), r.clone()
    v2[:, 71:] += 3.0
    r2[:, 71:] -= 2.0
    b = ppo.compute_ppo_inputs(v2, r2, done, None, 0.99, 0.95)
    assert torch.equal(a.gae_bt[:, :71], b.gae_bt[:, :71]) and torch.equal(a.returns_bt[:, :71], b.returns_bt[:, :71])
    z = torch.zeros(B, T, device=dev)
    c = ppo.compute_ppo_inputs(z, z + 2.0, torch.zeros(B, T, dtype=torch.bool, device=dev), None, 0.99, 0.95)
    n = (T - torch.arange(T, device=dev)).double()
    assert torch.allclose(c.returns_bt.double(), (2.0 * (1 - 0.99**n)).expand(B, T), rtol=2e-6, atol=1e-6)
    # linearity in (r, v) for a fixed mask
    s = ppo.compute_ppo_inputs(v + v2, r + r2, done, None, 0.99, 0.95)
    assert torch.allclose(s.gae_bt, a.gae_bt + b.gae_bt, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("B,T,A,with_entropy", [(4, 7, 1, False), (16, 24, 21, True), (4096, 128, 1, False)])
def test_ppo_loss_parity(B, T, A, with_entropy):
    from ksim_amd import ppo

    rng = np.random.default_rng(B + T + A)
    lp_on = rng.normal(size=(B, T, A)).astype(np.float32)
    lp_off = (lp_on + rng.normal(scale=0.05 if A == 1 else 0.2, size=(B, T, A))).astype(np.float32)
    v_on = rng.normal(size=(B, T)).astype(np.float32)
    v_off = (v_on + rng.normal(scale=0.3, size=(B, T))).astype(np.float32)
    adv = rng.normal(size=(B, T)).astype(np.float32)
    tgt = rng.normal(size=(B, T)).astype(np.float32)
    ent = rng.random((B, T, A)).astype(np.float32) if with_entropy else None
    want = oppo.compute_ppo_loss(adv, tgt, lp_on, v_on, lp_off, v_off, ent)
    dev = "cuda:0"
    t = lambda a: None if a is None else torch.from_numpy(a).to(dev)
    z = torch.zeros(B, T, device=dev)
    out = ppo.compute_ppo_loss(ppo.PPOInputs(t(adv), t(tgt), z, z), ppo.PPOVariables(t(lp_on), t(v_on)),
                               ppo.PPOVariables(t(lp_off), t(v_off), entropy=t(ent)))
    for k in ("policy", "value", "kl") + (("entropy",) if with_entropy else ()):
        _close(out[k], want[k])
    assert abs(out["total"].item() - want["total"]) <= 1e-5 * max(1.0, abs(want["total"]))


def test_reward_total_and_done_success():
    from ksim_amd import terms

    rng = np.random.default_rng(0)
    n, K, k = 1000, 5, 3
    comps = rng.normal(size=(K, n)).astype(np.float32)
    scales = [1.0, -0.5, 2.0, 0.01, -3.0]
    tvals = rng.integers(-1, 2, size=(k, n)).astype(np.int8)
    dev = "cuda:0"
    total, done, succ = terms.reward_total_and_done(torch.from_numpy(comps).to(dev), scales,
                                                    torch.from_numpy(tvals).to(dev), clip_min=-2.0, clip_max=None)
    want = np.maximum(sum(comps[j].astype(np.float64) * scales[j] for j in range(K)), -2.0)
    _close(total, want, 1e-6)
    wd, ws = oterms.combine_terminations([tvals[j] for j in range(k)])
    assert np.array_equal(done.cpu().numpy().astype(bool), wd)  # bit-exact masks
    assert np.array_equal(succ.cpu().numpy().astype(bool), ws)
