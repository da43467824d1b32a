"""numpy restatement of the reference GAE / PPO-loss arithmetic (test infrastructure).

Follows ksim/task/ppo.py:54-121 (compute_ppo_inputs), 124-135
(clipped_value_loss), 149-246 (compute_ppo_loss) and 485-486 (total loss).
All arrays are (B, T) like the reference's ``*_bt`` arguments.
"""

from __future__ import annotations

import numpy as np


def compute_ppo_inputs(
    values_bt,
    rewards_bt,
    dones_bt,
    successes_bt,
    decay_gamma: float,
    gae_lambda: float,
    normalize_advantages: bool = False,
    monte_carlo_returns: bool = False,
    dtype=np.float64,
):
    """ksim/task/ppo.py:54-121, sequential reverse scan over T."""
    v = np.asarray(values_bt, dtype=dtype)
    r = np.asarray(rewards_bt, dtype=dtype)
    done = np.asarray(dones_bt).astype(bool)
    succ = np.asarray(successes_bt).astype(bool)
    g = dtype(decay_gamma)
    lam = dtype(gae_lambda)
    one = dtype(1.0)

    # ppo.py:79 — V(s_{t+1}), last value repeated as the bootstrap.
    v_shift = np.concatenate([v[..., 1:], v[..., -1:]], axis=-1)
    # ppo.py:82-83 — 1-step bootstrap on success; rewards scaled by (1 - gamma).
    trunc = np.where(succ, one, dtype(0.0))
    rb = (one - g) * r + g * v * trunc
    # ppo.py:85-86
    mask = np.where(done, dtype(0.0), one)
    delta = rb + g * v_shift * mask - v

    T = v.shape[-1]
    ret = np.zeros_like(v)
    adv = np.zeros_like(v)
    ret_next = np.zeros(v.shape[:-1], dtype=dtype)
    adv_next = np.zeros(v.shape[:-1], dtype=dtype)
    # ppo.py:66-75,94-100 — reverse scan from zeros.
    for t in range(T - 1, -1, -1):
        ret_next = rb[..., t] + g * mask[..., t] * ret_next
        adv_next = delta[..., t] + g * lam * mask[..., t] * adv_next
        ret[..., t] = ret_next
        adv[..., t] = adv_next

    targets = ret if monte_carlo_returns else adv + v  # ppo.py:107
    out = {"advantages": adv.copy(), "value_targets": targets, "gae": adv, "returns": ret}
    if normalize_advantages:  # ppo.py:116-119 — population std over all elements, clipped >= 1e-6
        mean = adv.mean(dtype=dtype)
        std = max(adv.std(dtype=dtype), dtype(1e-6))
        out["advantages"] = (adv - mean) / std
    return out


def clipped_value_loss(target_values, values, value_targets, clip_param):
    """ksim/task/ppo.py:124-135."""
    value_clipped = target_values + np.clip(values - target_values, -clip_param, clip_param)
    clipped_error = value_clipped - value_targets
    error = values - value_targets
    return np.maximum(error**2, clipped_error**2)


def compute_ppo_loss(
    advantages_bt,
    value_targets_bt,
    on_log_probs_bta,
    on_values_bt,
    off_log_probs_bta,
    off_values_bt,
    off_entropy_bta=None,
    *,
    clip_param: float = 0.2,
    value_loss_coef: float = 0.5,
    entropy_coef: float = 0.008,
    kl_coef: float = 1e-3,
    log_clip_value: float = 5.0,
    use_clipped_value_loss: bool = True,
    kl_scale: float = 1.0,
    dtype=np.float64,
):
    """ksim/task/ppo.py:207-246 per-element terms, 473-486 total (mean over (B,T) of the sum)."""
    adv = np.asarray(advantages_bt, dtype=dtype)
    tgt = np.asarray(value_targets_bt, dtype=dtype)
    lp_on = np.asarray(on_log_probs_bta, dtype=dtype)
    lp_off = np.asarray(off_log_probs_bta, dtype=dtype)
    v_on = np.asarray(on_values_bt, dtype=dtype)
    v_off = np.asarray(off_values_bt, dtype=dtype)

    log_ratio = np.sum(lp_off - lp_on, axis=-1)
    ratio = np.exp(np.clip(log_ratio, -log_clip_value, log_clip_value))
    clipped_ratio = np.clip(ratio, 1 - clip_param, 1 + clip_param)
    policy = -np.minimum(ratio * adv, clipped_ratio * adv)

    if use_clipped_value_loss:
        value_obj = dtype(0.5) * clipped_value_loss(v_on, v_off, tgt, dtype(clip_param))
    else:
        value_obj = dtype(0.5) * (tgt - v_off) ** 2
    value = value_obj * dtype(value_loss_coef)

    kl = (lp_on - lp_off).sum(axis=-1) * dtype(kl_coef) * dtype(kl_scale)
    losses = {"policy": policy, "value": value, "kl": kl}
    if off_entropy_bta is not None:
        ent = np.asarray(off_entropy_bta, dtype=dtype)
        losses["entropy"] = -ent.sum(axis=-1) * dtype(entropy_coef)
    total = np.stack(list(losses.values()), axis=-1).sum(axis=-1).mean(dtype=dtype)
    losses["total"] = total
    return losses
