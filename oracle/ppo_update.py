"""TEST INFRASTRUCTURE: float64 restatement of the PPO policy update for an MLP actor / critic with a Gaussian head.

Follows ksim/task/ppo.py:412-492 (`_get_ppo_loss_and_metrics`: forward, GAE as a constant, loss, mean),
495-565 (`_single_step`: gradient, optimiser, adaptive KL), 572-694 (`update_model`: on-policy variables once,
passes x minibatches) and the optax chain of examples/walking.py:373-387.  The gradient is taken by torch's
CPU autograd in float64 (the library routine the hand-written backward pass is checked against); the loss written
here in torch is pinned against the numpy restatement in oracle/ppo.py by tests/test_oracle_ppo_update.py.
Distribution formulas (xax.Normal, not in the reference tree): log N(a; mu, sigma) per action and the Gaussian
entropy 0.5 + 0.5 log(2 pi) + log sigma.  Only tests may import this module.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

from . import ppo as oppo

_ACT = {"elu": F.elu, "relu": F.relu, "tanh": torch.tanh, "none": lambda t: t,
        "gelu": lambda t: F.gelu(t, approximate="tanh")}  # jax.nn.gelu's default form


def mlp(x, ws, bs, act="elu"):
    h = x
    for i, (w, b) in enumerate(zip(ws, bs)):
        h = F.linear(h, w, b)
        if i + 1 < len(ws):
            h = _ACT[act](h)
    return h


def gaussian(mean, log_std, action):
    z = (action - mean) * torch.exp(-log_std)
    lp = -0.5 * z * z - log_std - 0.5 * math.log(2 * math.pi)
    ent = (0.5 + 0.5 * math.log(2 * math.pi) + log_std).expand_as(mean)
    return lp, ent


def gaussian_head(raw, action, min_std, max_std, var_scale, mean_bias=None):
    """Log-density and entropy per action for the mean | raw deviation head (examples/kbot/train.py:915-932):
    std = min((softplus(raw_std) + min_std) * var_scale, max_std)."""
    nu = raw.shape[-1] // 2
    mean = raw[..., :nu] + (0.0 if mean_bias is None else mean_bias)
    std = torch.clamp((F.softplus(raw[..., nu:]) + min_std) * var_scale, max=max_std)
    return gaussian(mean, torch.log(std), action)


def mixture_head(raw, action, num_mixtures, min_std, max_std, var_scale, mean_bias=None, clip_lo=None, clip_hi=None):
    """Log-density per action of the mixture-of-Gaussians head (examples/walking.py:127-144) and the upper bound
    sum_k pi_k H_k + H(pi) of its entropy (a mixture's entropy has no closed form; xax's own choice is unpinned)."""
    K = num_mixtures
    nu = raw.shape[-1] // (3 * K)
    lead = raw.shape[:-1]
    mean = raw[..., : nu * K].reshape(*lead, nu, K)
    if mean_bias is not None:
        mean = mean + mean_bias[..., None]
    if clip_lo is not None:
        mean = torch.maximum(torch.minimum(mean, clip_hi[..., None]), clip_lo[..., None])
    std = torch.clamp((F.softplus(raw[..., nu * K: 2 * nu * K].reshape(*lead, nu, K)) + min_std) * var_scale, max=max_std)
    logw = torch.log_softmax(raw[..., 2 * nu * K:].reshape(*lead, nu, K), dim=-1)
    z = (action[..., None] - mean) / std
    lp = torch.logsumexp(logw - 0.5 * z * z - torch.log(std) - 0.5 * math.log(2 * math.pi), dim=-1)
    ent = (torch.exp(logw) * (0.5 + 0.5 * math.log(2 * math.pi) + torch.log(std) - logw)).sum(-1)
    return lp, ent


def ppo_loss_torch(adv, tgt, on_lp, on_v, lp, v, ent, cfg, kl_scale=1.0):
    """ppo.py:207-246 per element and 485-486 total, in torch so that autograd can differentiate it."""
    log_ratio = (lp - on_lp).sum(-1)
    ratio = torch.exp(torch.clamp(log_ratio, -cfg["log_clip_value"], cfg["log_clip_value"]))
    clipped = torch.clamp(ratio, 1 - cfg["clip_param"], 1 + cfg["clip_param"])
    policy = -torch.minimum(ratio * adv, clipped * adv)
    if cfg["use_clipped_value_loss"]:
        vc = on_v + torch.clamp(v - on_v, -cfg["clip_param"], cfg["clip_param"])
        value = 0.5 * torch.maximum((v - tgt) ** 2, (vc - tgt) ** 2)
    else:
        value = 0.5 * (tgt - v) ** 2
    value = value * cfg["value_loss_coef"]
    kl = (on_lp - lp).sum(-1) * cfg["kl_coef"] * kl_scale
    entropy = -ent.sum(-1) * cfg["entropy_coef"]
    return (policy + value + kl + entropy).mean(), {"policy": policy, "value": value, "kl": kl, "entropy": entropy}


def mirror_terms(mean, v, actor_obs, critic_obs, tp, mirror, act):
    """The K-Bot task's mirror losses per transition (examples/kbot/train.py:1458-1477): the actor's mode against the
    mirrored-back mode on the mirrored observation, and the value against the value of the mirrored observation.
    mirror: dict(actor_obs=(perm, sign), critic_obs=(perm, sign), action=(perm, sign), actor_scale, critic_scale) with
    mirrored[j] = sign[j] x[perm[j]]."""
    def m(x, key):
        perm, sign = mirror[key]
        return x[..., list(perm)] * torch.tensor(np.asarray(sign, dtype=np.float64))
    out = {}
    if mirror.get("actor_scale", 0.0):
        mean_m = mlp(m(actor_obs, "actor_obs"), tp["actor_w"], tp["actor_b"], act)
        out["action_mirror_loss"] = ((mean - m(mean_m, "action")) ** 2).mean(-1) * mirror["actor_scale"]
    if mirror.get("critic_scale", 0.0):
        v_m = mlp(m(critic_obs, "critic_obs"), tp["critic_w"], tp["critic_b"], act)[..., 0]
        out["value_mirror_loss"] = (v - v_m) ** 2 * mirror["critic_scale"]
    return out


def loss_and_grads(params, batch, cfg, kl_scale=1.0, act="elu", mirror=None):
    """params: dict(actor_w, actor_b, critic_w, critic_b: lists of float64 arrays; log_std).  batch: (T, b, ...) arrays.
    `mirror`: see mirror_terms; its terms join the loss like any auxiliary loss (ppo.py:241-244).
    Returns (loss, grads with the structure of params, aux)."""
    tp = {k: ([torch.tensor(np.asarray(a, dtype=np.float64), requires_grad=True) for a in v] if isinstance(v, list)
              else torch.tensor(np.asarray(v, dtype=np.float64), requires_grad=True)) for k, v in params.items()}
    t64 = lambda a: torch.tensor(np.asarray(a, dtype=np.float64))  # noqa: E731
    Tn, b = batch["done"].shape
    mean = mlp(t64(batch["actor_obs"]), tp["actor_w"], tp["actor_b"], act)
    v = mlp(t64(batch["critic_obs"]), tp["critic_w"], tp["critic_b"], act)[..., 0]
    lp, ent = gaussian(mean, tp["log_std"], t64(batch["action"]))
    # GAE on (B, T) arrays with the current values, as a constant (ppo.py:121 stop_gradient)
    gi = oppo.compute_ppo_inputs(v.detach().numpy().T, np.asarray(batch["rewards"], np.float64).T, np.asarray(batch["done"]).T,
                                 np.asarray(batch["success"]).T, cfg["gamma"], cfg["lam"], cfg["normalize_advantages"],
                                 cfg["monte_carlo_returns"], np.float64)
    adv, tgt = t64(gi["advantages"].T), t64(gi["value_targets"].T)
    loss, terms = ppo_loss_torch(adv, tgt, t64(batch["on_log_probs"]), t64(batch["on_values"]), lp, v, ent, cfg, kl_scale)
    if mirror:
        extra = mirror_terms(mean, v, t64(batch["actor_obs"]), t64(batch["critic_obs"]), tp, mirror, act)
        for name, term in extra.items():
            loss = loss + term.mean()
            terms[name] = term
    loss.backward()
    grads = {k: ([a.grad.numpy() for a in v] if isinstance(v, list) else v.grad.numpy()) for k, v in tp.items()}
    aux = {"mean": mean.detach().numpy(), "values": v.detach().numpy(), "log_probs": lp.detach().numpy(),
           "advantages": adv.numpy(), "value_targets": tgt.numpy(), "terms": {k: t.detach().numpy() for k, t in terms.items()}}
    return float(loss.detach()), grads, aux


def flat(tree):
    out = []
    for k in ("actor_w", "actor_b", "critic_w", "critic_b"):
        out += list(tree[k])
    return out + [tree["log_std"]]


def optax_chain_step(params, grads, m1, m2, step, cfg):
    """zero_nans -> clip_by_global_norm -> add_decayed_weights -> scale_by_adam -> lr -> -1 (examples/walking.py:380-387;
    optax: clip scales by max_norm / norm when norm > max_norm; Adam with bias correction, eps outside the root)."""
    g = [np.nan_to_num(np.asarray(x, np.float64), nan=0.0, posinf=np.inf, neginf=-np.inf) for x in grads]
    norm = math.sqrt(sum(float((x * x).sum()) for x in g))
    if cfg["grad_clip"] > 0 and norm > cfg["grad_clip"]:
        g = [x / norm * cfg["grad_clip"] for x in g]
    new_p, new_m1, new_m2 = [], [], []
    for p, x, a, b in zip(params, g, m1, m2):
        x = x + cfg["adam_weight_decay"] * p
        a = cfg["adam_b1"] * a + (1 - cfg["adam_b1"]) * x
        b = cfg["adam_b2"] * b + (1 - cfg["adam_b2"]) * x * x
        ah, bh = a / (1 - cfg["adam_b1"] ** step), b / (1 - cfg["adam_b2"] ** step)
        new_p.append(p - cfg["learning_rate"] * ah / (np.sqrt(bh) + cfg["adam_eps"]))
        new_m1.append(a)
        new_m2.append(b)
    return new_p, new_m1, new_m2, norm


def unflat(vals, like):
    it = iter(vals)
    out = {}
    for k in ("actor_w", "actor_b", "critic_w", "critic_b"):
        out[k] = [next(it) for _ in like[k]]
    out["log_std"] = next(it)
    return out


def update_model(params, rollout, cfg, permutations, act="elu"):
    """ppo.py:572-694 with explicit minibatch permutations.  rollout arrays are (T, N, ...)."""
    params = {k: ([np.asarray(a, np.float64) for a in v] if isinstance(v, list) else np.asarray(v, np.float64)) for k, v in params.items()}
    t64 = lambda a: torch.tensor(np.asarray(a, dtype=np.float64))  # noqa: E731
    with torch.no_grad():
        tw = lambda k: [t64(a) for a in params[k]]  # noqa: E731
        mean = mlp(t64(rollout["actor_obs"]), tw("actor_w"), tw("actor_b"), act)
        on_v = mlp(t64(rollout["critic_obs"]), tw("critic_w"), tw("critic_b"), act)[..., 0].numpy()
        on_lp = gaussian(mean, t64(params["log_std"]), t64(rollout["action"]))[0].numpy()
    m1 = [np.zeros_like(x) for x in flat(params)]
    m2 = [np.zeros_like(x) for x in flat(params)]
    step, losses = 0, []
    N = rollout["done"].shape[1]
    bs = min(cfg["batch_size"], N)
    for perm in permutations:
        for idx in np.asarray(perm).reshape(-1, bs):
            batch = {k: np.asarray(v)[:, idx] for k, v in rollout.items()}
            batch["on_log_probs"], batch["on_values"] = on_lp[:, idx], on_v[:, idx]
            loss, grads, _ = loss_and_grads(params, batch, cfg, 1.0, act)
            step += 1
            new_p, m1, m2, _ = optax_chain_step(flat(params), flat(grads), m1, m2, step, cfg)
            params = unflat(new_p, params)
            losses.append(loss)
    return params, losses


def lowpass_torch(x, ctrl_dt, fc, y0, fresh):
    """ksim.lowpass_one_pole (ksim/actions.py:248-257) threaded through time on torch tensors, x (T, b, n): the state is y0
    before the first step and zero at the steps flagged fresh (the model carry was replaced by the initial one after a
    done step, examples/kbot/train.py:1529-1533)."""
    alpha = ctrl_dt / (1.0 / (2.0 * math.pi * fc) + ctrl_dt)
    last = torch.tensor(np.asarray(y0, dtype=np.float64))
    out = []
    for t in range(x.shape[0]):
        keep = torch.tensor(1.0 - np.asarray(fresh[t], dtype=np.float64))[:, None]
        last = last * keep
        last = last + alpha * (x[t] - last)
        out.append(last)
    return torch.stack(out)


def recurrent_loss_and_grads(actor, critic, batch, cfg, head, act="none", lowpass=None, mirror=None):
    """The minibatch loss of PPOTask for a recurrent actor with the mean | raw deviation head and a recurrent critic
    (ppo.py:412-492 with the scan over time), and its gradients by float64 reverse-mode differentiation.
    actor / critic: dict(input_proj, cells, out_w, out_b, carry0); batch: (T, b, ...) arrays with `fresh`; head:
    dict(min_std, max_std, var_scale, mean_bias).

    `lowpass`: dict(ctrl_dt, cutoff, y0 (b, nu), optional obs_bias=(first obs column, first action, count)): the biased
    means pass ksim.lowpass_one_pole before they become the distribution's location (examples/kbot/train.py:917-932; the
    command-dependent bias of train.py:920-921 is read from the observation row), the filter state riding in the carry.
    `mirror`: dict(actor_obs=(perm, sign), critic_obs=(perm, sign), action=(perm, sign), actor_scale, critic_scale,
    actor_carry0, critic_carry0, y0): both networks run a second time on the mirrored observations from their own mirrored
    carries (and the actor's mirrored filter state); the squared differences of the modes (mirrored back) and of the values
    join the loss as auxiliary terms (train.py:1458-1496, ppo.py:241-244).
    Returns (loss, actor gradients, critic gradients, aux)."""
    from . import recurrent as orec

    pa = orec.torch_parameters(actor["input_proj"], actor["cells"], actor["out_w"], actor["out_b"])
    pc = orec.torch_parameters(critic["input_proj"], critic["cells"], critic["out_w"], critic["out_b"])
    bias = None if head.get("mean_bias") is None else torch.tensor(np.asarray(head["mean_bias"], dtype=np.float64))
    nu = np.asarray(batch["action"]).shape[-1]

    def run_actor(obs, carry0, y0):
        """raw (T, b, 2 nu) with the location (biased, filtered when asked) in the first half; with a filter the head's own
        bias is spent."""
        raw = orec.torch_sequence(obs, carry0, batch["fresh"], *pa, act=act)
        if lowpass is None:
            return raw, bias
        mean = raw[..., :nu] + (0.0 if bias is None else bias)
        if lowpass.get("obs_bias") is not None:
            col0, a0, cnt = lowpass["obs_bias"]
            extra = torch.zeros_like(mean)
            extra[..., a0:a0 + cnt] = torch.tensor(np.asarray(obs, dtype=np.float64)[..., col0:col0 + cnt])
            mean = mean + extra
        mean = lowpass_torch(mean, lowpass["ctrl_dt"], lowpass["cutoff"], y0, batch["fresh"])
        return torch.cat([mean, raw[..., nu:]], dim=-1), None

    raw, head_bias = run_actor(batch["actor_obs"], actor["carry0"], None if lowpass is None else lowpass["y0"])
    v = orec.torch_sequence(batch["critic_obs"], critic["carry0"], batch["fresh"], *pc, act=act)[..., 0]
    # GAE from the current values, as a constant (ppo.py:450-459); the oracle works on (B, T)
    gae = oppo.compute_ppo_inputs(v.detach().numpy().T, batch["rewards"].T, batch["done"].T, batch["success"].T, cfg["gamma"],
                                  cfg["lam"], normalize_advantages=cfg["normalize_advantages"],
                                  monte_carlo_returns=cfg["monte_carlo_returns"])
    adv, tgt = torch.tensor(gae["advantages"].T.copy()), torch.tensor(gae["value_targets"].T.copy())
    lp, ent = gaussian_head(raw, torch.tensor(np.asarray(batch["action"], dtype=np.float64)), head["min_std"], head["max_std"],
                            head["var_scale"], head_bias)
    loss, _ = ppo_loss_torch(adv, tgt, torch.tensor(batch["on_log_probs"]), torch.tensor(batch["on_values"]), lp, v, ent, cfg)
    aux = {}
    if mirror:
        def m(x, key):
            perm, sign = mirror[key]
            return x[..., list(perm)] * np.asarray(sign, dtype=np.float64)

        if mirror.get("actor_scale", 0.0):
            raw_m, bias_m = run_actor(m(np.asarray(batch["actor_obs"], dtype=np.float64), "actor_obs"), mirror["actor_carry0"],
                                      mirror.get("y0"))
            mode = raw[..., :nu] + (0.0 if head_bias is None else head_bias)
            mode_m = raw_m[..., :nu] + (0.0 if bias_m is None else bias_m)
            perm, sign = mirror["action"]
            back = mode_m[..., list(perm)] * torch.tensor(np.asarray(sign, dtype=np.float64))
            term = ((mode - back) ** 2).mean(-1) * mirror["actor_scale"]  # train.py:1466-1469
            loss = loss + term.mean()
            aux["action_mirror_loss"] = term.detach().numpy()
            aux["raw_mirror"] = raw_m.detach().numpy()
        if mirror.get("critic_scale", 0.0):
            v_m = orec.torch_sequence(m(np.asarray(batch["critic_obs"], dtype=np.float64), "critic_obs"), mirror["critic_carry0"],
                                      batch["fresh"], *pc, act=act)[..., 0]
            term = (v - v_m) ** 2 * mirror["critic_scale"]  # train.py:1477
            loss = loss + term.mean()
            aux["value_mirror_loss"] = term.detach().numpy()
    loss.backward()
    aux.update({"raw": raw.detach().numpy(), "values": v.detach().numpy()})
    return float(loss.detach()), orec.parameter_gradients(pa), orec.parameter_gradients(pc), aux
