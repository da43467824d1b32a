"""Policy update of a PPO iteration (ksim/task/ppo.py:495-565 `_single_step`, 572-694 `update_model`) for an MLP
actor / critic with a state-independent Gaussian head.

The reference differentiates `_get_ppo_loss_and_metrics` (ppo.py:412-492) with `jax.grad` and applies the task's
optax chain; here the same gradient is written out: the loss gradient w.r.t. the policy outputs
(`ks_ppo_loss_grad`), the networks' backward passes (`ks_mlp_train_backward`, three MFMA GEMMs per layer) and the
optimiser chain of the examples (`ks_mlp_adam_step`).  As in the reference, GAE is recomputed from the current
value estimates at every minibatch step and enters the loss as a constant.
Trajectories are time-major (T, N, ...), the rollout buffers' own layout; a minibatch is a set of env columns.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Sequence

import torch

from . import _lib
from . import _lib_terms as T
from . import ppo as ppo_mod
from .actions import LowPass
from .mlp import MLP


@dataclass
class PPOUpdateConfig:  # ksim/task/ppo.py:254-311 defaults, examples/walking.py:373-387 optimiser
    gamma: float = 0.99
    lam: float = 0.95
    normalize_advantages: bool = True
    monte_carlo_returns: bool = False
    clip_param: float = 0.2
    value_loss_coef: float = 0.5
    entropy_coef: float = 0.008
    kl_coef: float = 1e-3
    log_clip_value: float = 5.0
    use_clipped_value_loss: bool = True
    adaptive_kl: bool = False
    desired_kl: float = 0.01
    num_passes: int = 1
    batch_size: int = 256          # envs per minibatch
    learning_rate: float = 3e-4
    adam_b1: float = 0.9
    adam_b2: float = 0.999
    adam_eps: float = 1e-8
    adam_weight_decay: float = 0.0
    grad_clip: float = 2.0
    actor_mirror_loss_scale: float = 0.0   # examples/kbot/train.py:117-124
    critic_mirror_loss_scale: float = 0.0


@dataclass
class MirrorSpec:
    """Left / right mirror maps of a task as signed permutations (examples/kbot/train.py:1565-1760: mirror_joints, mirror_obs
    and mirror_cmd reorder and negate entries): mirrored[j] = sign[j] * x[perm[j]] for the actor's observation row, the
    critic's observation row and the action vector."""
    actor_obs_perm: Sequence[int]
    actor_obs_sign: Sequence[float]
    critic_obs_perm: Sequence[int]
    critic_obs_sign: Sequence[float]
    action_perm: Sequence[int]
    action_sign: Sequence[float]
    _dev: dict = field(default_factory=dict, repr=False)

    def __post_init__(self):
        for name in ("actor_obs", "critic_obs", "action"):
            perm, sign = list(getattr(self, name + "_perm")), list(getattr(self, name + "_sign"))
            if sorted(perm) != list(range(len(perm))) or len(sign) != len(perm):
                raise ValueError(f"{name}: the mirror map must be a permutation with one sign per entry")

    def device(self, name: str, dev) -> tuple[torch.Tensor, torch.Tensor]:
        """(perm int32, sign float32) of one of the maps on `dev`; "value" is the critic output's own map, one entry kept
        as it is.  Cached per (map, device)."""
        key = (name, str(torch.device(dev)))
        if key not in self._dev:
            perm, sign = ([0], [1.0]) if name == "value" else (list(getattr(self, name + "_perm")), list(getattr(self, name + "_sign")))
            self._dev[key] = (torch.tensor(perm, dtype=torch.int32, device=dev), torch.tensor(sign, dtype=torch.float32, device=dev))
        return self._dev[key]


def kbot_mirror_joints() -> tuple[list[int], list[float]]:
    """mirror_joints of the K-Bot example (examples/kbot/train.py:1565-1573) as (perm, sign): the legs swap, the arm blocks
    keep their places, every joint is negated."""
    return list(range(5, 10)) + list(range(0, 5)) + list(range(10, 20)), [-1.0] * 20


@dataclass
class GaussianMlpPolicy:
    """Actor (obs -> action means), critic (obs -> value) and one log standard deviation per action."""
    actor: MLP
    critic: MLP
    log_std: torch.Tensor
    opt_step: int = 0
    kl_scale: torch.Tensor | None = None  # adaptive KL: current coefficient / cfg.kl_coef, one device float
    mirror: MirrorSpec | None = None      # the task's symmetry, for the mirror losses
    _m1: torch.Tensor | None = field(default=None, repr=False)
    _m2: torch.Tensor | None = field(default=None, repr=False)

    def kl_coef(self, cfg: "PPOUpdateConfig") -> float:
        """The current KL coefficient (reads the device scalar: for logging, not for the update loop)."""
        return cfg.kl_coef * (float(self.kl_scale.item()) if self.kl_scale is not None else 1.0)

    def train_init(self) -> None:
        self.actor.train_init()
        self.critic.train_init()
        self._m1, self._m2 = torch.zeros_like(self.log_std), torch.zeros_like(self.log_std)


def get_ppo_variables(policy: GaussianMlpPolicy, actor_obs: torch.Tensor, critic_obs: torch.Tensor,
                      action: torch.Tensor, train: bool = False):
    """log-probabilities (rows, nu), values (rows), entropy (rows, nu) and the means, for flattened rows."""
    lib = _lib.load()
    mean = policy.actor.train_forward(actor_obs) if train else policy.actor(actor_obs)
    value = (policy.critic.train_forward(critic_obs) if train else policy.critic(critic_obs)).reshape(-1)
    lp, ent = torch.empty_like(mean), torch.empty_like(mean)
    _lib.check(lib.ks_gaussian_log_prob(_lib.current_stream(), mean.shape[0], mean.shape[1], _lib.ptr(mean),
                                        _lib.ptr(policy.log_std), _lib.ptr(action), _lib.ptr(lp), _lib.ptr(ent)))
    return lp, value, ent, mean


def _adam(cfg: PPOUpdateConfig, step: int) -> T.KsAdamParams:
    return T.KsAdamParams(cfg.learning_rate, cfg.adam_b1, cfg.adam_b2, cfg.adam_eps, cfg.adam_weight_decay,
                          cfg.grad_clip, step)


def single_step(policy: GaussianMlpPolicy, cfg: PPOUpdateConfig, actor_obs, critic_obs, action, rewards, done, success,
                on_log_probs, on_values) -> dict:
    """One minibatch step (ppo.py:495-565): arrays are (T, b, ...) time-major slices of the rollout."""
    lib = _lib.load()
    Tn, b = done.shape
    rows = Tn * b
    nu = action.shape[-1]
    a_obs, c_obs, act = actor_obs.reshape(rows, -1), critic_obs.reshape(rows, -1), action.reshape(rows, nu)
    # Mirror losses (examples/kbot/train.py:1458-1477): each network also runs on the mirrored rows.  Both passes share the
    # weights, so the mirrored rows ride in the same forward and backward pass as rows [rows, 2 rows).
    mirror_a = cfg.actor_mirror_loss_scale != 0.0
    mirror_c = cfg.critic_mirror_loss_scale != 0.0
    if (mirror_a or mirror_c) and policy.mirror is None:
        raise _lib.KsError("mirror loss scales are set but the policy has no MirrorSpec")
    st = _lib.current_stream()

    def with_mirrored(x, name):
        perm, sign = policy.mirror.device(name, x.device)
        if perm.numel() != x.shape[1]:
            raise _lib.KsError(f"the {name} mirror map has {perm.numel()} entries, the rows have {x.shape[1]}")
        both = torch.empty(2 * rows, x.shape[1], dtype=torch.float32, device=x.device)
        both[:rows].copy_(x)
        _lib.check(lib.ks_signed_permute(st, rows, x.shape[1], _lib.ptr(both[:rows]), _lib.ptr(perm), _lib.ptr(sign), _lib.ptr(both[rows:])))
        return both

    a_in = with_mirrored(a_obs, "actor_obs") if mirror_a else a_obs
    c_in = with_mirrored(c_obs, "critic_obs") if mirror_c else c_obs
    mean_all = policy.actor.train_forward(a_in)
    value_all = policy.critic.train_forward(c_in)
    mean, value = mean_all[:rows], value_all[:rows].reshape(-1)
    lp, ent = torch.empty_like(mean), torch.empty_like(mean)
    _lib.check(lib.ks_gaussian_log_prob(st, rows, nu, _lib.ptr(mean), _lib.ptr(policy.log_std), _lib.ptr(act), _lib.ptr(lp), _lib.ptr(ent)))
    inputs = ppo_mod.compute_ppo_inputs(value.view(Tn, b), rewards, done, success, cfg.gamma, cfg.lam,
                                        normalize_advantages=cfg.normalize_advantages,
                                        monte_carlo_returns=cfg.monte_carlo_returns, time_major=True)
    # adaptive KL (ppo.py:546-563): the running factor kl_coef_now / kl_coef is a device scalar that the loss kernel reads
    # and ks_ppo_adapt_kl updates after the step, so no value crosses to the host between minibatch steps
    if cfg.adaptive_kl and policy.kl_scale is None:
        policy.kl_scale = torch.ones(1, dtype=torch.float32, device=actor_obs.device)
    p = _lib.KsPpoLossParams(cfg.clip_param, cfg.value_loss_coef, cfg.entropy_coef, cfg.kl_coef, cfg.log_clip_value,
                             1.0, int(cfg.use_clipped_value_loss), _lib.ptr(policy.kl_scale) if cfg.adaptive_kl else None)
    d_mean_all = torch.empty_like(mean_all)
    d_value_all = torch.empty(value_all.shape[0], 1, dtype=torch.float32, device=mean.device)
    d_mean, d_value = d_mean_all[:rows], d_value_all[:rows]
    d_log_std = torch.empty_like(policy.log_std)
    ws = torch.empty(256 * nu, dtype=torch.float32, device=mean.device)
    on_lp, on_v = on_log_probs.reshape(rows, nu), on_values.reshape(rows)
    _lib.check(lib.ks_ppo_loss_grad(_lib.current_stream(), rows, nu, ctypes.byref(p), _lib.ptr(mean),
                                    _lib.ptr(policy.log_std), _lib.ptr(act), _lib.ptr(on_lp),
                                    _lib.ptr(inputs.advantages_bt), _lib.ptr(inputs.value_targets_bt), _lib.ptr(on_v),
                                    _lib.ptr(value), _lib.ptr(d_mean), _lib.ptr(d_value), _lib.ptr(d_log_std), _lib.ptr(ws)))
    aux = {}
    if mirror_a:
        perm, sign = policy.mirror.device("action", mean.device)
        aux["action_mirror_loss"] = torch.empty(rows, dtype=torch.float32, device=mean.device)
        _lib.check(lib.ks_mirror_loss_grad(st, rows, nu, cfg.actor_mirror_loss_scale, _lib.ptr(mean), _lib.ptr(mean_all[rows:]),
                                           _lib.ptr(perm), _lib.ptr(sign), _lib.ptr(d_mean), _lib.ptr(d_mean_all[rows:]),
                                           _lib.ptr(aux["action_mirror_loss"])))
    if mirror_c:
        perm, sign = policy.mirror.device("value", mean.device)
        aux["value_mirror_loss"] = torch.empty(rows, dtype=torch.float32, device=mean.device)
        _lib.check(lib.ks_mirror_loss_grad(st, rows, 1, cfg.critic_mirror_loss_scale, _lib.ptr(value_all), _lib.ptr(value_all[rows:]),
                                           _lib.ptr(perm), _lib.ptr(sign), _lib.ptr(d_value), _lib.ptr(d_value_all[rows:]),
                                           _lib.ptr(aux["value_mirror_loss"])))
    policy.actor.backward(a_in, d_mean_all)
    policy.critic.backward(c_in, d_value_all)
    # optimiser chain over every parameter together: global norm first
    sq = torch.zeros(1, dtype=torch.float64, device=mean.device)
    policy.actor.grad_sqnorm(sq)
    policy.critic.grad_sqnorm(sq)
    _lib.check(lib.ks_grad_sqnorm(_lib.current_stream(), nu, _lib.ptr(d_log_std), _lib.ptr(sq)))
    policy.opt_step += 1
    ap = _adam(cfg, policy.opt_step)
    policy.actor.adam_step(ap, sq)
    policy.critic.adam_step(ap, sq)
    _lib.check(lib.ks_adam_step(_lib.current_stream(), nu, _lib.ptr(policy.log_std), _lib.ptr(d_log_std),
                                _lib.ptr(policy._m1), _lib.ptr(policy._m2), ctypes.byref(ap), _lib.ptr(sq)))
    metrics = {"grad_norm": sq.sqrt(), "d_mean": d_mean, "d_value": d_value, "d_log_std": d_log_std,
               "log_probs": lp, "values": value, "advantages": inputs.advantages_bt, **aux}
    if cfg.adaptive_kl:
        _lib.check(lib.ks_ppo_adapt_kl(_lib.current_stream(), rows, nu, _lib.ptr(on_lp), _lib.ptr(lp), cfg.kl_coef,
                                       cfg.desired_kl, _lib.ptr(policy.kl_scale), _lib.ptr(ws)))
    return metrics


def update_model(policy: GaussianMlpPolicy, cfg: PPOUpdateConfig, actor_obs, critic_obs, action, rewards, done, success,
                 permutations: list[torch.Tensor] | None = None, seed: int = 0, after_step=None) -> list[dict]:
    """num_passes x (N / batch_size) minibatch steps over a (T, N) rollout (ppo.py:572-694).

    `permutations` (one index vector per pass) replaces the reference's `jax.random.permutation`.  `after_step(idx)`,
    when given, runs after every minibatch step with the env indices of that minibatch: the hook through which the AMP
    task's `_single_step` appends its discriminator passes (ksim/task/amp.py:455-545); what it returns is stored in the
    step's metrics under "after_step"."""
    Tn, N = done.shape
    if policy._m1 is None:
        policy.train_init()
    nu = action.shape[-1]
    # on-policy variables of the whole rollout with the pre-update parameters (ppo.py:603-607)
    on_lp, on_v, _, _ = get_ppo_variables(policy, actor_obs.reshape(Tn * N, -1), critic_obs.reshape(Tn * N, -1),
                                          action.reshape(Tn * N, nu))
    on_lp, on_v = on_lp.view(Tn, N, nu).clone(), on_v.view(Tn, N).clone()
    bs = min(cfg.batch_size, N)
    if N % bs:
        raise _lib.KsError("the env count must be a multiple of the batch size (ppo.py:647 reshapes the permutation)")
    gen = torch.Generator(device=done.device)
    gen.manual_seed(seed)
    out = []
    for k in range(cfg.num_passes):
        perm = permutations[k] if permutations is not None else torch.randperm(N, generator=gen, device=done.device)
        for idx in perm.view(-1, bs):
            sel = lambda t: t.index_select(1, idx).contiguous()  # noqa: E731
            out.append(single_step(policy, cfg, sel(actor_obs), sel(critic_obs), sel(action), sel(rewards), sel(done),
                                   sel(success), sel(on_lp), sel(on_v)))
            if after_step is not None:
                out[-1]["after_step"] = after_step(idx)
    return out


# --------------------------------------------------------------------------- recurrent actor / critic (GRU or LSTM stacks)
@dataclass
class MirrorCarries:
    """The mirrored pass's own carries at the first step of the trajectory slice (`actor_mirror`, `critic_mirror`,
    `lpf_params_mirror` of examples/kbot/train.py:1506-1515); None entries start from zero, which is what the task's
    rollout leaves there (it never advances them)."""
    actor: torch.Tensor | None = None
    critic: torch.Tensor | None = None
    lpf: torch.Tensor | None = None


def _cat_env(a: torch.Tensor, b: torch.Tensor | None) -> torch.Tensor:
    """Carries of the first and the mirrored pass side by side on the env axis ((depth, 2, N, H) or (depth, N, H))."""
    ax = 2 if a.dim() == 4 else 1
    return torch.cat([a, torch.zeros_like(a) if b is None else b], dim=ax).contiguous()


def actor_locations(policy: "RecurrentHeadPolicy", raw: torch.Tensor, obs: torch.Tensor, fresh: torch.Tensor,
                    lpf0: torch.Tensor | None, y_last: torch.Tensor | None = None) -> torch.Tensor:
    """raw (T, M, 2 nu) -> the same rows with the distribution's location (bias added, filtered) in the first half, when
    the policy filters its means; `obs` (T, M, in) supplies the observation-dependent part of the bias."""
    lp = policy.lowpass
    if lp is None:
        return raw
    Tn, M, W = raw.shape
    nu = W // 2
    add, add_ld, a0, cnt = None, 0, 0, 0
    if lp.obs_bias is not None:
        col0, a0, cnt = (int(v) for v in lp.obs_bias)
        if col0 < 0 or col0 + cnt > obs.shape[-1] or not obs.is_contiguous():
            raise _lib.KsError("the observation-dependent bias reads columns outside the observation rows")
        add, add_ld = ctypes.c_void_p(obs.data_ptr() + 4 * col0), obs.shape[-1]
    out = torch.empty_like(raw)
    _lib.check(_lib.load().ks_lowpass_scan(_lib.current_stream(), Tn, M, nu, W, float(lp.ctrl_dt), float(lp.cutoff_frequency),
                                           _lib.ptr(raw), _lib.ptr(policy.mean_bias), add, add_ld, a0, cnt, _lib.ptr(lpf0),
                                           _lib.ptr(fresh), _lib.ptr(out), _lib.ptr(y_last)))
    return out


@dataclass
class RecurrentHeadPolicy:
    """Recurrent actor whose output is (means | raw deviations) per action (examples/kbot/train.py:903-932) and a
    recurrent critic; `min_std`, `max_std`, `var_scale`, `mean_bias` describe the deviation head."""
    actor: "object"
    critic: "object"
    min_std: float
    max_std: float
    var_scale: float = 1.0
    mean_bias: torch.Tensor | None = None
    opt_step: int = 0
    # a mixture-of-Gaussians head instead (examples/walking.py:127-144): the actor emits 3 K values per action
    num_mixtures: int = 0
    clip_lo: torch.Tensor | None = None
    clip_hi: torch.Tensor | None = None
    kl_scale: torch.Tensor | None = None  # adaptive KL: current coefficient / cfg.kl_coef, one device float
    lowpass: "LowPass | None" = None      # the actor's means pass a one-pole low-pass whose state rides in the model carry
    mirror: MirrorSpec | None = None      # the task's symmetry, for the mirror losses (second pass from mirrored carries)

    def kl_coef(self, cfg: "PPOUpdateConfig") -> float:
        """The KL coefficient now in force (a host read: for logging and tests)."""
        return cfg.kl_coef * (float(self.kl_scale.item()) if self.kl_scale is not None else 1.0)

    def train_init(self) -> None:
        self.actor.train_init()
        self.critic.train_init()

    def width(self, nu: int) -> int:
        return 3 * nu * self.num_mixtures if self.num_mixtures else 2 * nu

    def _mixture(self) -> "T.KsMixtureHead":
        return T.KsMixtureHead(int(self.num_mixtures), float(self.min_std), float(self.max_std), float(self.var_scale), 0,
                               _lib.ptr(self.mean_bias).value, _lib.ptr(self.clip_lo).value, _lib.ptr(self.clip_hi).value)


def single_step_recurrent(policy: RecurrentHeadPolicy, cfg: PPOUpdateConfig, actor_obs, critic_obs, action, rewards, done, success,
                          on_log_probs, on_values, actor_carry0, critic_carry0, fresh, lpf0=None,
                          mirror_carries: MirrorCarries | None = None) -> dict:
    """One minibatch step (ppo.py:495-565) for recurrent networks: both networks run over the (T, b) trajectory slice
    from the carries the rollout started with, envs flagged in `fresh` (T, b) restart their carry, and the gradient goes
    back through time.  GAE is recomputed from the current values and enters as a constant.

    With `policy.lowpass` the actor's biased means pass the one-pole filter from the state `lpf0` (b, nu) and its gradient
    runs back through time with the networks'.  With mirror loss scales set (`policy.mirror` names the maps) each network
    runs a second time on the mirrored observations from `mirror_carries` (examples/kbot/train.py:1458-1496): the mirrored
    envs ride as columns [b, 2b) of the same forward and backward pass, so both passes' gradients meet in one sweep."""
    lib = _lib.load()
    Tn, b = done.shape
    rows = Tn * b
    nu = action.shape[-1]
    st = _lib.current_stream()
    dev = actor_obs.device
    mixture = policy.num_mixtures > 0
    mirror_a, mirror_c = cfg.actor_mirror_loss_scale != 0.0, cfg.critic_mirror_loss_scale != 0.0
    if (mirror_a or mirror_c) and policy.mirror is None:
        raise _lib.KsError("mirror loss scales are set but the policy has no MirrorSpec")
    if mixture and (policy.lowpass is not None or mirror_a):
        raise _lib.KsError("the low-pass filter and the action mirror loss are built for the mean | deviation head")
    mc = mirror_carries or MirrorCarries()

    def both(x, name):  # (T, b, n) -> (T, 2b, n): the rows and their mirror images side by side
        perm, sign = policy.mirror.device(name, dev)
        if perm.numel() != x.shape[-1]:
            raise _lib.KsError(f"the {name} mirror map has {perm.numel()} entries, the rows have {x.shape[-1]}")
        x = x.contiguous()
        xm = torch.empty_like(x)
        _lib.check(lib.ks_signed_permute(st, rows, x.shape[-1], _lib.ptr(x), _lib.ptr(perm), _lib.ptr(sign), _lib.ptr(xm)))
        return torch.cat([x, xm], dim=1).contiguous()

    fresh2 = torch.cat([fresh, fresh], dim=1).contiguous() if (mirror_a or mirror_c) else None
    a_in = both(actor_obs, "actor_obs") if mirror_a else actor_obs.contiguous()
    c_in = both(critic_obs, "critic_obs") if mirror_c else critic_obs.contiguous()
    a_fresh, c_fresh = (fresh2 if mirror_a else fresh), (fresh2 if mirror_c else fresh)
    raw_all = policy.actor.train_forward(a_in, _cat_env(actor_carry0, mc.actor) if mirror_a else actor_carry0, a_fresh)
    value_all = policy.critic.train_forward(c_in, _cat_env(critic_carry0, mc.critic) if mirror_c else critic_carry0, c_fresh)
    y0 = None
    if policy.lowpass is not None:
        y0 = lpf0 if lpf0 is not None else torch.zeros(b, nu, dtype=torch.float32, device=dev)
        if mirror_a:
            y0 = torch.cat([y0, torch.zeros_like(y0) if mc.lpf is None else mc.lpf], dim=0).contiguous()
    loc_all = actor_locations(policy, raw_all, a_in, a_fresh, y0)   # (T, b or 2b, 2 nu): location | raw deviation
    raw = loc_all[:, :b].contiguous() if mirror_a else loc_all
    value = value_all[:, :b].contiguous() if mirror_c else value_all
    inputs = ppo_mod.compute_ppo_inputs(value.view(Tn, b), rewards, done, success, cfg.gamma, cfg.lam,
                                        normalize_advantages=cfg.normalize_advantages,
                                        monte_carlo_returns=cfg.monte_carlo_returns, time_major=True)
    if cfg.adaptive_kl and policy.kl_scale is None:  # as in single_step: the factor stays on the device
        policy.kl_scale = torch.ones(1, dtype=torch.float32, device=dev)
    p = _lib.KsPpoLossParams(cfg.clip_param, cfg.value_loss_coef, cfg.entropy_coef, cfg.kl_coef, cfg.log_clip_value, 1.0,
                             int(cfg.use_clipped_value_loss), _lib.ptr(policy.kl_scale) if cfg.adaptive_kl else None)
    # behind the filter the bias is already inside the location
    bias_ptr = None if policy.lowpass is not None else _lib.ptr(policy.mean_bias).value
    head = policy._mixture() if mixture else T.KsGaussianHead(float(policy.min_std), float(policy.max_std), float(policy.var_scale), 0, bias_ptr)
    d_raw = torch.empty(Tn, b, policy.width(nu), dtype=torch.float32, device=dev)
    d_value = torch.empty(Tn, b, 1, dtype=torch.float32, device=dev)
    grad_fn = lib.ks_ppo_loss_grad_mixture if mixture else lib.ks_ppo_loss_grad_head
    _lib.check(grad_fn(st, rows, nu, ctypes.byref(p), ctypes.byref(head), _lib.ptr(raw),
                       _lib.ptr(action.contiguous()), _lib.ptr(on_log_probs.contiguous()),
                       _lib.ptr(inputs.advantages_bt), _lib.ptr(inputs.value_targets_bt),
                       _lib.ptr(on_values.contiguous()), _lib.ptr(value), _lib.ptr(d_raw), _lib.ptr(d_value)))
    aux = {}
    d_raw_all, d_value_all = d_raw, d_value
    if mirror_a:
        # modes of the two passes (the head's bias, where no filter has absorbed it, is part of the mode)
        mode, mode_m = raw[..., :nu].contiguous(), loc_all[:, b:, :nu].contiguous()
        if policy.lowpass is None and policy.mean_bias is not None:
            mode, mode_m = mode + policy.mean_bias, mode_m + policy.mean_bias
        d_mode, d_mode_m = d_raw[..., :nu].contiguous(), torch.empty(Tn, b, nu, dtype=torch.float32, device=dev)
        perm, sign = policy.mirror.device("action", dev)
        aux["action_mirror_loss"] = torch.empty(Tn, b, dtype=torch.float32, device=dev)
        _lib.check(lib.ks_mirror_loss_grad(st, rows, nu, cfg.actor_mirror_loss_scale, _lib.ptr(mode), _lib.ptr(mode_m), _lib.ptr(perm),
                                           _lib.ptr(sign), _lib.ptr(d_mode), _lib.ptr(d_mode_m), _lib.ptr(aux["action_mirror_loss"])))
        d_raw_all = torch.zeros(Tn, 2 * b, 2 * nu, dtype=torch.float32, device=dev)  # the mirrored deviations enter nothing
        d_raw_all[:, :b] = d_raw
        d_raw_all[:, :b, :nu] = d_mode
        d_raw_all[:, b:, :nu] = d_mode_m
    if mirror_c:
        v_main, v_m = value.view(rows, 1), value_all[:, b:].contiguous().view(rows, 1)
        d_v, d_vm = d_value.view(rows, 1), torch.empty(rows, 1, dtype=torch.float32, device=dev)
        perm, sign = policy.mirror.device("value", dev)
        aux["value_mirror_loss"] = torch.empty(Tn, b, dtype=torch.float32, device=dev)
        _lib.check(lib.ks_mirror_loss_grad(st, rows, 1, cfg.critic_mirror_loss_scale, _lib.ptr(v_main), _lib.ptr(v_m), _lib.ptr(perm),
                                           _lib.ptr(sign), _lib.ptr(d_v), _lib.ptr(d_vm), _lib.ptr(aux["value_mirror_loss"])))
        d_value_all = torch.cat([d_value, d_vm.view(Tn, b, 1)], dim=1).contiguous()
    if policy.lowpass is not None:  # dL/d location -> dL/d raw mean, back through the filter's own recursion
        if d_raw_all is d_raw:
            d_raw_all = d_raw.clone()  # d_raw stays what the loss kernel wrote, for the caller's metrics
        lp_ = policy.lowpass
        _lib.check(lib.ks_lowpass_scan_backward(st, Tn, d_raw_all.shape[1], nu, 2 * nu, float(lp_.ctrl_dt), float(lp_.cutoff_frequency),
                                                _lib.ptr(a_fresh), _lib.ptr(d_raw_all), None))
    policy.actor.backward(d_raw_all)
    policy.critic.backward(d_value_all)
    sq = torch.zeros(1, dtype=torch.float64, device=dev)
    policy.actor.grad_sqnorm(sq)
    policy.critic.grad_sqnorm(sq)
    policy.opt_step += 1
    ap = _adam(cfg, policy.opt_step)
    policy.actor.adam_step(ap, sq)
    policy.critic.adam_step(ap, sq)
    metrics = {"grad_norm": sq.sqrt(), "d_raw": d_raw, "d_value": d_value, "raw": raw, "values": value,
               "advantages": inputs.advantages_bt, **aux}
    if cfg.adaptive_kl:  # ppo.py:546-563 on the log-probabilities of this step's forward pass
        lp = torch.empty(rows, nu, dtype=torch.float32, device=dev)
        if mixture:
            _lib.check(lib.ks_mixture_head_log_prob(st, rows, nu, ctypes.byref(head), _lib.ptr(raw),
                                                    _lib.ptr(action.contiguous()), _lib.ptr(lp)))
        else:
            _lib.check(lib.ks_gaussian_head_log_prob(st, rows, nu, ctypes.byref(head), _lib.ptr(raw),
                                                     _lib.ptr(action.contiguous()), _lib.ptr(lp), None))
        ws = torch.empty(256 * nu, dtype=torch.float32, device=dev)
        _lib.check(lib.ks_ppo_adapt_kl(st, rows, nu, _lib.ptr(on_log_probs.contiguous()), _lib.ptr(lp), cfg.kl_coef,
                                       cfg.desired_kl, _lib.ptr(policy.kl_scale), _lib.ptr(ws)))
        metrics["log_probs"] = lp
    return metrics


def recurrent_on_policy(policy: RecurrentHeadPolicy, actor_obs, critic_obs, action, actor_carry0, critic_carry0, fresh, lpf0=None,
                        return_raw: bool = False):
    """Log-probabilities (T, N, nu) and values (T, N) of the recorded actions under the current parameters: the pass that
    update_model makes once over the whole rollout before any minibatch step (ppo.py:603-607).  With `return_raw` also the
    head's input rows (T, N, width), locations filtered where the policy filters them."""
    Tn, N, nu = action.shape
    a_carry, c_carry = actor_carry0.clone(), critic_carry0.clone()
    raw = torch.empty(Tn, N, policy.width(nu), dtype=torch.float32, device=action.device)
    values = torch.empty(Tn, N, 1, dtype=torch.float32, device=action.device)
    for t in range(Tn):
        policy.actor(actor_obs[t], a_carry, fresh=fresh[t], out=raw[t])
        policy.critic(critic_obs[t], c_carry, fresh=fresh[t], out=values[t])
    if policy.lowpass is not None:
        raw = actor_locations(policy, raw, actor_obs.contiguous(), fresh.contiguous(), lpf0)
    lp = torch.empty(Tn, N, nu, dtype=torch.float32, device=action.device)
    if policy.num_mixtures:
        head = policy._mixture()
        _lib.check(_lib.load().ks_mixture_head_log_prob(_lib.current_stream(), Tn * N, nu, ctypes.byref(head), _lib.ptr(raw),
                                                        _lib.ptr(action.contiguous()), _lib.ptr(lp)))
    else:
        head = T.KsGaussianHead(float(policy.min_std), float(policy.max_std), float(policy.var_scale), 0,
                                None if policy.lowpass is not None else _lib.ptr(policy.mean_bias).value)
        _lib.check(_lib.load().ks_gaussian_head_log_prob(_lib.current_stream(), Tn * N, nu, ctypes.byref(head), _lib.ptr(raw),
                                                         _lib.ptr(action.contiguous()), _lib.ptr(lp), None))
    return (lp, values[..., 0], raw) if return_raw else (lp, values[..., 0])


def update_model_recurrent(policy: RecurrentHeadPolicy, cfg: PPOUpdateConfig, actor_obs, critic_obs, action, rewards, done, success,
                           actor_carry0, critic_carry0, fresh, permutations: list[torch.Tensor] | None = None,
                           seed: int = 0, lpf0=None, mirror_carries: MirrorCarries | None = None) -> list[dict]:
    """num_passes x (N / batch_size) minibatch steps over a (T, N) rollout for a recurrent actor and critic
    (ppo.py:572-694): a minibatch is a set of env columns together with their carries at the rollout's first step
    (`lpf0` (N, nu): the filter state there; `mirror_carries`: the mirrored pass's, zero when None)."""
    Tn, N = done.shape
    on_lp, on_v = recurrent_on_policy(policy, actor_obs, critic_obs, action, actor_carry0, critic_carry0, fresh, lpf0)
    mc = mirror_carries or MirrorCarries()
    bs = min(cfg.batch_size, N)
    if N % bs:
        raise _lib.KsError("the env count must be a multiple of the batch size (ppo.py:647 reshapes the permutation)")
    gen = torch.Generator(device=done.device)
    gen.manual_seed(seed)
    env_axis = {True: 2, False: 1}  # carries: (depth, 2, N, H) for LSTM stacks, (depth, N, H) for GRU stacks
    out = []
    for k in range(cfg.num_passes):
        perm = permutations[k] if permutations is not None else torch.randperm(N, generator=gen, device=done.device)
        for idx in perm.view(-1, bs):
            sel = lambda t: t.index_select(1, idx).contiguous()  # noqa: E731
            ca = actor_carry0.index_select(env_axis[actor_carry0.dim() == 4], idx).contiguous()
            cc = critic_carry0.index_select(env_axis[critic_carry0.dim() == 4], idx).contiguous()
            env_sel = lambda c: None if c is None else c.index_select(env_axis[c.dim() == 4], idx).contiguous()  # noqa: E731
            rows_sel = lambda c: None if c is None else c.index_select(0, idx).contiguous()  # noqa: E731
            out.append(single_step_recurrent(policy, cfg, sel(actor_obs), sel(critic_obs), sel(action), sel(rewards), sel(done),
                                             sel(success), sel(on_lp), sel(on_v), ca, cc, sel(fresh), rows_sel(lpf0),
                                             MirrorCarries(env_sel(mc.actor), env_sel(mc.critic), rows_sel(mc.lpf))))
    return out
