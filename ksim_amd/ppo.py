"""GAE / PPO-loss host interface with the reference's names and argument meaning.

Mirrors ksim/task/ppo.py: ``compute_ppo_inputs`` (54-121), ``clipped_value_loss``
(124-135 — folded into the loss kernel), ``compute_ppo_loss`` (149-246),
``PPOInputs`` / ``PPOVariables`` (ppo.py:30-47 in the reference).  Arrays are torch
CUDA tensors of shape (B, T) (log-probs (B, T, A)); the arithmetic runs in the HIP
kernels of libksimhip.so.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping

import torch

from . import _lib


@dataclass
class PPOInputs:
    advantages_bt: torch.Tensor
    value_targets_bt: torch.Tensor
    gae_bt: torch.Tensor
    returns_bt: torch.Tensor


@dataclass
class PPOVariables:
    log_probs: torch.Tensor
    values: torch.Tensor
    entropy: torch.Tensor | None = None
    aux_losses: Mapping[str, torch.Tensor] | None = None


def _as_bytes(x: torch.Tensor) -> torch.Tensor:
    if x.dtype == torch.bool:
        return x.view(torch.uint8)
    if x.dtype in (torch.uint8, torch.int8):
        return x
    raise _lib.KsError(f"dones/successes must be bool or 1-byte integers, got {x.dtype}")


def _workspace(device) -> torch.Tensor:
    return torch.empty(_lib.KS_REDUCE_WORKSPACE_BYTES, dtype=torch.uint8, device=device)


def compute_ppo_inputs(
    values_bt: torch.Tensor,
    rewards_bt: torch.Tensor,
    dones_bt: torch.Tensor,
    successes_bt: torch.Tensor | None,
    decay_gamma: float,
    gae_lambda: float,
    normalize_advantages: bool = False,
    monte_carlo_returns: bool = False,
    *,
    time_major: bool = False,
) -> PPOInputs:
    """GAE and returns. ``time_major=True`` takes (T, N) arrays (the rollout buffer's layout)."""
    lib = _lib.load()
    dones = _as_bytes(dones_bt)
    succ = None if successes_bt is None else _as_bytes(successes_bt)
    _lib.require_cuda(values_bt, rewards_bt, dtype=torch.float32)
    _lib.require_cuda(dones, succ)
    if values_bt.dim() != 2 or rewards_bt.shape != values_bt.shape or dones.shape != values_bt.shape:
        raise _lib.KsError("values, rewards and dones must share one 2-D shape")
    if succ is not None and succ.shape != values_bt.shape:
        raise _lib.KsError("successes must have the shape of values")
    gae = torch.empty_like(values_bt)
    ret = torch.empty_like(values_bt)
    tgt = torch.empty_like(values_bt)
    fn = lib.ks_gae_tn if time_major else lib.ks_gae_bt
    _lib.check(
        fn(_lib.current_stream(), values_bt.shape[0], values_bt.shape[1], _lib.ptr(values_bt), _lib.ptr(rewards_bt),
           _lib.ptr(dones), _lib.ptr(succ), float(decay_gamma), float(gae_lambda), int(monte_carlo_returns),
           _lib.ptr(gae), _lib.ptr(ret), _lib.ptr(tgt))
    )
    adv = gae
    if normalize_advantages:
        adv = torch.empty_like(gae)
        ws = _workspace(gae.device)
        _lib.check(lib.ks_normalize_advantages(_lib.current_stream(), gae.numel(), _lib.ptr(gae), _lib.ptr(adv),
                                               _lib.ptr(ws)))
    return PPOInputs(advantages_bt=adv, value_targets_bt=tgt, gae_bt=gae, returns_bt=ret)


def compute_ppo_loss(
    ppo_inputs: PPOInputs,
    on_policy_variables: PPOVariables,
    off_policy_variables: PPOVariables,
    *,
    clip_param: float = 0.2,
    value_loss_coef: float = 0.5,
    entropy_coef: float = 0.008,
    kl_coef: float = 1e-3,
    log_clip_value: float = 5.0,
    use_clipped_value_loss: bool = True,
    kl_scale: float = 1.0,
) -> dict[str, torch.Tensor]:
    """Per-element loss terms (B, T) plus ``"total"`` = mean over (B, T) of their sum (ppo.py:485-486)."""
    lib = _lib.load()
    on, off = on_policy_variables, off_policy_variables
    if on.log_probs.dim() != 3 or off.log_probs.shape != on.log_probs.shape:
        raise _lib.KsError("log_probs must be rank 3 (B, T, A) and match")
    if on.values.dim() != 2 or off.values.dim() != 2 or ppo_inputs.advantages_bt.dim() != 2:
        raise _lib.KsError("values and advantages must be rank 2 (B, T)")
    B, T, A = on.log_probs.shape
    for x in (on.values, off.values, ppo_inputs.advantages_bt, ppo_inputs.value_targets_bt):
        if tuple(x.shape) != (B, T):
            raise _lib.KsError("shape prefix mismatch between log_probs, values and ppo inputs")
    _lib.require_cuda(on.log_probs, on.values, off.log_probs, off.values, off.entropy, ppo_inputs.advantages_bt,
                      ppo_inputs.value_targets_bt, dtype=torch.float32)
    dev = on.values.device
    out = {k: torch.empty((B, T), dtype=torch.float32, device=dev) for k in ("policy", "value", "kl")}
    if off.entropy is not None:
        out["entropy"] = torch.empty((B, T), dtype=torch.float32, device=dev)
    total = torch.empty((), dtype=torch.float32, device=dev)
    params = _lib.KsPpoLossParams(clip_param, value_loss_coef, entropy_coef, kl_coef, log_clip_value, kl_scale,
                                  int(use_clipped_value_loss))
    ws = _workspace(dev)
    _lib.check(
        lib.ks_ppo_loss(_lib.current_stream(), B * T, A, params, _lib.ptr(ppo_inputs.advantages_bt),
                        _lib.ptr(ppo_inputs.value_targets_bt), _lib.ptr(on.log_probs), _lib.ptr(on.values),
                        _lib.ptr(off.log_probs), _lib.ptr(off.values), _lib.ptr(off.entropy), _lib.ptr(out["policy"]),
                        _lib.ptr(out["value"]), _lib.ptr(out["kl"]), _lib.ptr(out.get("entropy")), _lib.ptr(total),
                        _lib.ptr(ws))
    )
    if off.aux_losses is not None:  # ppo.py:242-244 — user terms pass through and join the mean
        aux_sum = None
        for name, term in off.aux_losses.items():
            out[name] = term
            aux_sum = term if aux_sum is None else aux_sum + term
        total = total + aux_sum.mean()
    out["total"] = total
    return out
