"""TEST INFRASTRUCTURE: float64 restatement of the AMP discriminator's loss and of its gradient (ksim/task/amp.py:360-438).

`disc_loss` follows `get_disc_losses` (least-squares targets +1 for reference motions, -1 for simulated ones, summed)
and `_grad_penalty` (per motion the squared norm of the gradient of the summed logits with respect to the whole motion,
averaged over the motions, times coef / 2).  The discriminator is an MLP applied to each frame, so the logits of a motion
are (T,) as `call_discriminator` requires (amp.py:257-268).  The gradient with respect to the parameters is taken by
torch's CPU autograd in float64 through the input gradient (create_graph).  Pinned by tests/test_oracle_amp.py: a linear
discriminator's closed forms, a numpy evaluation whose input gradient comes from central differences, and central
differences of the loss in single parameters.  Only tests may import this module.
"""
from __future__ import annotations

import numpy as np
import torch

from .ppo_update import mlp


def disc_loss(ws, bs, real, sim, coef, act="elu"):
    """real (B, T, F), sim (B2, T2, F) float64 tensors; returns (total, real term, simulated term, penalty term)."""
    x = real.detach().clone().requires_grad_(True)
    real_logits = mlp(x, ws, bs, act)[..., 0]                 # (B, T)
    sim_logits = mlp(sim, ws, bs, act)[..., 0]
    real_loss = 0.5 * ((real_logits - 1.0) ** 2).sum()       # amp.py:365
    sim_loss = 0.5 * ((sim_logits + 1.0) ** 2).sum()         # amp.py:366
    # amp.py:369-389: vmap over motions of grad(sum of the motion's logits); frames do not interact, so one call does it
    (g,) = torch.autograd.grad(real_logits.sum(), x, create_graph=True)
    per_motion = (g ** 2).sum(dim=(1, 2))                      # (B,)
    gp = coef / 2.0 * per_motion.mean()                       # amp.py:423
    return real_loss + sim_loss + gp, real_loss, sim_loss, gp


def disc_loss_and_grads(weights, biases, real, sim, coef, act="elu"):
    """numpy in, numpy out: (losses (3,), [(dW, db) per layer])."""
    ws = [torch.tensor(np.asarray(w, dtype=np.float64), requires_grad=True) for w in weights]
    bs = [torch.tensor(np.asarray(b, dtype=np.float64), requires_grad=True) for b in biases]
    total, rl, sl, gp = disc_loss(ws, bs, torch.tensor(np.asarray(real, dtype=np.float64)),
                                  torch.tensor(np.asarray(sim, dtype=np.float64)), coef, act)
    total.backward()
    zero = lambda p: np.zeros(tuple(p.shape)) if p.grad is None else p.grad.numpy()  # noqa: E731
    return (np.array([rl.item(), sl.item(), gp.item()]), [(zero(w), zero(b)) for w, b in zip(ws, bs)])
