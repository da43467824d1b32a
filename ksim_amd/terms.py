"""Reward total and termination combination on device (ksim/task/rl.py:219-239, 1049-1050)."""
from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from . import _lib


def reward_total_and_done(
    components: torch.Tensor | None,
    scales: Sequence[float],
    terminations: torch.Tensor | None,
    clip_min: float | None = None,
    clip_max: float | None = None,
):
    """components (K, n) f32 with K sign-folded scales; terminations (k, n) int8 in {-1, 0, 1}.

    Returns (total (n) f32 | None, done (n) uint8 | None, success (n) uint8 | None).
    """
    lib = _lib.load()
    _lib.require_cuda(components, dtype=torch.float32)
    _lib.require_cuda(terminations, dtype=torch.int8)
    ref = components if components is not None else terminations
    if ref is None:
        raise _lib.KsError("nothing to reduce")
    n = ref.shape[1]
    K = 0 if components is None else components.shape[0]
    k = 0 if terminations is None else terminations.shape[0]
    if K != len(scales):
        raise _lib.KsError("one scale per reward component is required")
    total = torch.empty(n, dtype=torch.float32, device=ref.device) if K else None
    done = torch.empty(n, dtype=torch.uint8, device=ref.device) if k else None
    succ = torch.empty(n, dtype=torch.uint8, device=ref.device) if k else None
    sc = (ctypes.c_float * max(K, 1))(*[float(s) for s in scales])
    _lib.check(
        lib.ks_reward_total(_lib.current_stream(), n, K, _lib.ptr(components), sc, int(clip_min is not None),
                            float(clip_min or 0.0), int(clip_max is not None), float(clip_max or 0.0), _lib.ptr(total),
                            k, _lib.ptr(terminations), _lib.ptr(done), _lib.ptr(succ))
    )
    return total, done, succ
