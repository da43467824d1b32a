"""ctypes binding of libksimhip.so (the C ABI in include/ksim_hip.h).

There is no CPU fallback: if the library has not been built the import of any
compute entry point raises.  torch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int8, c_int32, c_int64, c_uint8, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libksimhip.so")


class KsError(RuntimeError):
    pass


class KsPpoLossParams(ctypes.Structure):
    _fields_ = [
        ("clip_param", c_float),
        ("value_loss_coef", c_float),
        ("entropy_coef", c_float),
        ("kl_coef", c_float),
        ("log_clip_value", c_float),
        ("kl_scale", c_float),
        ("use_clipped_value_loss", c_int32),
        ("kl_scale_device", c_void_p),
    ]


KS_REDUCE_WORKSPACE_BYTES = 2 * 1024 * 8 + 64
KS_MAX_REWARD_TERMS = 32

_lib = None


def load() -> ctypes.CDLL:
    """Loads the built library; raises KsError when it is missing (no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise KsError(
            f"{LIB_PATH} is not built; run `python -m ksim_amd.csrc.build` (hipcc, gfx950). "
            "ksim_amd has no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.ks_version.restype = c_char_p
    lib.ks_last_error.restype = c_char_p
    p = c_void_p
    lib.ks_gae_bt.argtypes = [p, c_int64, c_int64, p, p, p, p, c_float, c_float, c_int32, p, p, p]
    lib.ks_gae_tn.argtypes = lib.ks_gae_bt.argtypes
    lib.ks_normalize_advantages.argtypes = [p, c_int64, p, p, p]
    lib.ks_normalize_advantages_static.argtypes = [p, c_int64, p, p]
    lib.ks_normalize_advantages_static.restype = c_int32
    lib.ks_ppo_loss.argtypes = [p, c_int64, c_int32, POINTER(KsPpoLossParams)] + [p] * 13
    lib.ks_reward_total.argtypes = [p, c_int64, c_int32, p, POINTER(c_float), c_int32, c_float, c_int32, c_float, p,
                                    c_int32, p, p, p]
    lib.ks_copy_f32.argtypes = [p, c_int64, p, p]
    lib.ks_mfma_yardstick.argtypes = [p, c_int32, c_int32, p, p]
    lib.ks_mfma_yardstick.restype = c_int32
    lib.ks_ppo_loss_grad.argtypes = [p, c_int64, c_int32, POINTER(KsPpoLossParams)] + [p] * 12
    lib.ks_ppo_loss_grad.restype = c_int32
    lib.ks_signed_permute.argtypes = [p, c_int64, c_int32, p, p, p, p]
    lib.ks_signed_permute.restype = c_int32
    lib.ks_mirror_loss_grad.argtypes = [p, c_int64, c_int32, c_float, p, p, p, p, p, p, p]
    lib.ks_mirror_loss_grad.restype = c_int32
    lib.ks_lowpass_scan.argtypes = [p, c_int64, c_int64, c_int32, c_int32, c_float, c_float, p, p, p, c_int64, c_int32, c_int32, p, p, p, p]
    lib.ks_lowpass_scan.restype = c_int32
    lib.ks_lowpass_scan_backward.argtypes = [p, c_int64, c_int64, c_int32, c_int32, c_float, c_float, p, p, p]
    lib.ks_lowpass_scan_backward.restype = c_int32
    lib.ks_ppo_adapt_kl.argtypes = [p, c_int64, c_int32, p, p, c_float, c_float, p, p]
    lib.ks_ppo_adapt_kl.restype = c_int32
    for name in ("ks_gae_bt", "ks_gae_tn", "ks_normalize_advantages", "ks_ppo_loss", "ks_reward_total", "ks_copy_f32"):
        getattr(lib, name).restype = c_int32
    _bind_optional(lib)
    _lib = lib
    return lib


def _bind_optional(lib) -> None:
    from . import _lib_dyn, _lib_terms  # noqa: PLC0415

    _lib_dyn.bind(lib)
    _lib_terms.bind(lib)


def check(rc: int) -> None:
    if rc != 0:
        raise KsError(f"libksimhip error {rc}: {load().ks_last_error().decode()}")


def ptr(t) -> c_void_p:
    """Device pointer of a torch tensor (or None)."""
    if t is None:
        return c_void_p(0)
    return c_void_p(t.data_ptr())


def current_stream() -> c_void_p:
    import torch

    return c_void_p(torch.cuda.current_stream().cuda_stream)


def require_cuda(*tensors, dtype=None):
    import torch

    for t in tensors:
        if t is None:
            continue
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise KsError("ksim_amd kernels take torch tensors resident on the GPU (there is no CPU path)")
        if not t.is_contiguous():
            raise KsError("ksim_amd kernels take contiguous tensors")
        if dtype is not None and t.dtype != dtype:
            raise KsError(f"expected dtype {dtype}, got {t.dtype}")
