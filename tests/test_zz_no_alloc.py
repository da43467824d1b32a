"""The allocation-free variant of advantage normalisation against the workspace-taking entry point (through the C ABI).

Two calls in a row on the same GPU, the second with a smaller input: the library's own scratch array keeps the first
call's partial sums, and the second call must not read any of them.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(lib, _lib, x):
    n = x.numel()
    want = torch.empty_like(x)
    got = torch.full_like(x, float("nan"))
    ws = torch.empty(_lib.KS_REDUCE_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
    _lib.check(lib.ks_normalize_advantages(_lib.current_stream(), n, _lib.ptr(x), _lib.ptr(want), _lib.ptr(ws)))
    _lib.check(lib.ks_normalize_advantages_static(_lib.current_stream(), n, _lib.ptr(x), _lib.ptr(got)))
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_variant_matches_on_two_calls_the_second_smaller():
    from ksim_amd import _lib

    lib = _lib.load()
    rng = np.random.default_rng(77)
    # 4096 x 128 fills 512 block partials; the second call uses 3 of them and a different mean and deviation
    big = torch.from_numpy((rng.normal(size=4096 * 128) * 3.0 + 5.0).astype(np.float32)).to("cuda:0")
    small = torch.from_numpy((rng.normal(size=2500) * 0.2 - 1.0).astype(np.float32)).to("cuda:0")
    for x in (big, small):
        got, want = _both(lib, _lib, x)
        assert torch.equal(got, want)  # same kernels, same partial order: bit-equal
        xs = x.cpu().numpy().astype(np.float64)
        ref = (xs - xs.mean()) / max(xs.std(), 1e-6)  # ksim/task/ppo.py:116-119
        assert np.abs(got.cpu().numpy() - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())


def test_static_scratch_variant_rejects_oversize_and_bad_arguments():
    from ksim_amd import _lib

    lib = _lib.load()
    x = torch.zeros(8, device="cuda:0")
    rc = lib.ks_normalize_advantages_static(_lib.current_stream(), (1 << 28) + 1, _lib.ptr(x), _lib.ptr(x))
    assert rc == -3 and b"maximum" in lib.ks_last_error()
    assert lib.ks_normalize_advantages_static(_lib.current_stream(), -1, _lib.ptr(x), _lib.ptr(x)) == -1
    assert lib.ks_normalize_advantages_static(_lib.current_stream(), 8, ctypes.c_void_p(0), _lib.ptr(x)) == -1
    assert lib.ks_normalize_advantages_static(_lib.current_stream(), 0, ctypes.c_void_p(0), ctypes.c_void_p(0)) == 0
