"""MLP forward on the matrix cores against a float64 torch reference (F.linear + F.elu)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def reference(x, ws, bs, act, bf16):
    """float64 library reference; for the bf16 path weights and layer inputs are rounded to bf16 first."""
    rnd = (lambda t: t.to(torch.bfloat16).to(torch.float64)) if bf16 else (lambda t: t.to(torch.float64))
    h = torch.from_numpy(x)
    fn = {"elu": F.elu, "relu": F.relu, "tanh": torch.tanh, None: lambda t: t, "none": lambda t: t}[act]
    for i, (w, b) in enumerate(zip(ws, bs)):
        h = F.linear(rnd(h.to(torch.float32)), rnd(torch.from_numpy(w)), torch.from_numpy(b).to(torch.float64))
        if i + 1 < len(ws):
            h = fn(h)
    return h.numpy()


@pytest.mark.parametrize("dims,dtype,act,M", [
    ((71, 256, 256, 256, 21), "f32", "elu", 300),      # benchmark config 3 actor
    ((68, 512, 512, 512, 20), "bf16", "elu", 1000),    # config 4 actor
    ((68, 512, 512, 512, 1), "bf16", "elu", 129),      # config 4 critic, ragged tile
    ((71, 256, 256, 1), "bf16", "relu", 64),           # config 5 discriminator shape
    ((5, 3), "f32", None, 7), ((40, 100, 9), "f32", "tanh", 1), ((33, 130, 130, 2), "bf16", "tanh", 257),
    ((68, 512, 512, 512, 20), "bf16", "elu", 16384 + 45),   # 64-row tiles of the whole-network kernel
    ((68, 512, 512, 512, 20), "bf16", "elu", 32768 + 77),   # 128-row tiles
    ((71, 256, 256, 1), "bf16", "relu", 40000),             # 128-row tiles, one output tile per wavefront
    ((64, 1024, 8), "bf16", "elu", 500),                    # wider than the whole-network kernel takes: per-layer path
    ((600, 64, 3), "bf16", "none", 100),
])
def test_mlp_matches_reference(dims, dtype, act, M):
    from ksim_amd.mlp import MLP

    rng = np.random.default_rng(sum(dims) + M)
    ws = [rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.normal(scale=0.1, size=o).astype(np.float32) for o in dims[1:]]
    x = rng.normal(size=(M, dims[0])).astype(np.float32)
    net = MLP(ws, bs, activation=act if act not in (None, "none") else "none", dtype=dtype)
    y = net(torch.from_numpy(x).to(DEV)).cpu().numpy()
    want = reference(x, ws, bs, act, dtype == "bf16")
    scale = np.abs(want).max()
    # f32: fp32 accumulation error only; bf16: inputs rounded identically, so only accumulation order differs,
    # plus re-rounding of hidden activations that land on a bf16 tie
    tol = 2e-5 if dtype == "f32" else 6e-3
    assert np.abs(y - want).max() <= tol * scale, np.abs(y - want).max() / scale
    assert net.flops_per_row() == 2 * sum(a * b for a, b in zip(dims[:-1], dims[1:]))


def test_mlp_rows_are_independent_and_errors():
    from ksim_amd import _lib
    from ksim_amd.mlp import random_mlp

    net, ws, bs = random_mlp((68, 512, 512, 512, 20), seed=3)
    x = torch.randn(700, 68, device=DEV)
    y = net(x)
    y2 = net(x[123:460].contiguous())
    assert torch.equal(y[123:460], y2)
    big = torch.randn(33000, 68, device=DEV)  # another row tile size, same bits per row
    assert torch.equal(net(big)[5000:5700], net(big[5000:5700].contiguous()))
    with pytest.raises(_lib.KsError):
        net(torch.randn(4, 67, device=DEV))
    with pytest.raises(_lib.KsError):
        net(torch.randn(4, 68))
    assert net(torch.empty(0, 68, device=DEV)).shape == (0, 20)


@pytest.mark.parametrize("M", [8192, 777, 20000])
def test_paired_forward_equals_two_single_forwards(M):
    """Actor and critic over the same rows in one launch (below 16384 rows) or two: bit-identical to separate calls,
    also for networks of different widths and for a pair that cannot share a launch."""
    from ksim_amd import _lib
    from ksim_amd.mlp import random_mlp

    actor, _, _ = random_mlp((68, 512, 512, 512, 20), seed=5)
    critic, _, _ = random_mlp((68, 512, 512, 512, 1), seed=6)
    narrow, _, _ = random_mlp((68, 256, 256, 1), seed=7)
    wide, _, _ = random_mlp((68, 1024, 1), seed=8)  # per-layer path: the pair falls back to two launches
    x0, x1 = torch.randn(M, 68, device=DEV), torch.randn(M, 68, device=DEV)
    for other in (critic, narrow, wide):
        y0 = torch.full((M, 20), 7.0, device=DEV)
        y1 = torch.full((M, 1), 7.0, device=DEV)
        actor.forward_pair(x0, y0, other, x1, y1)
        assert torch.equal(y0, actor(x0)) and torch.equal(y1, other(x1))
    with pytest.raises(_lib.KsError):
        actor.forward_pair(x0, torch.empty(M, 20, device=DEV), critic, x1[:-1], torch.empty(M - 1, 1, device=DEV))
