"""AMP discriminator update on the GPU against the float64 oracle (ksim/task/amp.py:360-545)."""
import numpy as np
import pytest
import torch

from oracle import amp as oamp
from oracle import ppo_update as oup

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GRAD_TOL = 2e-4   # fp32 products against float64, relative to the largest entry of each gradient
LOSS_TOL = 1e-5


def _params(dims, seed):
    rng = np.random.default_rng(seed)
    ws = [(rng.normal(size=(o, i)) / np.sqrt(i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    bs = [(rng.normal(size=o) * 0.1).astype(np.float32) for o in dims[1:]]
    return ws, bs


def _check(disc, ws, bs, real, sim, coef, act):
    losses = disc.disc_loss_grad(torch.tensor(real, device=DEV), torch.tensor(sim, device=DEV), coef).cpu().numpy()
    want_l, want_g = oamp.disc_loss_and_grads(ws, bs, real, sim, coef, act=act)
    np.testing.assert_allclose(losses, want_l, rtol=LOSS_TOL, atol=1e-6)
    for l, ((gw, gb), (ww, wb)) in enumerate(zip(disc.parameters(gradients=True), want_g)):
        for name, got, want in (("weight", gw, ww), ("bias", gb, wb)):
            err = np.abs(got.cpu().numpy() - want).max() / max(np.abs(want).max(), 1e-6)
            assert err <= GRAD_TOL, f"layer {l} {name}: {err:.2e}"
    return losses


@pytest.mark.parametrize("act,dims,dtype", [("elu", [37, 96, 64, 1], "f32"), ("tanh", [12, 50, 1], "f32"), ("relu", [20, 33, 17, 1], "f32"),
                                            ("elu", [5, 1], "f32"), ("elu", [24, 128, 128, 1], "bf16")])
def test_discriminator_loss_gradient_matches_oracle(act, dims, dtype):
    """Squared-error terms and the gradient penalty (which differentiates the network twice); ragged widths, a linear
    network, and a bf16 network (the update itself runs on the fp32 master weights)."""
    from ksim_amd.mlp import MLP

    ws, bs = _params(dims, seed=len(dims) * 7 + dims[0])
    disc = MLP(ws, bs, activation=act, dtype=dtype)
    disc.train_init()
    rng = np.random.default_rng(5)
    real = rng.normal(size=(6, 11, dims[0])).astype(np.float32)
    sim = rng.normal(size=(4, 9, dims[0])).astype(np.float32)
    l1 = _check(disc, ws, bs, real, sim, 10.0, act)
    assert l1[2] > 1e-3
    # a second call on fewer rows reuses the workspace and overwrites the gradients; no penalty this time
    l0 = _check(disc, ws, bs, real[:2], sim[:1], 0.0, act)
    assert l0[2] == 0.0


@pytest.mark.parametrize("dims", [[30, 64, 1], [30, 256, 130, 1]])
def test_discriminator_many_rows_split_reduction(dims):
    """Enough frames that the weight-gradient products cut their row range into slices; with layers of 128 units and more
    they run on the wide tiles, the bias gradients summed in the same pass (a width that ends inside a tile included)."""
    from ksim_amd.mlp import MLP

    ws, bs = _params(dims, seed=3)
    disc = MLP(ws, bs, activation="elu", dtype="f32")
    disc.train_init()
    rng = np.random.default_rng(8)
    real = rng.normal(size=(32, 100, 30)).astype(np.float32)
    sim = rng.normal(size=(32, 100, 30)).astype(np.float32)
    _check(disc, ws, bs, real, sim, 10.0, "elu")


def test_discriminator_update_learns_and_matches_oracle_steps():
    """Three optimiser steps on fixed batches against the oracle's Adam (the optax chain restated for the policy update),
    then the loop with sampled batches: the loss on separable data goes down."""
    from ksim_amd import amp
    from ksim_amd.mlp import MLP

    dims = [8, 32, 1]
    ws, bs = _params(dims, seed=21)
    disc = MLP(ws, bs, activation="elu", dtype="f32")
    cfg = amp.AMPConfig(amp_reference_batch_size=4, disc_num_passes=2, amp_grad_penalty_coef=5.0, learning_rate=1e-2, max_grad_norm=1.0)
    upd = amp.DiscriminatorUpdate(disc, cfg)
    rng = np.random.default_rng(2)
    real = (rng.normal(size=(4, 6, 8)) + 1.0).astype(np.float32)
    sim = (rng.normal(size=(4, 6, 8)) - 1.0).astype(np.float32)
    # oracle: gradient, global-norm clip, Adam with bias correction
    pw, pb = [w.astype(np.float64) for w in ws], [b.astype(np.float64) for b in bs]
    m1 = [np.zeros_like(p) for p in pw + pb]; m2 = [np.zeros_like(p) for p in pw + pb]
    for step in range(1, 4):
        upd.step(torch.tensor(real, device=DEV), torch.tensor(sim, device=DEV))
        _, g = oamp.disc_loss_and_grads(pw, pb, real, sim, cfg.amp_grad_penalty_coef, act="elu")
        flat = [gw for gw, _ in g] + [gb for _, gb in g]
        norm = np.sqrt(sum((x ** 2).sum() for x in flat))
        flat = [x * min(1.0, cfg.max_grad_norm / norm) for x in flat]
        for i, (p, x) in enumerate(zip(pw + pb, flat)):
            m1[i] = 0.9 * m1[i] + 0.1 * x
            m2[i] = 0.999 * m2[i] + 0.001 * x * x
            p -= cfg.learning_rate * (m1[i] / (1 - 0.9 ** step)) / (np.sqrt(m2[i] / (1 - 0.999 ** step)) + 1e-8)
    for (gw, gb), w, b in zip(disc.parameters(), pw, pb):
        np.testing.assert_allclose(gw.cpu().numpy(), w, rtol=0, atol=2e-4)
        np.testing.assert_allclose(gb.cpu().numpy(), b, rtol=0, atol=2e-4)
    # the network that the rollout's forward pass uses follows the master weights
    x = torch.tensor(real.reshape(-1, 8), device=DEV)
    want = oup.mlp(torch.tensor(real.reshape(-1, 8), dtype=torch.float64), [torch.tensor(w) for w in pw], [torch.tensor(b) for b in pb]).numpy()
    np.testing.assert_allclose(disc(x).cpu().numpy(), want, rtol=0, atol=1e-3)

    gen = torch.Generator().manual_seed(0)
    clips = torch.tensor((rng.normal(size=(5, 4, 8)) + 1.0).astype(np.float32), device=DEV)   # clips shorter than the window: they loop
    sims = torch.tensor((rng.normal(size=(16, 6, 8)) - 1.0).astype(np.float32), device=DEV)
    first = upd.update(clips, sims, gen)
    for _ in range(30):
        last = upd.update(clips, sims, gen)
    assert float(last["disc_loss"]) < 0.5 * float(first["disc_loss"])
    assert set(last) == {"disc_loss", "disc_real_loss", "disc_sim_loss", "disc_gp_loss"}


def test_discriminator_argument_errors():
    from ksim_amd import _lib, amp
    from ksim_amd.mlp import MLP

    ws, bs = _params([6, 8, 2], seed=1)
    two = MLP(ws, bs, activation="elu", dtype="f32")
    with pytest.raises(_lib.KsError, match="one number"):
        amp.DiscriminatorUpdate(two, amp.AMPConfig())
    ws, bs = _params([6, 8, 1], seed=1)
    gelu = MLP(ws, bs, activation="gelu", dtype="f32")
    gelu.train_init()
    x = torch.zeros(2, 3, 6, device=DEV)
    with pytest.raises(_lib.KsError, match="GELU"):
        gelu.disc_loss_grad(x, x, 1.0)
    with pytest.raises(ValueError, match="must divide"):
        amp.make_sim_batch(torch.zeros(10, 3, 6, device=DEV), 4, torch.Generator())
    w = amp.loop_slice(torch.arange(3, device=DEV), 2, 5)
    assert w.tolist() == [2, 0, 1, 2, 0]
    # a batch of reference windows is those slices, of the clips and starts the generator draws, gathered at once
    motions = torch.arange(4 * 7 * 2, device=DEV, dtype=torch.float32).reshape(4, 7, 2)
    batch = amp.make_real_batch(motions, 10, 6, torch.Generator().manual_seed(5))
    g = torch.Generator().manual_seed(5)
    clips, starts = torch.randint(0, 4, (6,), generator=g), torch.randint(0, 7, (6,), generator=g)
    want = torch.stack([amp.loop_slice(motions[int(c)], int(s0), 10) for c, s0 in zip(clips, starts)])
    assert batch.shape == (6, 10, 2) and torch.equal(batch, want)
