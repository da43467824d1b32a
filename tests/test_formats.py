"""Disk formats on either side of the rollout path: the trajectory dataset (float32 memory map + .meta.json) and the
reference-motion .npz.  CPU only; layouts are checked against the format the reference's writer produces
(ksim/dataset.py:60-104, ksim/utils/priors.py:91-111), stated here field by field."""
import json

import numpy as np
import pytest
import torch

from ksim_amd.dataset import TrajectoryDataset, recursive_flatten
from ksim_amd.priors import MotionReferenceData
from ksim_amd.types import RewardState, Trajectory


def _rollout(T, N, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    done = torch.rand(T, N, generator=g) < 0.1
    traj = Trajectory(qpos=r(T, N, 9), qvel=r(T, N, 8), xpos=r(T, N, 6), xquat=r(T, N, 8), ctrl=r(T, N, 2),
                      obs={"obs": r(T, N, 5), "noisy_obs": r(T, N, 5)}, command={"_buffer": r(T, N, 2), "vel": r(T, N, 1)},
                      event_state={}, action=r(T, N, 2), done=done, success=done & (torch.rand(T, N, generator=g) < 0.5),
                      timestep=r(T, N).abs(), termination_components={"fell": torch.randint(-1, 2, (T, N), generator=g).to(torch.int8)})
    rew = RewardState(total=r(T, N), components={"alive": r(T, N), "gait/air": r(T, N)}, carry={})
    return traj, rew


def test_trajectory_dataset_layout_and_round_trip(tmp_path):
    T, N = 6, 5
    path = tmp_path / "sub" / "data.bin"
    traj, rew = _rollout(T, N, 0)
    traj2, rew2 = _rollout(T, N, 1)
    with TrajectoryDataset.writer(path, num_samples=8) as w:
        assert w.write_batch(traj, rew) == 5
        assert w.write_batch(traj2, rew2) == 3  # full after eight samples
        with pytest.raises(ValueError, match="full"):
            w.write(traj, rew)
    meta = json.loads(path.with_suffix(".meta.json").read_text())
    # the reference writer's leaf order, nested dicts as "leaf.key", one sample = one env's (T, ...) leaves
    assert meta["names"] == ["xquat", "xpos", "qpos", "qvel", "ctrl", "action", "done", "success", "timestep", "obs.obs",
                             "obs.noisy_obs", "command.vel", "termination_components.fell", "reward",
                             "reward_components.alive", "reward_components.gait/air"]
    assert meta["shapes"][:3] == [[T, 8], [T, 6], [T, 9]] and meta["shapes"][6] == [T] and meta["num_samples"] == 8
    assert meta["total_size"] == sum(int(np.prod(s)) for s in meta["shapes"])
    raw = np.fromfile(path, dtype=np.float32)
    assert raw.size == 8 * meta["total_size"]
    # first floats of sample 3 are env 3's xquat of the first rollout, row-major over (T, 8)
    np.testing.assert_array_equal(raw.reshape(8, -1)[3, :T * 8], traj.xquat[:, 3].reshape(-1).numpy())
    ds = TrajectoryDataset(path)
    assert len(ds) == 8
    for idx, (src_t, src_r, e) in {0: (traj, rew, 0), 4: (traj, rew, 4), 6: (traj2, rew2, 1)}.items():
        t, r = ds.get(idx)
        assert torch.equal(t.qpos, src_t.qpos[:, e]) and torch.equal(t.obs["noisy_obs"], src_t.obs["noisy_obs"][:, e])
        assert torch.equal(t.done, src_t.done[:, e].float()) and torch.equal(t.success, src_t.success[:, e].float())
        assert torch.equal(t.termination_components["fell"], src_t.termination_components["fell"][:, e].float())
        assert torch.equal(r.total, src_r.total[:, e]) and torch.equal(r.components["gait/air"], src_r.components["gait/air"][:, e])
        assert t.command.keys() == {"vel"} and t.event_state == {} and t.curriculum_level is None and r.carry == {}
    a, b = TrajectoryDataset(path).next(), TrajectoryDataset(path).next()
    assert torch.equal(a[0].qpos, b[0].qpos)  # the default sampler is seeded (1337), like the reference's
    with TrajectoryDataset.writer(tmp_path / "d2.bin", num_samples=10) as w:
        w.write_batch(traj, rew)
        short, rs = _rollout(T - 1, N, 2)
        with pytest.raises(ValueError, match="layout"):
            w.write_batch(short, rs)
    assert recursive_flatten({"a": 1, "b": {"c": 2, "d": 3}}) == [("a", 1), ("b.c", 2), ("b.d", 3)]


def test_motion_reference_npz_round_trip(tmp_path):
    rng = np.random.default_rng(0)
    T = 7
    ref = MotionReferenceData(qpos=rng.normal(size=(T, 9)), qvel=rng.normal(size=(T, 8)),
                              cartesian_poses={3: rng.normal(size=(T, 3)), 11: rng.normal(size=(T, 3))}, ctrl_dt=0.02)
    p = tmp_path / "motions" / "walk.npz"
    ref.save(p)
    with np.load(p) as z:  # the reference's keys and shapes
        assert sorted(z.files) == ["cartesian_pose_body_ids", "cartesian_poses_stacked", "ctrl_dt", "qpos", "qvel"]
        assert z["cartesian_poses_stacked"].shape == (2, T, 3) and z["cartesian_pose_body_ids"].tolist() == [3, 11]
        assert z["ctrl_dt"].shape == () and float(z["ctrl_dt"]) == 0.02
    back = MotionReferenceData.load(p)
    np.testing.assert_array_equal(back.qpos, ref.qpos)
    np.testing.assert_array_equal(back.cartesian_poses[11], ref.cartesian_poses[11])
    assert back.num_frames == T and back.ctrl_dt == 0.02
    # frame lookup wraps around; time lookup rounds to the nearest control step
    np.testing.assert_array_equal(back.get_qpos_at_step(T + 2), ref.qpos[2])
    np.testing.assert_array_equal(back.get_qvel_at_step(np.array([0, 8])), ref.qvel[[0, 1]])
    np.testing.assert_array_equal(back.get_qpos_at_time(0.051), ref.qpos[3])
    np.testing.assert_array_equal(back.get_cartesian_pose_at_time(0.02 * 9)[3], ref.cartesian_poses[3][2])
    with pytest.raises(FileNotFoundError):
        MotionReferenceData.load(tmp_path / "missing.npz")
