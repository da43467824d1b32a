"""Reference-motion container and its .npz format (ksim/utils/priors.py:52-143): the real-motion side of the AMP
discriminator.  Keys: `qpos (T, nq)`, `qvel (T, nv)`, `cartesian_pose_body_ids (B)`, `cartesian_poses_stacked
(B, T, 3)`, `ctrl_dt ()`."""
from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Mapping

import numpy as np
import torch


@dataclass(frozen=True)
class MotionReferenceData:
    qpos: np.ndarray                        # (T, nq)
    qvel: np.ndarray                        # (T, nv)
    cartesian_poses: Mapping[int, np.ndarray]  # body id -> (T, 3)
    ctrl_dt: float

    @property
    def num_frames(self) -> int:
        return int(self.qpos.shape[0])

    def _frame(self, step):
        return np.asarray(step) % self.num_frames  # the motion loops (priors.py:67-70)

    def get_qpos_at_step(self, step):
        return np.take(self.qpos, self._frame(step), axis=0)

    def get_qvel_at_step(self, step):
        return np.take(self.qvel, self._frame(step), axis=0)

    def get_cartesian_pose_at_step(self, step) -> dict[int, np.ndarray]:
        f = self._frame(step)
        return {b: np.take(p, f, axis=0) for b, p in self.cartesian_poses.items()}

    def _step_at(self, time):
        return np.int32(np.round(np.asarray(time) / self.ctrl_dt))  # nearest frame (priors.py:86-88)

    def get_qpos_at_time(self, time):
        return self.get_qpos_at_step(self._step_at(time))

    def get_cartesian_pose_at_time(self, time):
        return self.get_cartesian_pose_at_step(self._step_at(time))

    def frames(self, device="cuda") -> torch.Tensor:
        """(T, nq) float32 on the device: the rows a discriminator MLP consumes as "real" motion frames."""
        return torch.as_tensor(np.ascontiguousarray(self.qpos), dtype=torch.float32, device=device)

    def save(self, path: str | Path) -> None:
        p = Path(path)
        p.parent.mkdir(parents=True, exist_ok=True)
        ids = np.array(list(self.cartesian_poses.keys()))
        stacked = np.stack([np.asarray(v) for v in self.cartesian_poses.values()], axis=0) if len(ids) else np.zeros((0, self.num_frames, 3))
        np.savez(p, qpos=np.asarray(self.qpos), qvel=np.asarray(self.qvel), cartesian_pose_body_ids=ids,
                 cartesian_poses_stacked=stacked, ctrl_dt=np.array(self.ctrl_dt))

    @classmethod
    def load(cls, path: str | Path) -> "MotionReferenceData":
        p = Path(path)
        if not p.exists():
            raise FileNotFoundError(f"Reference motion file not found: {p}")
        with np.load(p, allow_pickle=False) as data:
            ids, stacked = data["cartesian_pose_body_ids"], data["cartesian_poses_stacked"]
            return cls(qpos=np.array(data["qpos"]), qvel=np.array(data["qvel"]),
                       cartesian_poses={int(b): np.array(stacked[i]) for i, b in enumerate(ids)},
                       ctrl_dt=float(data["ctrl_dt"].item()))
