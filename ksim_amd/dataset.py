"""On-disk trajectory dataset in the reference's format (ksim/dataset.py:37-173).

A dataset is one float32 memory-mapped matrix `(num_samples, total_size)` plus a `.meta.json` beside it with
`names`, `shapes`, `num_samples`, `total_size`.  A sample is one env's rollout: the leaves listed by the writer,
each flattened and concatenated in that order; nested dicts contribute `"<leaf>.<key>"` entries.  Files written here
can be read by the reference's `TrajectoryDataset` and the other way round.

Rollouts live on the GPU as time-major `(T, N, ...)` tensors; `write_batch` copies a rollout to the host once and
writes its N envs as N samples of shape `(T, ...)`.
"""
from __future__ import annotations

import json
import random
from pathlib import Path
from typing import Mapping

import numpy as np
import torch

from .types import RewardState, Trajectory

_LEAVES = ("xquat", "xpos", "qpos", "qvel", "ctrl", "action", "done", "success", "timestep", "obs", "command",
           "termination_components")  # dataset.py:64-79, in the writer's order; reward and reward_components follow


def recursive_flatten(arr: Mapping, join: str = ".") -> list[tuple[str, object]]:
    """One level of dict nesting flattened to `"outer.inner"` names (dataset.py:26-34)."""
    flat = []
    for k, v in arr.items():
        if isinstance(v, Mapping):
            flat.extend((f"{k}{join}{kk}", vv) for kk, vv in v.items())
        else:
            flat.append((k, v))
    return flat


def _host(x) -> np.ndarray:
    if isinstance(x, torch.Tensor):
        x = x.detach().cpu().numpy()
    return np.asarray(x)


def _sample_dict(trajectory: Trajectory, rewards: RewardState) -> dict:
    sample = {}
    for name in _LEAVES:
        v = getattr(trajectory, name)
        if v is None:
            raise ValueError(f"trajectory.{name} is None: the dataset format stores every leaf")
        sample[name] = {k: vv for k, vv in v.items() if not k.startswith("_")} if isinstance(v, Mapping) else v
    sample["reward"] = rewards.total
    sample["reward_components"] = dict(rewards.components)
    return sample


class TrajectoryDatasetWriter:
    """Context manager that appends samples to a memory-mapped file created on the first write (dataset.py:37-105)."""

    def __init__(self, path: str | Path, num_samples: int) -> None:
        self.path = Path(path)
        self.num_samples = int(num_samples)
        self.path.parent.mkdir(parents=True, exist_ok=True)
        self.fp: np.memmap | None = None
        self.index = 0
        self._names: list[str] | None = None

    def __enter__(self) -> "TrajectoryDatasetWriter":
        return self

    def __exit__(self, exc_type, exc_value, traceback) -> None:
        if self.fp is not None:
            self.fp.flush()
            self.fp = None

    def _open(self, flat: list[tuple[str, np.ndarray]]) -> None:
        total = sum(int(np.prod(v.shape)) for _, v in flat)
        meta = {"names": [n for n, _ in flat], "shapes": [list(v.shape) for _, v in flat],
                "num_samples": self.num_samples, "total_size": total}
        with open(self.path.with_suffix(".meta.json"), "w") as f:
            json.dump(meta, f, indent=2)
        self.fp = np.memmap(self.path, dtype=np.float32, mode="w+", shape=(self.num_samples, total))
        self._names, self._shapes, self.index = meta["names"], meta["shapes"], 0

    def _append(self, flat: list[tuple[str, np.ndarray]]) -> None:
        if self.index >= self.num_samples:
            raise ValueError("Dataset is full")
        if self.fp is None:
            self._open(flat)
        elif [n for n, _ in flat] != self._names or [list(v.shape) for _, v in flat] != self._shapes:
            raise ValueError("sample layout differs from the first sample written to this dataset")
        self.fp[self.index] = np.concatenate([v.astype(np.float32).reshape(-1) for _, v in flat])
        self.index += 1

    def write(self, trajectory: Trajectory, rewards: RewardState) -> None:
        """One sample: leaves of one env, `(T, ...)` each."""
        self._append([(n, _host(v)) for n, v in recursive_flatten(_sample_dict(trajectory, rewards))])

    def write_batch(self, trajectory: Trajectory, rewards: RewardState) -> int:
        """A time-major rollout `(T, N, ...)`: one device-to-host copy per leaf, then env e becomes one sample
        `(T, ...)`.  Stops when the dataset is full; returns the number of samples written."""
        flat = [(n, _host(v)) for n, v in recursive_flatten(_sample_dict(trajectory, rewards))]
        N = flat[0][1].shape[1]
        written = 0
        for e in range(N):
            if self.index >= self.num_samples:
                break
            self._append([(n, v[:, e]) for n, v in flat])
            written += 1
        return written


class TrajectoryDataset:
    """Random-access reader (dataset.py:108-168): `next()` returns one sample and moves to a random index."""

    def __init__(self, path: str | Path, meta_path: str | Path | None = None, rng: random.Random | None = None,
                 device: str | torch.device = "cpu") -> None:
        self.path = Path(path)
        self.meta_path = self.path.with_suffix(".meta.json") if meta_path is None else Path(meta_path)
        self.rng = random.Random(1337) if rng is None else rng
        self.device = device
        with open(self.meta_path, "r") as f:
            self.meta = json.load(f)
        shape = (self.meta["num_samples"], self.meta["total_size"])
        self.ds = np.memmap(self.path, dtype=np.float32, mode="r", shape=shape)
        self.index = self.rng.randint(0, self.meta["num_samples"] - 1)

    def __len__(self) -> int:
        return int(self.meta["num_samples"])

    def get(self, index: int) -> tuple[Trajectory, RewardState]:
        sample = torch.from_numpy(np.array(self.ds[index])).to(self.device)
        arrs: dict[str, torch.Tensor] = {}
        offset = 0
        for name, shape in zip(self.meta["names"], self.meta["shapes"], strict=True):
            n = int(np.prod(shape))
            arrs[name] = sample[offset:offset + n].reshape(tuple(shape))
            offset += n

        def sub(prefix: str) -> dict[str, torch.Tensor]:
            return {k.split(".", 1)[1]: v for k, v in arrs.items() if k.startswith(prefix + ".")}

        # the writer stores no curriculum level, event state, auxiliary outputs or reward carry: they come back empty
        traj = Trajectory(qpos=arrs["qpos"], qvel=arrs["qvel"], xpos=arrs["xpos"], xquat=arrs["xquat"], ctrl=arrs["ctrl"],
                          obs=sub("obs"), command=sub("command"), event_state=sub("event_state"), action=arrs["action"],
                          done=arrs["done"], success=arrs["success"], timestep=arrs["timestep"],
                          curriculum_level=arrs.get("curriculum_level"),
                          termination_components=sub("termination_components"), aux_outputs=sub("aux_outputs"))
        return traj, RewardState(total=arrs["reward"], components=sub("reward_components"), carry=sub("reward_carry"))

    def next(self) -> tuple[Trajectory, RewardState]:
        out = self.get(self.index)
        self.index = self.rng.randint(0, self.meta["num_samples"] - 1)
        return out

    @classmethod
    def writer(cls, path: str | Path, num_samples: int) -> TrajectoryDatasetWriter:
        return TrajectoryDatasetWriter(path, num_samples)
