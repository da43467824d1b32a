"""Curriculum scales (ksim/scales.py:21-117): maps from the curriculum level to a multiplier.  They are evaluated
on the host, once per launch, and the kernels receive the resulting float."""
from __future__ import annotations

import math
from dataclasses import dataclass


class Scale:
    def get_scale(self, curriculum_level: float) -> float:
        raise NotImplementedError


def _check(scale: float, bias: float) -> None:
    if bias < 0.0:
        raise ValueError(f"bias must be non-negative, got {bias}")
    if scale + bias < 0.0:
        raise ValueError(f"scale + bias must be non-negative, got {scale} + {bias} = {scale + bias}")


@dataclass(frozen=True, kw_only=True)
class ConstantScale(Scale):  # scales.py:28-35
    scale: float

    def __post_init__(self):
        if self.scale < 0.0:
            raise ValueError("scale must be non-negative")

    def get_scale(self, curriculum_level: float) -> float:
        return float(self.scale)


@dataclass(frozen=True, kw_only=True)
class _Affine(Scale):
    scale: float
    bias: float = 0.0

    def __post_init__(self):
        _check(self.scale, self.bias)

    @classmethod
    def from_endpoints(cls, start: float, end: float):
        return cls(scale=end - start, bias=start)


class LinearScale(_Affine):  # scales.py:38-56
    def get_scale(self, curriculum_level: float) -> float:
        return self.scale * float(curriculum_level) + self.bias


class QuadraticScale(_Affine):  # scales.py:59-77
    def get_scale(self, curriculum_level: float) -> float:
        return self.scale * float(curriculum_level) ** 2 + self.bias


class SquareRootScale(_Affine):  # scales.py:80-96
    def get_scale(self, curriculum_level: float) -> float:
        return self.scale * math.sqrt(float(curriculum_level)) + self.bias


@dataclass(frozen=True, kw_only=True)
class NonZeroScale(Scale):  # scales.py:99-107: the scale once the curriculum has left level zero, else the bias
    scale: float
    bias: float = 0.0

    def __post_init__(self):
        if self.bias < 0.0:
            raise ValueError("bias must be non-negative")

    def get_scale(self, curriculum_level: float) -> float:
        return float(self.scale if curriculum_level > 0.0 else self.bias)


def convert_to_scale(value) -> Scale:  # scales.py:110-115
    if isinstance(value, (float, int)) and not isinstance(value, bool):
        return ConstantScale(scale=float(value))
    if isinstance(value, Scale):
        return value
    raise ValueError(f"Invalid scale: {value}")
