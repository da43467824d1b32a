"""Random variables, noises and biases with the reference's names (ksim/noise.py:50-229).

Objects here only carry parameters; the draws happen in the HIP kernels (explicit buffers or the
in-kernel Philox stream).  ``scale`` is the std (Gaussian) or magnitude (uniform) that the kernels
multiply by the curriculum level (noise.py:86,102).
"""
from __future__ import annotations

from dataclasses import dataclass

from . import _lib_terms as T


@dataclass(frozen=True)
class Noise:
    kind: int = T.NOISE_NONE
    mean: float = 0.0
    scale: float = 0.0


class NoNoise(Noise):
    def __init__(self) -> None:
        super().__init__(T.NOISE_NONE, 0.0, 0.0)


class AdditiveGaussianNoise(Noise):  # noise.py:196-198
    def __init__(self, std: float, mean: float = 0.0) -> None:
        if std < 0:
            raise ValueError("std must be non-negative")
        super().__init__(T.NOISE_ADD_GAUSSIAN, mean, std)


class AdditiveUniformNoise(Noise):  # noise.py:206-208
    def __init__(self, mag: float, mean: float = 0.0) -> None:
        if mag < 0:
            raise ValueError("mag must be non-negative")
        super().__init__(T.NOISE_ADD_UNIFORM, mean, mag)


class MultiplicativeGaussianNoise(Noise):  # noise.py:201-203
    def __init__(self, std: float, mean: float = 1.0) -> None:
        super().__init__(T.NOISE_MUL_GAUSSIAN, mean, std)


class MultiplicativeUniformNoise(Noise):  # noise.py:211-213
    def __init__(self, mag: float, mean: float = 1.0) -> None:
        super().__init__(T.NOISE_MUL_UNIFORM, mean, mag)


@dataclass(frozen=True)
class RandomVariable:
    """UniformRandomVariable / GaussianRandomVariable (noise.py:74-102) as parameters for init-time draws."""
    mean: float = 0.0
    mag: float = 0.0
    std: float = 0.0

    def sample(self, shape, gen, level: float = 1.0):
        import torch

        out = torch.full(shape, float(self.mean), dtype=torch.float32, device=gen.device)
        if self.mag:
            out += (torch.rand(shape, generator=gen, device=gen.device) * 2 - 1) * (self.mag * level)
        if self.std:
            out += torch.randn(shape, generator=gen, device=gen.device) * (self.std * level)
        return out


def UniformRandomVariable(mean: float, mag: float) -> RandomVariable:
    return RandomVariable(mean=mean, mag=mag)


def GaussianRandomVariable(mean: float, std: float) -> RandomVariable:
    return RandomVariable(mean=mean, std=std)


def convert_to_noise(noise) -> Noise | None:
    """A float means additive Gaussian noise of that std (ksim/observation.py:69-76)."""
    if noise is None or isinstance(noise, Noise):
        return noise
    if isinstance(noise, float):
        return AdditiveGaussianNoise(std=noise)
    raise ValueError(f"Invalid noise: {noise}")
