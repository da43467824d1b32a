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
    scale2: float = 0.0  # mag of the uniform part of the uniform-Gaussian kinds

    def stages(self) -> tuple["Noise", ...]:
        """The stages the kernel applies in order, all with the same draws (one stage unless chained)."""
        return () if self.kind == T.NOISE_NONE else (self,)


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
        if std < 0:
            raise ValueError("std must be non-negative")
        super().__init__(T.NOISE_MUL_GAUSSIAN, mean, std)


class MultiplicativeUniformNoise(Noise):  # noise.py:211-213
    def __init__(self, mag: float, mean: float = 1.0) -> None:
        if mag < 0:
            raise ValueError("mag must be non-negative")
        super().__init__(T.NOISE_MUL_UNIFORM, mean, mag)


class AdditiveUniformGaussianNoise(Noise):
    """AdditiveNoise over a UniformGaussianRandomVariable (noise.py:106-121,184-187): mean + normal + uniform, both parts
    drawn with one key."""
    def __init__(self, std: float, mag: float, mean: float = 0.0) -> None:
        if std < 0 or mag < 0:
            raise ValueError("std and mag must be non-negative")
        super().__init__(T.NOISE_ADD_UNIFORM_GAUSSIAN, mean, std, mag)


class MultiplicativeUniformGaussianNoise(Noise):
    def __init__(self, std: float, mag: float, mean: float = 1.0) -> None:
        if std < 0 or mag < 0:
            raise ValueError("std and mag must be non-negative")
        super().__init__(T.NOISE_MUL_UNIFORM_GAUSSIAN, mean, std, mag)


class ChainedNoise(Noise):  # noise.py:222-229: every noise of the chain is applied with the same key
    def __init__(self, noises) -> None:
        noises = tuple(noises)
        flat = tuple(st for n in noises for st in n.stages())
        if len(flat) > T.KS_MAX_NOISE_CHAIN:
            raise ValueError(f"at most {T.KS_MAX_NOISE_CHAIN} chained noises")
        super().__init__(T.NOISE_NONE, 0.0, 0.0)
        object.__setattr__(self, "noises", flat)

    def stages(self):
        return self.noises


# Per-episode biases (noise.py:129-170): the same kinds, drawn once per episode.
class Bias(Noise):
    pass


class NoBias(Bias):
    def __init__(self) -> None:
        super().__init__(T.NOISE_NONE, 0.0, 0.0)


class AdditiveGaussianBias(Bias):  # noise.py:148-150
    def __init__(self, std: float, mean: float = 0.0) -> None:
        if std < 0:
            raise ValueError("std must be non-negative")
        super().__init__(T.NOISE_ADD_GAUSSIAN, mean, std)


class MultiplicativeGaussianBias(Bias):  # noise.py:153-155
    def __init__(self, std: float, mean: float = 1.0) -> None:
        if std < 0:
            raise ValueError("std must be non-negative")
        super().__init__(T.NOISE_MUL_GAUSSIAN, mean, std)


class AdditiveUniformBias(Bias):  # noise.py:158-160
    def __init__(self, mag: float, mean: float = 0.0) -> None:
        if mag < 0:
            raise ValueError("mag must be non-negative")
        super().__init__(T.NOISE_ADD_UNIFORM, mean, mag)


class MultiplicativeUniformBias(Bias):  # noise.py:163-165
    def __init__(self, mag: float, mean: float = 1.0) -> None:
        if mag < 0:
            raise ValueError("mag must be non-negative")
        super().__init__(T.NOISE_MUL_UNIFORM, mean, mag)


@dataclass(frozen=True)
class RandomVariable:
    """ZeroRandomVariable / UniformRandomVariable / GaussianRandomVariable / UniformGaussianRandomVariable
    (noise.py:62-121) as parameters: value = mean + level (std z + mag w).  `same_key`: both parts come from one key."""
    mean: float = 0.0
    mag: float = 0.0
    std: float = 0.0
    same_key: bool = False

    def __post_init__(self):
        if self.mag < 0 or self.std < 0:
            raise ValueError("mag and std must be non-negative")

    def desc(self) -> T.KsRandomVar:
        return T.KsRandomVar(float(self.mean), float(self.mag), float(self.std), int(self.same_key))

    def sample(self, shape, gen, level: float = 1.0):
        """Host-side draw with torch's generator (for code that wants values outside the kernels)."""
        import torch

        out = torch.full(shape, float(self.mean), dtype=torch.float32, device=gen.device)
        z = torch.randn(shape, generator=gen, device=gen.device) if (self.std or self.same_key) else None
        if self.std:
            out += z * (self.std * level)
        if self.mag:
            w = torch.erf(z * 0.7071067811865476) if self.same_key else torch.rand(shape, generator=gen, device=gen.device) * 2 - 1
            out += w * (self.mag * level)
        return out


def ZeroRandomVariable() -> RandomVariable:
    return RandomVariable()


def UniformRandomVariable(mean: float, mag: float) -> RandomVariable:
    return RandomVariable(mean=mean, mag=mag)


def GaussianRandomVariable(mean: float, std: float) -> RandomVariable:
    return RandomVariable(mean=mean, std=std)


def UniformGaussianRandomVariable(mean: float, std: float, mag: float) -> RandomVariable:
    return RandomVariable(mean=mean, mag=mag, std=std, same_key=True)


def _kind_of(rv: RandomVariable, additive: bool) -> tuple[int, float, float, float]:
    """(kind, mean, scale, scale2) of `observation (+ | *) rv` for the kernels' noise stages."""
    if rv.std and rv.mag:
        if not rv.same_key:
            raise ValueError("a normal and a uniform part are drawn with one key (UniformGaussianRandomVariable, noise.py:106-121)")
        return (T.NOISE_ADD_UNIFORM_GAUSSIAN if additive else T.NOISE_MUL_UNIFORM_GAUSSIAN), rv.mean, rv.std, rv.mag
    if rv.mag:
        return (T.NOISE_ADD_UNIFORM if additive else T.NOISE_MUL_UNIFORM), rv.mean, rv.mag, 0.0
    return (T.NOISE_ADD_GAUSSIAN if additive else T.NOISE_MUL_GAUSSIAN), rv.mean, rv.std, 0.0  # a zero variable: the mean alone


class AdditiveNoise(Noise):  # noise.py:184-187: observation + random variable, over any of the random variables above
    def __init__(self, random_variable: RandomVariable) -> None:
        super().__init__(*_kind_of(random_variable, True))


class MultiplicativeNoise(Noise):  # noise.py:190-193
    def __init__(self, random_variable: RandomVariable) -> None:
        super().__init__(*_kind_of(random_variable, False))


class AdditiveBias(Bias):  # noise.py:135-138
    def __init__(self, random_variable: RandomVariable) -> None:
        super().__init__(*_kind_of(random_variable, True))


class MultiplicativeBias(Bias):  # noise.py:141-144
    def __init__(self, random_variable: RandomVariable) -> None:
        super().__init__(*_kind_of(random_variable, False))


def convert_to_noise(noise) -> Noise | None:
    """A float means additive Gaussian noise of that std (ksim/observation.py:69-76)."""
    if noise is None or isinstance(noise, Noise):
        return noise
    if isinstance(noise, float):
        return AdditiveGaussianNoise(std=noise)
    raise ValueError(f"Invalid noise: {noise}")


def convert_to_bias(bias) -> Bias | None:
    """A float means an additive Gaussian bias of that std (ksim/observation.py:79-86)."""
    if bias is None or isinstance(bias, Bias):
        return bias
    if isinstance(bias, float):
        return AdditiveGaussianBias(std=bias)
    raise ValueError(f"Invalid bias: {bias}")
