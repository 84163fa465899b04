"""Initialisers: src/module/init/{mod,he,xavier,sigma}.rs.

``weight(input_size, output_size)`` returns shape (output_size, input_size); ``bias`` defaults
to zeros of shape (1, output_size).  The reference draws from an unseedable thread RNG; here the
values come from the backend's counter-based generator, seeded from the OS unless a seed is given,
and are produced directly in device memory.
"""
import itertools
import math
import os

_stream_counter = itertools.count(1)


def _fresh_seed():
    return int.from_bytes(os.urandom(8), "little")


class InitParameters:
    """src/module/init/mod.rs:11-18."""

    def weight(self, input_size, output_size, engine):
        raise NotImplementedError

    def bias(self, input_size, output_size, engine):
        return engine.zeros(1, output_size)


class Normal(InitParameters):
    """src/module/init/sigma.rs:7-37: N(mean, std)."""

    def __init__(self, mean=0.0, std=1.0, seed=None):
        if not math.isfinite(std):
            raise ValueError("std must be finite")
        self.mean, self.std = float(mean), float(std)
        self.seed = seed

    @classmethod
    def new(cls, mean, std):
        return cls(mean, std) if math.isfinite(std) else None

    @classmethod
    def new_std(cls, std):
        return cls.new(0.0, std)

    def _sigma(self, input_size, output_size):
        return self.std

    def weight(self, input_size, output_size, engine):
        seed = self.seed if self.seed is not None else _fresh_seed()
        return engine.normal(output_size, input_size, seed, next(_stream_counter), self.mean,
                             self._sigma(input_size, output_size))


class KaimingNormal(Normal):
    """src/module/init/he.rs:9-15: sigma = 1 / sqrt(input_size)."""

    def __init__(self, seed=None):
        super().__init__(0.0, 1.0, seed)

    def _sigma(self, input_size, output_size):
        return 1.0 / math.sqrt(float(input_size))


class XavierNormal(Normal):
    """src/module/init/xavier.rs:9-15: sigma = sqrt(2 / (input_size + output_size))."""

    def __init__(self, seed=None):
        super().__init__(0.0, 1.0, seed)

    def _sigma(self, input_size, output_size):
        return math.sqrt(2.0 / (float(input_size) + float(output_size)))


class FromArrays(InitParameters):
    """Injects given host arrays: the seam the reference's own tests use (a custom
    ``InitParameters`` passed to ``Linear::new_with_kernel``, src/module/linear.rs:86-95)."""

    def __init__(self, weight, bias=None):
        self._weight, self._bias = weight, bias

    def weight(self, input_size, output_size, engine):
        return engine.from_numpy(self._weight)

    def bias(self, input_size, output_size, engine):
        if self._bias is None:
            return engine.zeros(1, output_size)
        return engine.from_numpy(self._bias)
