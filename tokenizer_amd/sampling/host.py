"""Greedy and temperature / nucleus sampling on the host, with the reference's rules.

`greedy_token` and `sample_token` follow qwen-infer/src/sample.rs:43-137 step by step in
float32; the work is done in C++ (`csrc/host/sampler.cpp`), bound here.  The random numbers
come from `Rng`, a counter-based generator seeded per request: draw k of seed s is a function
of (s, k) alone, so a sequence's draws do not depend on what else is in the batch.  Its stream
is this framework's own (the reference's StdRng stream is not reproduced).
"""
from __future__ import annotations

import ctypes
import math

import numpy as np

from .. import host as _host


class SampleError(ValueError):
    pass


_M64 = (1 << 64) - 1
_f32p = ctypes.POINTER(ctypes.c_float)


def _logits(logits) -> np.ndarray:
    values = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
    if values.size == 0:
        raise SampleError("no logits to sample")
    return values


class Rng:
    """Counter-based uniform generator; one per sequence, created from the request's seed."""

    def __init__(self, seed: int):
        self.seed = int(seed) & _M64
        self.counter = 0

    def random_f32(self) -> float:
        """Uniform in [0, 1) with 24 bits, as a float32 value."""
        value = _host.lib().ta_uniform_f32(self.seed, self.counter)
        self.counter += 1
        return float(value)


def check_params(temperature: float, top_p: float) -> None:
    """sample.rs:77-88."""
    if not math.isfinite(temperature):
        raise SampleError(f"temperature {temperature} is not finite")
    if temperature < 0:
        raise SampleError(f"temperature {temperature} is negative")
    if not math.isfinite(top_p):
        raise SampleError(f"top_p {top_p} is not finite")
    if top_p < 0:
        raise SampleError(f"top_p {top_p} is negative")


def greedy_token(logits) -> int:
    """Lowest index among the maxima; NaN never wins (a scan with `>` from -inf, sample.rs:43-56)."""
    values = _logits(logits)
    return int(_host.lib().ta_greedy_token(values.ctypes.data_as(_f32p), values.size))


def sample_with_uniform(logits, temperature: float, top_p: float, uniform: float) -> int:
    """The draw of sample.rs:89-136 for a given uniform number in [0, 1): weights exp((x - max) / T) in
    float32, falling logit with the lower index first among equals, the nucleus cut where the running share
    reaches top_p, then the first token whose mass exceeds what is left of uniform * kept mass.  Sums that are
    zero or not finite fall back to the greedy pick."""
    values = _logits(logits)
    check_params(temperature, top_p)
    return int(_host.lib().ta_sample_with_uniform(values.ctypes.data_as(_f32p), values.size, temperature, top_p,
                                                  uniform))


def sample_token(logits, temperature: float, top_p: float, rng: Rng) -> int:
    """Draw one token (sample.rs:68-137).  Temperature 0 is greedy and draws nothing from `rng`."""
    values = _logits(logits)
    check_params(temperature, top_p)
    if temperature == 0:
        return greedy_token(values)
    return sample_with_uniform(values, temperature, top_p, rng.random_f32())
