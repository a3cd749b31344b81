"""Greedy and temperature / nucleus sampling on the host, with the reference's rules.

`greedy_token` and `sample_token` follow qwen-infer/src/sample.rs:43-137 step by step in
float32.  The random numbers come from `Rng`, a counter-based generator seeded per request:
draw k of seed s is a function of (s, k) alone, so a sequence's draws do not depend on what
else is in the batch.  Its stream is this framework's own (the reference's StdRng stream is
not reproduced).
"""
from __future__ import annotations

import math

import numpy as np


class SampleError(ValueError):
    pass


_M64 = (1 << 64) - 1


def _mix(z: int) -> int:
    """splitmix64 finaliser."""
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


class Rng:
    """Counter-based uniform generator; one per sequence, created from the request's seed."""

    def __init__(self, seed: int):
        self.key = _mix(int(seed) & _M64)
        self.counter = 0

    def random_f32(self) -> float:
        """Uniform in [0, 1) with 24 bits, as a float32 value."""
        bits = _mix(self.key ^ _mix(self.counter))
        self.counter += 1
        return float(np.float32((bits >> 40) * (1.0 / (1 << 24))))


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
    values = np.asarray(logits, dtype=np.float32)
    if values.size == 0:
        raise SampleError("no logits to sample")
    finite = np.where(np.isnan(values), -np.inf, values)
    best = finite.max()
    if best == -np.inf:
        return 0
    return int(np.argmax(finite == best))


def sample_with_uniform(logits, temperature: float, top_p: float, uniform: float) -> int:
    """The draw of sample.rs:89-136 for a given uniform number in [0, 1)."""
    values = np.asarray(logits, dtype=np.float32)
    if values.size == 0:
        raise SampleError("no logits to sample")
    check_params(temperature, top_p)
    if temperature == 0:
        return greedy_token(values)
    f32 = np.float32
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        weight = np.exp((values - values.max()) / f32(temperature)).astype(np.float32)
    # Descending logit, lower index first among equals (sample.rs:100-101); NaN sorts as total_cmp does not
    # matter here because a NaN weight makes the sums non-finite and the draw falls back to greedy.
    order = np.lexsort((np.arange(values.size), -values.astype(np.float64)))
    ordered = weight[order]
    if top_p >= 1.0:
        cutoff = values.size
    else:
        total = _sequential_sum(weight)
        if total == 0 or not math.isfinite(total):
            return greedy_token(values)
        shares = (ordered / f32(total)).astype(np.float32)
        cumulative = np.cumsum(shares, dtype=np.float32)     # sequential float32 adds
        reached = np.nonzero(cumulative >= f32(top_p))[0]
        cutoff = int(reached[0]) + 1 if reached.size else values.size
    kept = ordered[:cutoff]
    kept_sum = _sequential_sum(kept)
    if kept_sum == 0 or not math.isfinite(kept_sum):
        return greedy_token(values)
    threshold = f32(f32(uniform) * f32(kept_sum))
    for position in range(cutoff):
        mass = kept[position]
        if threshold < mass:
            return int(order[position])
        threshold = f32(threshold - mass)
    return int(order[cutoff - 1])


def _sequential_sum(values: np.ndarray) -> float:
    return float(np.cumsum(values, dtype=np.float32)[-1]) if values.size else 0.0


def sample_token(logits, temperature: float, top_p: float, rng: Rng) -> int:
    """Draw one token (sample.rs:68-137).  Temperature 0 is greedy and draws nothing from `rng`."""
    values = np.asarray(logits, dtype=np.float32)
    if values.size == 0:
        raise SampleError("no logits to sample")
    check_params(temperature, top_p)
    if temperature == 0:
        return greedy_token(values)
    return sample_with_uniform(values, temperature, top_p, rng.random_f32())
