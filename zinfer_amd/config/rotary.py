"""Rules that give a rotary encoding its frequencies.

A rotation of ``dims`` elements has dims/2 pairs; pair i turns by position * f_i.  The plain
rule is f_i = base^(-2i/dims).  Two published ways of stretching a trained range of positions
change the f_i (and one of them the length of the rotated vector); both are functions from the
plain frequencies to new ones, so they are written here once and every mixer that rotates can
name either.  All of it is computed in 64-bit on the host, once at load; the kernels get the
frequencies as 32-bit numbers.
"""
from __future__ import annotations

import math
from typing import Tuple

from ..errors import ConfigError
from .specs import LeadingRotarySpec


def plain_frequencies(base: float, dims: int) -> Tuple[float, ...]:
    if dims < 2 or dims % 2 != 0:
        raise ConfigError(f"a rotation needs an even number of elements, got dims={dims}")
    if not base > 0.0:
        raise ConfigError(f"a rotation's base must be positive, got {base}")
    return tuple(base ** (-2.0 * i / dims) for i in range(dims // 2))


def by_wavelength(freqs: Tuple[float, ...], factor: float, low: float, high: float,
                  original: float) -> Tuple[float, ...]:
    """Pairs whose wavelength 2 pi / f is shorter than original / high keep their frequency,
    those longer than original / low turn ``factor`` times slower, and between the two the
    frequency goes in a straight line (in original / wavelength) from the one to the other."""
    out = []
    for f in freqs:
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            out.append(f)
        elif wavelength > original / low:
            out.append(f / factor)
        elif high == low:              # no range between the two: the one wavelength on the edge
            out.append(f)
        else:
            t = (original / wavelength - low) / (high - low)
            out.append((1.0 - t) * f / factor + t * f)
    return tuple(out)


def by_turns(freqs: Tuple[float, ...], base: float, dims: int, factor: float, original: float,
             fast: float, slow: float) -> Tuple[Tuple[float, ...], float]:
    """(frequencies, magnitude).  A pair that makes more than ``fast`` turns over ``original``
    positions keeps its frequency, one that makes fewer than ``slow`` turns is slowed by
    ``factor``, with a ramp over the pair's index between: the index at which a pair makes t
    turns is dims * ln(original / (2 pi t)) / (2 ln base).  Cosine and sine grow by
    0.1 ln(factor) + 1."""
    def index_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    first = max(math.floor(index_of(fast)), 0)
    last = min(math.ceil(index_of(slow)), dims - 1)
    span = max(last - first, 0.001)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - first) / span, 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return tuple(out), 0.1 * math.log(factor) + 1.0


def leading_rotary(base: float, dims: int, scaling: dict = None) -> LeadingRotarySpec:
    """The specification for ``dims`` leading elements with the rule that ``scaling``'s keys
    name: none, {factor, low, high, original} or {factor, original, fast, slow}."""
    freqs = plain_frequencies(float(base), int(dims))
    if not scaling:
        return LeadingRotarySpec(int(dims), freqs)
    keys = set(scaling)
    try:
        if {"factor", "low", "high", "original"} <= keys:
            return LeadingRotarySpec(int(dims), by_wavelength(
                freqs, float(scaling["factor"]), float(scaling["low"]), float(scaling["high"]),
                float(scaling["original"])))
        if {"factor", "original", "fast", "slow"} <= keys:
            f, mag = by_turns(freqs, float(base), int(dims), float(scaling["factor"]),
                              float(scaling["original"]), float(scaling["fast"]),
                              float(scaling["slow"]))
            return LeadingRotarySpec(int(dims), f, mag)
    except (TypeError, ValueError, ZeroDivisionError) as e:
        raise ConfigError(f"rotary scaling {scaling!r}: {e}") from None
    raise ConfigError(f"rotary scaling with keys {sorted(keys)}: known are factor/low/high/"
                      "original and factor/original/fast/slow")
