"""Rotary position encoding: a float32 table of cosines and sines.

angle[p, i] = float(p) * (1 / theta^(2i / d)) with the frequency and the product
in float32, as the reference builds its table
(runtime/include/models/qwen3_model.hpp:410-436).  Its power is the C library's single
precision `pow`, which works in double precision inside and rounds the result once; the
same is done here (a float32 `pow` of another library may differ in the last bit, which
moves the angle of position 4,000 by 2e-4).  Cosine and sine are evaluated in float64 from
the float32 angle and rounded once.  Row p holds cos for the d/2 pairs, then sin; pairs are
(i, i + d/2).
"""
from __future__ import annotations

import math

import torch


class RotaryTable:
    def __init__(self, spec, device):
        if spec.dim % 2:
            raise ValueError("rotary dimension must be even")
        self.spec = spec
        half = spec.dim // 2
        exponent = (2.0 * torch.arange(half, dtype=torch.float32)) / float(spec.dim)
        theta = torch.tensor(float(spec.theta), dtype=torch.float32).to(torch.float64)
        frequency = 1.0 / torch.pow(theta, exponent.to(torch.float64)).to(torch.float32)
        position = torch.arange(spec.max_positions, dtype=torch.float32)
        angle = (position[:, None] * frequency[None, :]).to(torch.float64)
        table = torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).to(torch.float32)
        self.table = table.to(device).contiguous()

    @property
    def max_positions(self):
        return self.table.shape[0]


class NoPosition:
    """Mixers that take no position encoding get a table of None."""
    def __init__(self, spec, device):
        self.spec = spec
        self.table = None
        self.max_positions = None


class RotaryFrequencies:
    """Rotation of neighbouring pairs (2i, 2i + 1) by the angle position * theta^(-2i / dim):
    the kernels multiply the float32 position by the float32 frequency and take cosine and
    sine themselves, so there is no table and no position that is too far.  The frequencies
    are float64 powers rounded once."""
    def __init__(self, spec, device):
        if spec.dim % 2 or spec.dim < 2:
            raise ValueError("rotary dimension must be even and at least 2")
        self.spec = spec
        exponent = -2.0 * torch.arange(spec.dim // 2, dtype=torch.float64) / float(spec.dim)
        frequencies = torch.pow(torch.tensor(float(spec.theta), dtype=torch.float64), exponent)
        self.frequencies = frequencies.to(torch.float32).to(device).contiguous()
        self.table = None
        self.max_positions = None


def scaled_frequencies(spec) -> torch.Tensor:
    """theta^(-2i / dim) for i < dim / 2 in float64, with the long wavelengths stretched as
    `spec.scaling` says (see `config.specs.FrequencyScaling`)."""
    exponent = -2.0 * torch.arange(spec.dim // 2, dtype=torch.float64) / float(spec.dim)
    frequencies = torch.pow(torch.tensor(float(spec.theta), dtype=torch.float64), exponent)
    scaling = getattr(spec, "scaling", None)
    if scaling is None:
        return frequencies
    wavelength = 2.0 * math.pi / frequencies
    blend = (scaling.original / wavelength - scaling.low) / (scaling.high - scaling.low)
    between = (1.0 - blend) * frequencies / scaling.factor + blend * frequencies
    return torch.where(wavelength < scaling.original / scaling.high, frequencies,
                       torch.where(wavelength > scaling.original / scaling.low,
                                   frequencies / scaling.factor, between))


class RotaryHalfFrequencies:
    """Rotation of the pairs (i, i + dim/2) of a head's first `dim` elements by the angle
    position * f_i: the store kernel multiplies the position by the float64 frequency, takes
    the product modulo 2 pi, rounds it to float32 and takes cosine and sine itself, so there is
    no table, no position that is too far, and the float32 angle is the nearest one however
    far the position.  The frequencies are worked out in float64 (stretched where the spec
    says)."""
    def __init__(self, spec, device):
        if spec.dim % 2 or spec.dim < 2:
            raise ValueError("rotary dimension must be even and at least 2")
        self.spec = spec
        self.frequencies = scaled_frequencies(spec).to(device).contiguous()
        self.table = None
        self.max_positions = None
