"""Rotate-half rotary position encoding.

Table as the reference's table variant builds it (engine/nn/rope.py:28-29,105-109):
inv_freq[i] = 1/theta^(2i/dim) in float32, angle = float32(pos) * inv_freq, then
cos and sin; the pairing (x[i], x[i+dim/2]) is engine/kernels/triton/rope.py:53-65.
The table is computed on the host so every device run reads identical values.
"""

from __future__ import annotations

import math

import torch

from tokensprint_amd.parts.base import POSITIONS, PositionEncoding, register


@register(POSITIONS, "rope")
class RotaryEncoding(PositionEncoding):
    """params: dim (rotated head size), theta, max_position."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.dim = int(params["dim"])
        self.theta = float(params["theta"])
        self.max_position = int(params["max_position"])
        if self.dim % 2:
            raise ValueError(f"rotary dim must be even, got {self.dim}")
        idx = torch.arange(0, self.dim, 2, dtype=torch.float32)
        inv_freq = 1.0 / (self.theta ** (idx / self.dim))
        angles = torch.outer(torch.arange(self.max_position, dtype=torch.float32), inv_freq)
        self.cos = angles.cos().contiguous().to(ctx.device)
        self.sin = angles.sin().contiguous().to(ctx.device)

    def rotary_tables(self):
        return self.cos, self.sin

    def step_read_tensors(self):
        return []          # a step reads the rows of its positions, not the tables

    def apply(self, q, k, positions):
        self.ops.rope_inplace(q, positions, self.cos, self.sin)
        if k is not None:
            self.ops.rope_inplace(k, positions, self.cos, self.sin)


@register(POSITIONS, "rope_interleaved")
class InterleavedRotation(PositionEncoding):
    """Rotation of the pairs (2i, 2i+1) of a vector's first `dims` dimensions by the angle
    position * base^(-2i/dims); the rest passes unchanged.  The pair (u, v) becomes
    (u cos a - v sin a, v cos a + u sin a).  There is no table and so no longest position:
    kernels take `frequencies()` (float32 [dims/2], rounded once from float64) and compute
    the angle and its cosine and sine in float32 at the position they need.

    params: dims, base."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.dims = int(params["dims"])
        self.base = float(params["base"])
        if self.dims % 2 or self.dims < 2:
            raise ValueError(f"rotated dimensions must be even and at least 2, got {self.dims}")
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        self.freqs = (self.base ** (-2.0 * i / self.dims)).to(torch.float32).to(ctx.device)

    def frequencies(self):
        return self.freqs

    def step_read_tensors(self):
        return []

    def apply(self, q, k, positions):
        self.ops.rotate_interleaved_inplace(q, positions, self.freqs, self.dims, offset=0)
        if k is not None:
            self.ops.rotate_interleaved_inplace(k, positions, self.freqs, self.dims, offset=0)


@register(POSITIONS, "rope_partial")
class PartialRotaryEncoding(PositionEncoding):
    """Rotate-half rotation of the first `dims` dimensions of a head of `head_dim`
    dimensions: dimension i pairs with i + dims/2, angle position * base^(-2i/dims); the rest
    passes unchanged.  The kernels rotate whole heads, pairing j with j + head_dim/2, so a
    mixer that uses this lays its heads out by `layout()` (rotated first halves, the rest,
    rotated second halves, the rest: a permutation of a head's dimensions, the same for
    queries and keys, which changes no score) and the table holds cos = 1, sin = 0 for the
    pairs that are not rotated.  Frequencies are rounded once from float64; angles and their
    cosines and sines are float32, computed on the host.

    `scaling` = {factor, original, fast, slow} stretches the slow frequencies for contexts
    beyond the `original` length (YaRN): with d(t) = dims ln(original / (2 pi t)) / (2 ln
    base), lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1) and ramp_i =
    clamp((i - lo) / max(hi - lo, 0.001), 0, 1), frequency i becomes f_i / factor * ramp_i +
    f_i (1 - ramp_i), and cos and sin are multiplied by 0.1 ln(factor) + 1.

    params: dims, base, head_dim, max_position, scaling (None: plain frequencies)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.dims, self.base = int(params["dims"]), float(params["base"])
        self.head_dim, self.max_position = int(params["head_dim"]), int(params["max_position"])
        if self.dims % 2 or self.head_dim % 2 or not 2 <= self.dims <= self.head_dim:
            raise ValueError(f"rotated dimensions ({self.dims}) must be even and fit the head "
                             f"({self.head_dim}, even)")
        half, r = self.head_dim // 2, self.dims // 2
        i = torch.arange(r, dtype=torch.float64)
        freqs, magnitude = self.base ** (-2.0 * i / self.dims), 1.0
        scaling = params.get("scaling")
        if scaling:
            freqs, magnitude = self.stretched(freqs, i, scaling)
        freqs = freqs.to(torch.float32)
        angles = torch.outer(torch.arange(self.max_position, dtype=torch.float32), freqs)
        cos = torch.ones(self.max_position, half, dtype=torch.float32)
        sin = torch.zeros(self.max_position, half, dtype=torch.float32)
        cos[:, :r], sin[:, :r] = angles.cos() * magnitude, angles.sin() * magnitude
        self.cos, self.sin = cos.contiguous().to(ctx.device), sin.contiguous().to(ctx.device)

    def stretched(self, freqs, i, scaling):
        """(frequencies, factor on cos and sin) under `scaling`; float64."""
        factor, original = float(scaling["factor"]), float(scaling["original"])
        if not factor > 0 or not original > 0 or self.base <= 1.0:
            raise ValueError(f"rotation scaling needs factor > 0, original > 0 and base > 1, "
                             f"got {dict(scaling)} with base {self.base}")

        def turn_dim(turns):
            return self.dims * math.log(original / (2.0 * math.pi * turns)) \
                / (2.0 * math.log(self.base))

        lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(scaling["slow"]))), self.dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return freqs / factor * ramp + freqs * (1.0 - ramp), 0.1 * math.log(factor) + 1.0

    def layout(self, dim: int) -> list[int]:
        """For a head of `dim` given dimensions (dim <= head_dim): the given dimension that
        stands at each of the `head_dim` places, -1 where a zero stands."""
        half, r = self.head_dim // 2, self.dims // 2
        rest = list(range(self.dims, dim))
        first = list(range(r)) + rest[:half - r]
        second = list(range(r, self.dims)) + rest[half - r:]
        if len(second) > half:
            raise ValueError(f"a head of {dim} dimensions does not fit {self.head_dim}")
        return first + [-1] * (half - len(first)) + second + [-1] * (half - len(second))

    def rotary_tables(self):
        return self.cos, self.sin

    def step_read_tensors(self):
        return []

    def apply(self, q, k, positions):
        self.ops.rope_inplace(q, positions, self.cos, self.sin)
        if k is not None:
            self.ops.rope_inplace(k, positions, self.cos, self.sin)
