"""Position encodings and the token table.

A position encoding acts in one of two places: it gives a table that the embedding stage adds
to the token rows (`table()`), or it turns queries and keys inside a mixer (`rotates = True` and
`rotate(q, k, ctx)`, which changes q [T, heads * dh] and k [T, kv heads * dh] in place, rows
ctx.positions; a mixer that keeps keys then writes the turned keys to its cache).  One that does
not act in a place returns None there / has `rotates = False`.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import POSITIONS, Part


class TokenEmbedding(Part):
    """The token table [vocab, width]; also the head's weight when the head is tied."""
    graph_safe = True

    def __init__(self, vocab: int, width: int, name: str):
        self.vocab, self.width, self.name = vocab, width, name

    def param_specs(self):
        return [ParamSpec(self.name, (self.vocab, self.width), "table", ("normal", 0.0, 0.02))]

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.name]


@POSITIONS.register("learned_absolute")
class LearnedAbsolutePositions(Part):
    """x[i] += wpe[position_i]                    (crates/denno-engine/src/model/gpt2.rs:142-150)"""
    graph_safe = True
    rotates = False

    def __init__(self, n_positions: int, width: int, name: str):
        self.n_positions, self.width, self.name = n_positions, width, name

    def param_specs(self):
        return [ParamSpec(self.name, (self.n_positions, self.width), "table", ("normal", 0.0, 0.02))]

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.name]

    def table(self):
        return self.weight

    def rotate(self, q, k, ctx):
        return q, k


@POSITIONS.register("none")
class NoPositions(Part):
    graph_safe = True
    rotates = False

    def __init__(self):
        pass

    def table(self):
        return None

    def rotate(self, q, k, ctx):
        return q, k


@POSITIONS.register("rotary_pairs")
class RotaryPairs(Part):
    """Of a vector's first `dims` entries, entry 2i and entry 2i + 1 form a pair (u, v) that the position p turns by
    the angle p * f_i, f_i = base^(-2i / dims): (u cos - v sin, v cos + u sin).  The rest of the vector passes.  Angles are
    32-bit; the frequencies are made once, in 64-bit, and rounded.  head_dim: the width of the vectors that `rotate`
    finds side by side in q and k; a mixer whose turned parts lie elsewhere calls `turn` with its own layout.

    scaling = dict(factor, original, fast, slow) stretches the encoding beyond the length it was trained for: with
    d(t) = dims * ln(original / (2 pi t)) / (2 ln base), the pair index whose pair makes t turns over `original` positions,
    lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    pair i turns by p * (f_i / factor * ramp_i + f_i * (1 - ramp_i)): fast pairs stay, slow ones are slowed down by `factor`;
    and cos and sin are multiplied by `mag` = 0.1 ln(factor) + 1."""
    graph_safe = True
    rotates = True
    libraries = ("sequence",)

    def __init__(self, dims: int, base: float, head_dim: int = 0, scaling=None):
        if dims % 2 != 0 or dims < 0:
            raise ValueError(f"rotary_pairs: {dims} dimensions cannot be paired")
        self.dims, self.base, self.head_dim = int(dims), float(base), int(head_dim or dims)
        if self.dims > self.head_dim:
            raise ValueError(f"rotary_pairs: {dims} dimensions in vectors of {self.head_dim}")
        self.scaling = dict(scaling) if scaling else None
        self.mag = 1.0
        if self.scaling:
            missing = [k for k in ("factor", "original", "fast", "slow") if k not in self.scaling]
            if missing or not self.scaling["factor"] > 0 or not self.scaling["original"] > 0 or self.base <= 1:
                raise ValueError(f"rotary_pairs: scaling needs factor, original, fast and slow (and a base above 1); got {self.scaling}")
            self.mag = 0.1 * math.log(float(self.scaling["factor"])) + 1.0

    def frequencies(self):
        """The pairs' frequencies, 64-bit, on the CPU."""
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        f = torch.tensor(self.base, dtype=torch.float64) ** (-2.0 * i / max(self.dims, 1))
        if not self.scaling or self.dims == 0:
            return f
        sc = self.scaling
        factor, original = float(sc["factor"]), float(sc["original"])

        def pair_of(turns):
            return self.dims * math.log(original / (2.0 * math.pi * float(turns))) / (2.0 * math.log(self.base))
        lo = max(math.floor(pair_of(sc["fast"])), 0)
        hi = min(math.ceil(pair_of(sc["slow"])), self.dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / factor * ramp + f * (1.0 - ramp)

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.freq = self.frequencies().to(torch.float32).to(runtime.device)

    def table(self):
        return None

    def turn(self, src, dst, positions, n_vec, width, **layout):
        return ops.rotary(src, dst, positions, self.freq, n_vec, self.dims, width, mag=self.mag, **layout)

    def rotate(self, q, k, ctx):
        for t in (q, k):
            self.turn(t, t, ctx.positions, t.shape[1] // self.head_dim, self.head_dim)
        return q, k
