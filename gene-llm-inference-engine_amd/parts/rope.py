"""Rotary position encoding with half-split pairs.

Frequencies are computed once, in 64-bit on the host, as the reference computes them
(src/kernels/kernels.cpp:142-147): f_k = theta^(-2k/head_dim), unless the spec brings the
frequencies an architecture's own rule has made of them.  Per step, cos and sin of pos*f_k are
made on the device from 64-bit angles for the step's rows and shared by every layer with the
same spec."""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import PositionEncoding, register_position_encoding

def inverse_frequencies(head_dim: int, theta: float):
    return [1.0 / math.pow(float(theta), 2.0 * k / head_dim) for k in range(head_dim // 2)]


class RotaryHalfSplit(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        if spec.head_dim % 2:
            raise ValueError("rotary encoding needs an even head size")
        self.half = spec.head_dim // 2
        frequencies = spec.frequencies if spec.frequencies is not None else inverse_frequencies(spec.head_dim, spec.theta)
        self.inv_freq = torch.tensor(list(frequencies), dtype=torch.float64, device=device)
        self.magnitude = float(getattr(spec, "magnitude", 1.0))

    def half_split_tables(self, ctx):
        """(cos, sin), float32 [T, head_dim/2], for the rows of this step."""
        key = ("rotary", self.spec)
        if key not in ctx.memo:
            cos = torch.empty((ctx.n_rows, self.half), dtype=torch.float32, device=ctx.device)
            sin = torch.empty_like(cos)
            ops.rope_cos_sin(ctx.row_pos, self.inv_freq, cos, sin, self.magnitude)
            ctx.memo[key] = (cos, sin)
        return ctx.memo[key]


class RotaryPartial(PositionEncoding):
    """The same rotation on the first `rotary_dim` channels of a head only: pairs (i, i + rotary_dim/2); the rest of the head
    passes.  It has no tables for whole heads; a mixer whose kernels turn a part of a head asks `partial_tables`."""
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.rotary_dim = spec.rotary_dim
        frequencies = spec.frequencies if spec.frequencies is not None else inverse_frequencies(spec.rotary_dim, spec.theta)
        self.inv_freq = torch.tensor(list(frequencies), dtype=torch.float64, device=device)
        self.magnitude = float(getattr(spec, "magnitude", 1.0))

    def partial_tables(self, ctx):
        """(cos, sin, rotary_dim): float32 [T, rotary_dim/2] each, for the rows of this step."""
        key = ("rotary_partial", self.spec)
        if key not in ctx.memo:
            cos = torch.empty((ctx.n_rows, self.rotary_dim // 2), dtype=torch.float32, device=ctx.device)
            sin = torch.empty_like(cos)
            ops.rope_cos_sin(ctx.row_pos, self.inv_freq, cos, sin, self.magnitude)
            ctx.memo[key] = (cos, sin)
        return (*ctx.memo[key], self.rotary_dim)


class RotaryInterleaved(PositionEncoding):
    """Angles for a rotation of neighbouring pairs (2i, 2i + 1).  It has no tables for half-split pairs and no kernel of its
    own: a mixer whose kernels turn such pairs asks `pair_tables`."""
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.rotary_dim = spec.rotary_dim
        frequencies = spec.frequencies if spec.frequencies is not None else inverse_frequencies(spec.rotary_dim, spec.theta)
        self.inv_freq = torch.tensor(list(frequencies), dtype=torch.float64, device=device)
        self.magnitude = float(getattr(spec, "magnitude", 1.0))

    def pair_tables(self, ctx):
        """(cos, sin): float32 [T, rotary_dim/2] each, for the rows of this step; pair i is turned by angle i."""
        key = ("rotary_interleaved", self.spec)
        if key not in ctx.memo:
            cos = torch.empty((ctx.n_rows, self.rotary_dim // 2), dtype=torch.float32, device=ctx.device)
            sin = torch.empty_like(cos)
            ops.rope_cos_sin(ctx.row_pos, self.inv_freq, cos, sin, self.magnitude)
            ctx.memo[key] = (cos, sin)
        return ctx.memo[key]


def rotation_tables(position, ctx):
    """(cos, sin, channels turned) of an encoding that turns the pairs (i, i + r/2) of a head's first r channels (the whole head
    or a part), or None if `position` is no such encoding."""
    if position is None:
        return None
    if hasattr(position, "partial_tables"):
        return position.partial_tables(ctx)
    tables = position.half_split_tables(ctx)
    return None if tables is None else (*tables, 2 * tables[0].shape[1])


register_position_encoding("rotary_half_split", RotaryHalfSplit)
register_position_encoding("rotary_partial", RotaryPartial)
register_position_encoding("rotary_interleaved", RotaryInterleaved)
