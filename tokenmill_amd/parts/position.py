"""Position encodings applied to q and k before they are cached.

RotaryEmbedding: reference src/infer/model/layers.py:47-64. The cos/sin table is built once on
the host in 32-bit with the reference's expression and uploaded; the rotation runs in 32-bit in
the kernel that also stores k and v into the cache.
"""
from __future__ import annotations

import math

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import KVCacheView, PositionEncoding, StepContext


class RotaryEmbedding(PositionEncoding):
    """Pairs (j, j + rotary_dim/2) of each head rotate by position * theta^(-2j/rotary_dim). ``interleaved``: the pairs
    are the neighbours (2j, 2j + 1) instead; the table of angles is the same, and a mixer that wants that pairing rotates
    with kernels of its own (the kernel library's attention operation knows the first pairing only)."""

    def __init__(self, head_dim: int, theta: float, max_positions: int, rotary_dim: int | None = None,
                 interleaved: bool = False, scaling: dict | None = None, exact: bool = False):
        """``scaling`` (factor, original, fast, slow): the frequencies of pairs that turn fewer than ``slow`` times over
        ``original`` positions are divided by ``factor``, those that turn more than ``fast`` times stay, and the pairs between
        are blended linearly over the pair index; cos and sin are multiplied by 0.1 ln(factor) + 1. With j(t) =
        rotary_dim * ln(original / (2 pi t)) / (2 ln theta): lo = max(floor(j(fast)), 0), hi = min(ceil(j(slow)),
        rotary_dim - 1), ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i).
        A ``scaling`` that holds a ``factor`` alone is linear: every frequency is divided by the factor, cos and sin stay as
        they are. ``exact``: the frequencies are computed in 64-bit and rounded once to 32-bit (always so with ``scaling``)."""
        self.head_dim = head_dim
        self.interleaved = interleaved
        self.scaling = dict(scaling) if scaling else None
        self.exact = exact or self.scaling is not None
        self.linear = self.scaling is not None and set(self.scaling) == {"factor"}
        if self.scaling is not None:
            for key in ("factor",) if self.linear else ("factor", "original", "fast", "slow"):
                if key not in self.scaling:
                    raise ValueError(f"rotary scaling has no '{key}'")
            if not float(self.scaling["factor"]) > 0:
                raise ValueError("the rotary scaling factor must be positive")
        self.rotary_dim = rotary_dim or head_dim
        if self.rotary_dim % 2 or self.rotary_dim > head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {head_dim}")
        self.theta = float(theta)
        self.max_positions = max_positions
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def frequencies(self) -> tuple[torch.Tensor, float]:
        """(float32 [rotary_dim / 2] angle per position of every pair, what cos and sin are multiplied by)."""
        d = self.rotary_dim
        if not self.exact:
            return 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d)), 1.0
        i = torch.arange(d // 2, dtype=torch.float64)
        f = self.theta ** (-2.0 * i / d)
        sc = self.scaling
        if sc is None:
            return f.float(), 1.0
        if self.linear:
            return (f / float(sc["factor"])).float(), 1.0
        factor, original = float(sc["factor"]), float(sc["original"])

        def pair_of(turns: float) -> float:
            return d * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

        lo = max(math.floor(pair_of(float(sc["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(sc["slow"]))), d - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        return f.float(), 0.1 * math.log(factor) + 1.0

    def build_tables(self, device) -> None:
        inv_freq, magnitude = self.frequencies()
        freqs = torch.outer(torch.arange(self.max_positions).float(), inv_freq)     # [max_pos, d/2], 32-bit angles
        cos, sin = freqs.cos(), freqs.sin()
        if magnitude != 1.0:
            cos, sin = cos * magnitude, sin * magnitude
        self.cos = cos.contiguous().to(device)
        self.sin = sin.contiguous().to(device)

    def load(self, tensors, prefix: str) -> None:
        device = next(iter(tensors.values())).device
        if self.cos is None or self.cos.device != device:
            self.build_tables(device)

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step: StepContext, cache: KVCacheView | None):
        if self.interleaved:
            raise NotImplementedError("neighbouring pairs are rotated by the mixer that asked for them")
        if step.max_context_len > self.max_positions:
            raise ValueError(f"position {step.max_context_len - 1} is beyond the rotary table "
                             f"({self.max_positions} positions)")
        write = cache is not None and cache.write
        ops.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, self.cos, self.sin, step.positions,
                          step.groups[cache.group].slot_mapping if write else None,
                          cache.k if write else None, cache.v if write else None)

    def rotation(self):
        """(cos, sin, rotary width, positions): what the kernel library's attention operation rotates by."""
        if self.interleaved:
            return None
        return (self.cos, self.sin, self.rotary_dim, self.max_positions) if self.cos is not None else None


class NoPositionEncoding(PositionEncoding):
    """Stores k and v; q and k stay as they are."""

    def rotation(self):
        return ()

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step: StepContext, cache: KVCacheView | None):
        if cache is not None and cache.write:
            ops.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, None, None, None,
                              step.groups[cache.group].slot_mapping, cache.k, cache.v)
