"""Rotary position encoding with optional llama3 frequency scaling
(tinyserve_llm/model/llama.py:107-128,139-161).

The table [max_position, head_dim] = [cos | sin] is computed once, on the CPU, in 32-bit, with the
operations and operand order of the reference, and uploaded; mixers rotate with it inside their
own kernels (pairing i with i + head_dim/2, llama.py:131-136).
"""

from __future__ import annotations

import math

import torch

from tinyserve_llm_amd.parts.base import PositionEncoding, register


def inverse_frequencies(head_dim: int, theta: float, scaling: dict | None, max_position: int) -> torch.Tensor:
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    if scaling is None:
        return inv_freq
    factor, lo, hi = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
    old_len = scaling.get("original_max_position_embeddings", max_position)
    wavelen = 2 * math.pi / inv_freq
    slowed = torch.where(wavelen > old_len / lo, inv_freq / factor, inv_freq)
    smooth = (old_len / wavelen - lo) / (hi - lo)
    blended = (1 - smooth) * slowed / factor + smooth * slowed
    medium = ~(wavelen < old_len / hi) * ~(wavelen > old_len / lo)
    return torch.where(medium, blended, slowed)


@register("position_encoding", "rope")
class Rope(PositionEncoding):
    graph_safe = True

    def __init__(self, head_dim: int, max_position: int, theta: float, scaling: dict | None = None,
                 rotary_dim: int | None = None) -> None:
        """`rotary_dim` (even, up to head_dim; default: all of it): the leading dimensions of a head
        that turn, dimension j with j + rotary_dim / 2; the table is that wide and the rest of a head
        passes unchanged (the Llama models turn whole heads)."""
        rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if rotary_dim % 2 or not 2 <= rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim}: an even number from 2 to head_dim {head_dim}")
        self.head_dim = head_dim
        self.rotary_dim = rotary_dim
        self.max_position = max_position
        self.theta = theta
        self.scaling = scaling
        self.inv_freq = inverse_frequencies(rotary_dim, theta, scaling, max_position)
        self.cos_sin: torch.Tensor | None = None

    def host_table(self) -> torch.Tensor:
        t = torch.arange(self.max_position, dtype=torch.float)
        freqs = torch.einsum("i,j -> ij", t, self.inv_freq)
        return torch.cat((freqs.cos(), freqs.sin()), dim=-1).contiguous()

    def prepare(self, device: torch.device) -> None:
        self.cos_sin = self.host_table().to(device)

    def rotary_table(self) -> torch.Tensor | None:
        return self.cos_sin


@register("position_encoding", "rotary_frequencies")
class RotaryFrequencies(PositionEncoding):
    """Rotary positions without a table over positions, for models that set no limit to a request's
    length: only the frequencies f_i = theta^(-2i / rotary_dim), i < rotary_dim / 2, are kept (64-bit),
    and a mixer's kernel takes the angle position * f_i itself. `interleaved`: pair i is dimensions
    (2i, 2i+1) of a head; otherwise (i, i + rotary_dim/2). The first `rotary_dim` dimensions of a head
    turn, the rest pass."""

    graph_safe = True

    def __init__(self, rotary_dim: int, theta: float, interleaved: bool = True, ramp: dict | None = None) -> None:
        """`ramp` (factor s, original length L, fast, slow): frequencies are slowed down by s along a ramp over
        the pairs: with d(t) = rotary_dim ln(L / (2 pi t)) / (2 ln theta), lo = max(floor d(fast), 0),
        hi = min(ceil d(slow), rotary_dim - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i
        turns with f_i / s * r_i + f_i (1 - r_i), and cosine and sine are multiplied by `amplitude` =
        0.1 ln s + 1 (the mixers' kernels take it beside the frequencies)."""
        if rotary_dim % 2 or rotary_dim < 0:
            raise ValueError(f"rotary_dim {rotary_dim}: an even number of dimensions turns")
        self.rotary_dim, self.theta, self.interleaved = rotary_dim, float(theta), interleaved
        self.ramp = dict(ramp) if ramp else None
        if self.ramp is not None and not (self.ramp["factor"] > 0 and self.ramp["original"] > 0 and self.ramp["fast"] > 0
                                          and self.ramp["slow"] > 0 and self.theta > 1):
            raise ValueError("a frequency ramp needs positive factor, original, fast and slow, and a base above 1")
        self.amplitude = 0.1 * math.log(self.ramp["factor"]) + 1.0 if self.ramp is not None else 1.0
        self.freqs: torch.Tensor | None = None

    def host_frequencies(self) -> torch.Tensor:
        i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * i / max(1, self.rotary_dim))
        if self.ramp is None:
            return f
        r = self.ramp

        def crossing(turns: float) -> float:
            return self.rotary_dim * math.log(r["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

        lo, hi = max(math.floor(crossing(r["fast"])), 0), min(math.ceil(crossing(r["slow"])), self.rotary_dim - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / r["factor"] * ramp + f * (1.0 - ramp)

    def prepare(self, device: torch.device) -> None:
        self.freqs = self.host_frequencies().to(device) if self.rotary_dim else None

    def frequencies(self) -> torch.Tensor | None:
        return self.freqs
