"""Norms. RMSNorm with the residual add folded in (tinyserve_llm/model/llama.py:39-74).

`norm(x, residual)` returns (normalise(x + residual) * weight, x + residual): the sum, its mean
square, the rsqrt and the scaling are 32-bit; the returned residual is the sum rounded to the
storage type, while the normalisation uses the unrounded sum (llama.py:63-67).
"""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import Norm, ParamSpec, register
from tinyserve_llm_amd.parts.linear import DeferredNorm, NormRequest
from tinyserve_llm_amd.parts.stream import ResidualStream


@register("norm", "rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, hidden_size: int, eps: float, one_plus: bool = False) -> None:
        """`one_plus`: the weight is stored around zero and the rows are multiplied by 1 + weight (the sum taken
        in 32-bit, once, when the weights arrive); such a norm works on a 32-bit residual stream."""
        self.hidden_size = hidden_size
        self.eps = eps
        self.one_plus = one_plus
        self.weight: torch.Tensor | None = None
        self.applied: torch.Tensor | None = None      # what the rows are multiplied by: the weight, or 1 + weight in 32-bit

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.hidden_size,), init=(0.0, 0.1) if self.one_plus else (1.0, 0.1))}

    def bind(self, params) -> None:
        super().bind(params)
        self.applied = (1.0 + self.weight.float()).contiguous() if self.one_plus else self.weight
        self.weight32 = self.applied if self.applied.dtype == torch.float32 else self.applied.float().contiguous()

    def __call__(self, x, residual=None, rows=None):
        if isinstance(x, ResidualStream):
            # a 32-bit stream: its pending sum, then the norm, rounded to the weights' storage type on the way out
            if residual is not None:
                raise ValueError("a residual stream carries its own sum")
            return x.norm_rows(rows, self.applied, self.eps, self.weight.dtype), (None if rows is not None else x.x)
        if self.one_plus:
            raise TypeError("a norm with 1 + weight works on a 32-bit residual stream (ModelSpec.residual_dtype = 'float32')")
        return hip.rmsnorm(x, self.weight, self.eps, residual, rows)

    def defer(self, x, residual=None) -> DeferredNorm:
        """The same norm as an operand that the next projection may fuse."""
        return DeferredNorm(x, residual, self.weight, self.eps)

    def request(self, residual=None) -> NormRequest:
        """The same norm as a request to the projection before it (`linear(..., then=)`)."""
        return NormRequest(self.weight, self.eps, residual)

    def made_for(self, pending) -> bool:
        """Whether `pending` is this norm, deferred (by `defer` or through `request`)."""
        return isinstance(pending, DeferredNorm) and pending.weight is self.weight and pending.eps == self.eps


@register("norm", "channel_scale")
class ChannelScale(Norm):
    """A learned factor per channel (a layer scale): x * weight, no statistics. In an arrangement that keeps a 32-bit
    stream it rides on the kernel that adds a branch's rows (`ResidualStream(..., scale=weight32)`)."""

    graph_safe = True

    def __init__(self, hidden_size: int, init: float = 1.0) -> None:
        self.hidden_size, self.init = hidden_size, init
        self.weight: torch.Tensor | None = None
        self.weight32: torch.Tensor | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.hidden_size,), init=(self.init, 0.1))}

    def bind(self, params) -> None:
        super().bind(params)
        self.weight32 = self.weight.float().contiguous()

    def __call__(self, x, residual=None, rows=None):
        raise TypeError("a channel scale is applied by the arrangement that names it, in the kernel that adds the branch")


@register("norm", "dynamic_tanh")
class DynamicTanh(Norm):
    """tanh(alpha x) * weight + bias, element by element: no mean and no variance, so no reduction over
    the row. alpha is one learned scalar. All of it is 32-bit; what leaves for a projection is rounded to
    the storage type at the store. On a 32-bit residual stream the norm rides in the kernel that does the
    stream's pending sum (`ResidualStream.take`)."""

    graph_safe = True

    def __init__(self, hidden_size: int, alpha_init: float = 0.5) -> None:
        self.hidden_size, self.alpha_init = hidden_size, alpha_init
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None
        self.alpha: torch.Tensor | None = None
        self._f32: tuple[torch.Tensor, torch.Tensor, torch.Tensor] | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.hidden_size,), init=(1.0, 0.1)), "bias": ParamSpec((self.hidden_size,), init=(0.0, 0.02)),
                "alpha": ParamSpec((), init=(self.alpha_init, 0.05))}

    def bind(self, params) -> None:
        super().bind(params)
        # the kernels read 32-bit parameters (the stored type tells what the projections take)
        self._f32 = (self.alpha.float().reshape(1).contiguous(), self.weight.float().contiguous(), self.bias.float().contiguous())

    def elementwise(self) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """(alpha [1], weight, bias) in 32-bit: the norm as a kernel that works element by element takes it."""
        return self._f32

    def __call__(self, x, residual=None, rows=None):
        if isinstance(x, ResidualStream):
            if residual is not None:
                raise ValueError("a residual stream carries its own sum")
            stream, out = x.take(self, rows, self.weight.dtype)
            return out, (None if rows is not None else stream)
        out, total = hip.dyt(x, *self._f32, x.dtype, residual=residual, rows=rows, keep_sum=residual is not None)
        return out, (total if residual is not None else x)
