"""SiLU-gated feed-forward (tinyserve_llm/model/llama.py:77-83,215-225): one fused projection gives
[gate | up], then silu(gate) * up, then the down projection."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import FeedForward, ParamSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy


@register("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True
    takes_deferred_norm = True
    finishes_into_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu") -> None:
        if activation != "silu":
            raise ValueError(f"activation {activation!r}: the gated feed-forward kernel computes silu")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None
        self.gate_up_packed = None       # `streaming_copy` of each weight, if the model keeps them
        self.down_packed = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"gate_up": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
                "down": ParamSpec((self.hidden_size, self.intermediate_size))}

    def keep_streaming_copies(self) -> int:
        self.gate_up_packed, self.down_packed = streaming_copy(self.gate_up), streaming_copy(self.down)
        return sum(c.nbytes() for c in (self.gate_up_packed, self.down_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, then=None) -> torch.Tensor:
        gated = linear(x, self.gate_up, glu=True, packed=self.gate_up_packed, feeds=self.down)
        return linear(gated, self.down, packed=self.down_packed, then=then)


@register("feed_forward", "dense_mlp")
class DenseMLP(FeedForward):
    """A feed-forward without a gate: W_down act(W_up h + b_up) + b_down, `activation` one of
    `hip.ACTIVATIONS` ("relu2": the square of relu). The up projection's sums stay 32-bit until bias and
    activation are applied (by the projection's own kernel for steps of few rows, by a kernel of their own otherwise); the down projection's result is 32-bit. `forward(..., defer_bias=True)`
    returns (W_down a, b_down) for a caller that adds the bias with its residual sum."""

    graph_safe = True
    can_defer_bias = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2", bias: bool = True) -> None:
        if activation not in hip.ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: one of {sorted(hip.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.activation, self.has_bias = hidden_size, intermediate_size, activation, bias
        self.up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None
        self.up_bias: torch.Tensor | None = None
        self.down_bias: torch.Tensor | None = None
        self.up_packed = None
        self.down_packed = None

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {"up": ParamSpec((self.intermediate_size, self.hidden_size)),
                 "down": ParamSpec((self.hidden_size, self.intermediate_size))}
        if self.has_bias:
            specs["up_bias"] = ParamSpec((self.intermediate_size,), init=(0.0, 0.02))
            specs["down_bias"] = ParamSpec((self.hidden_size,), init=(0.0, 0.02))
        return specs

    def keep_streaming_copies(self) -> int:
        self.up_packed, self.down_packed = streaming_copy(self.up), streaming_copy(self.down)
        return sum(c.nbytes() for c in (self.up_packed, self.down_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, defer_bias: bool = False):
        if hip.skinny8_act_takes(x, self.up, self.up_bias):
            # few rows: bias and activation ride on the projection's way out, from its 32-bit sums
            act = hip.gemm_skinny8_act(x, self.up, self.up_bias, self.activation, x.dtype,
                                       None if self.up_packed is None else self.up_packed.by8)
        else:
            up = linear(x, self.up, out_dtype=torch.float32, packed=self.up_packed)
            act = hip.bias_activation(up, self.up_bias, self.activation, x.dtype)
        down = linear(act, self.down, out_dtype=torch.float32, packed=self.down_packed)
        if defer_bias:
            return down, self.down_bias
        return down if self.down_bias is None else hip.bias_activation(down, self.down_bias, "none", torch.float32)


@register("feed_forward", "capped_glu")
class CappedGLU(FeedForward):
    """A gated feed-forward with capped branches: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
    W_down (g sigmoid(slope g) (u + up_shift)); limit <= 0: no cap. One fused projection gives gate | up as
    32-bit sums; the unit is taken in 32-bit and rounded to the storage type for the down projection, whose
    result is 32-bit. `activation` "relu": the gate passes where it is positive, max(g, 0) (u + up_shift), instead of
    through the sigmoid."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float = 0.0, slope: float = 1.702,
                 up_shift: float = 1.0, activation: str = "sigmoid") -> None:
        if activation not in ("sigmoid", "relu"):
            raise ValueError(f"activation {activation!r}: 'sigmoid' (g sigmoid(slope g)) or 'relu'")
        self.activation = activation
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.limit, self.slope, self.up_shift = limit, slope, up_shift
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None
        self.gate_up_packed = None
        self.down_packed = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"gate_up": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
                "down": ParamSpec((self.hidden_size, self.intermediate_size))}

    def keep_streaming_copies(self) -> int:
        self.gate_up_packed, self.down_packed = streaming_copy(self.gate_up), streaming_copy(self.down)
        return sum(c.nbytes() for c in (self.gate_up_packed, self.down_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        sums = linear(x, self.gate_up, out_dtype=torch.float32, packed=self.gate_up_packed)
        unit = hip.capped_glu(sums, self.limit, self.slope, self.up_shift, x.dtype, relu=self.activation == "relu")
        return linear(unit, self.down, out_dtype=torch.float32, packed=self.down_packed)


@register("feed_forward", "none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: `forward` gives None, which a block's residual sum leaves out."""

    graph_safe = True

    def forward(self, x, ctx: StepContext, **_):
        return None
