"""Two mixers side by side: both read the same input, and the result is left_scale * left + right_scale * right. Each is a
mixer of its own kind with its own parameters (`left_...`, `right_...`); at most one of them keeps a cache and at most
one keeps per-request state, which the pair passes on as its own."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import KVSpec, LayerMemory, Mixer, ParamSpec, PartSpec, StateSpec, StepContext, make, register


@register("mixer", "side_by_side")
class SideBySide(Mixer):
    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0) -> None:
        self.left, self.right = make("mixer", left), make("mixer", right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        if self.left.kv_spec() is not None and self.right.kv_spec() is not None:
            raise ValueError("of two mixers side by side at most one keeps a cache")
        if self.left.state_spec() is not None and self.right.state_spec() is not None:
            raise ValueError("of two mixers side by side at most one keeps per-request state")

    @property
    def graph_safe(self) -> bool:
        return self.left.graph_safe and self.right.graph_safe

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {f"left_{n}": ps for n, ps in self.left.param_specs().items()}
        specs.update({f"right_{n}": ps for n, ps in self.right.param_specs().items()})
        return specs

    def bind(self, params) -> None:
        self.left.bind({n[len("left_"):]: t for n, t in params.items() if n.startswith("left_")})
        self.right.bind({n[len("right_"):]: t for n, t in params.items() if n.startswith("right_")})

    def kv_spec(self) -> KVSpec | None:
        return self.left.kv_spec() or self.right.kv_spec()

    def state_spec(self) -> StateSpec | None:
        return self.left.state_spec() or self.right.state_spec()

    def widest_activation(self) -> int:
        return max(self.left.widest_activation(), self.right.widest_activation())

    def keep_streaming_copies(self) -> int:
        return self.left.keep_streaming_copies() + self.right.keep_streaming_copies()

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        a = self.left.forward(x, ctx, mem)
        b = self.right.forward(x, ctx, mem)
        return hip.scaled_sum(a, self.left_scale, b, self.right_scale)
