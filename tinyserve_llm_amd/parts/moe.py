"""A mixture of experts as a feed-forward: a router scores the experts for every token, the token goes
through the `top` best of them, and their outputs are added with the router's weights; a shared expert
may run for every token beside them. Routing lives inside the part: a step's (token, expert) pairs are
grouped by expert on the device (`hip.moe_group`), so that the experts' products run as one launch over
tiles of rows and nothing comes back to the host (the part can be recorded into a graph)."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import FeedForward, ParamSpec, StepContext, register
from tinyserve_llm_amd.parts.mlp import CappedGLU


@register("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """Experts of the capped gated form (`parts.mlp.CappedGLU`: limit, slope, up_shift), without biases.
    Scores s = sigmoid(W_r h), the logits in 32-bit; the `top` experts with the largest s + correction are
    chosen (`correction` False: largest s); their weights are their s without the correction, over the chosen
    ones' sum (+ 1e-20) if `normalize`, times `router_scale`. `shared`: the constructor arguments of a
    `CappedGLU` that runs for every token and is added (None: no shared expert). The experts' matrices are
    stacked: gate_up [experts, 2 ff, hidden], down [experts, hidden, ff]. `scoring` "softmax_all": s is the softmax
    over all the router's outputs instead of sigmoids. `identity`: the router has that many more outputs than there
    are experts with matrices; they stand for experts that hand their input through (times the weight). `shared_gate`:
    the shared expert's output is multiplied by sigmoid(w_sg . h), one number per token; w_sg is the router's last
    row, so that its logit is 32-bit like the others."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_experts: int, top: int, intermediate_size: int, limit: float = 0.0,
                 slope: float = 1.702, up_shift: float = 1.0, router_scale: float = 1.0, normalize: bool = True,
                 correction: bool = True, shared: dict | None = None, scoring: str = "sigmoid", identity: int = 0,
                 shared_gate: bool = False) -> None:
        if scoring not in ("sigmoid", "softmax_all") or identity < 0 or (shared_gate and shared is None):
            raise ValueError("scoring 'sigmoid' or 'softmax_all'; identity >= 0; a gate on the shared expert needs one")
        if top > num_experts + identity or num_experts + identity > hip.MOE_MAX_EXPERTS:
            raise ValueError(f"top {top} of {num_experts} + {identity} experts, of which there may be {hip.MOE_MAX_EXPERTS}")
        self.scoring, self.identity, self.shared_gate = scoring, identity, shared_gate
        if not 1 <= top <= min(num_experts + identity, hip.MOE_MAX_TOP) or num_experts > hip.MOE_MAX_EXPERTS:
            raise ValueError(f"top {top} of {num_experts} experts: 1 <= top <= min(experts, {hip.MOE_MAX_TOP}), "
                             f"experts <= {hip.MOE_MAX_EXPERTS}")
        self.hidden_size, self.num_experts, self.top, self.intermediate_size = hidden_size, num_experts, top, intermediate_size
        self.limit, self.slope, self.up_shift = limit, slope, up_shift
        self.router_scale, self.normalize, self.has_correction = router_scale, normalize, correction
        self.shared = CappedGLU(hidden_size=hidden_size, **shared) if shared is not None else None
        self.router: torch.Tensor | None = None
        self.correction: torch.Tensor | None = None
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        E, F, H = self.num_experts, self.intermediate_size, self.hidden_size
        specs = {"router": ParamSpec((E + self.identity + int(self.shared_gate), H), "float32", init=(0.0, 0.2)),
                 "gate_up": ParamSpec((E, 2 * F, H)), "down": ParamSpec((E, H, F))}
        if self.has_correction:
            specs["correction"] = ParamSpec((E + self.identity,), "float32", init=(0.0, 0.1))
        if self.shared is not None:
            specs.update({f"shared_{name}": ps for name, ps in self.shared.param_specs().items()})
        return specs

    def bind(self, params) -> None:
        own = {n: t for n, t in params.items() if not n.startswith("shared_")}
        super().bind(own)
        if self.shared is not None:
            self.shared.bind({n[len("shared_"):]: t for n, t in params.items() if n.startswith("shared_")})

    def widest_activation(self) -> int:
        shared = self.shared.widest_activation() if self.shared is not None else 0
        return max(2 * self.top * self.hidden_size, self.top * self.intermediate_size, shared)

    def keep_streaming_copies(self) -> int:
        return self.shared.keep_streaming_copies() if self.shared is not None else 0

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        routed = hip.moe_route(x, self.router, self.correction, self.top, self.router_scale, self.normalize,
                               softmax_all=self.scoring == "softmax_all", extras=int(self.shared_gate))
        experts, weights = routed[0], routed[1]
        tile_rows = hip.moe_tile_rows(experts.numel(), self.num_experts, x.dtype, (self.hidden_size, self.intermediate_size))
        grouped = hip.moe_group(experts, self.num_experts, tile_rows)
        unit = hip.moe_gemm(x, self.gate_up, grouped, x.dtype, per_token=True, glu=(self.limit, self.slope, self.up_shift))
        rows = hip.moe_gemm(unit, self.down, grouped, torch.float32, per_token=False)
        shared = self.shared.forward(x, ctx) if self.shared is not None else None
        return hip.moe_combine(rows, weights, shared, identity=(experts, self.num_experts, x) if self.identity else None,
                               shared_gate=routed[2] if self.shared_gate else None)


@register("feed_forward", "routed_dense_experts")
class RoutedDenseExperts(FeedForward):
    """Experts without a gate and without biases: W_down act(W_up h), `activation` "relu2" (the square of relu) or
    "none". Router logits z = W_r h in 32-bit; the `top` experts with the largest logits are chosen and their weights
    are the softmax over the chosen logits alone (`scoring` "softmax_chosen"), or sigmoid scores normalised over the
    chosen (`scoring` "sigmoid"), times `router_scale`. The experts' matrices are stacked: up [experts, ff, hidden],
    down [experts, hidden, ff]; the activation rides on the up product's way out, the down product and the weighted
    sum are 32-bit."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_experts: int, top: int, intermediate_size: int, activation: str = "relu2",
                 scoring: str = "softmax_chosen", router_scale: float = 1.0) -> None:
        if not 1 <= top <= min(num_experts, hip.MOE_MAX_TOP) or num_experts > hip.MOE_MAX_EXPERTS:
            raise ValueError(f"top {top} of {num_experts} experts: 1 <= top <= min(experts, {hip.MOE_MAX_TOP}), "
                             f"experts <= {hip.MOE_MAX_EXPERTS}")
        if activation not in ("relu2", "none") or scoring not in ("softmax_chosen", "sigmoid"):
            raise ValueError("activation 'relu2' or 'none'; scoring 'softmax_chosen' or 'sigmoid'")
        self.hidden_size, self.num_experts, self.top, self.intermediate_size = hidden_size, num_experts, top, intermediate_size
        self.activation, self.scoring, self.router_scale = activation, scoring, router_scale
        self.router: torch.Tensor | None = None
        self.up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        E, F, H = self.num_experts, self.intermediate_size, self.hidden_size
        return {"router": ParamSpec((E, H), "float32", init=(0.0, 0.2)), "up": ParamSpec((E, F, H)), "down": ParamSpec((E, H, F))}

    def widest_activation(self) -> int:
        return max(2 * self.top * self.hidden_size, self.top * self.intermediate_size)

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        experts, weights = hip.moe_route(x, self.router, None, self.top, self.router_scale, True,
                                         softmax_chosen=self.scoring == "softmax_chosen")
        tile_rows = hip.moe_tile_rows(experts.numel(), self.num_experts, x.dtype, (self.hidden_size, self.intermediate_size))
        grouped = hip.moe_group(experts, self.num_experts, tile_rows)
        act = hip.moe_gemm(x, self.up, grouped, x.dtype, per_token=True, activation=self.activation)
        rows = hip.moe_gemm(act, self.down, grouped, torch.float32, per_token=False)
        return hip.moe_combine(rows, weights, None)
