"""Per-layer token inputs: what a layer adds to the residual stream from the token ids themselves.

`GatedTokenRows` ("gated_token_rows"): a second, narrow token table gives every token a row of which each layer reads
a stretch of its own, e = table[token, offset : offset + dim]; with x the stream after the layer's other parts,
g = act(W_gate x) * e, y = W_proj g, and the stream takes y divided by its root mean square times a weight (`post`: an
RMS norm with a plain weight, whatever norm the model's layers have). The gate's sums, the activation and the norm are
32-bit; the two projections read operands of the engine's storage type."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import ParamSpec, StepContext, TokenInput, register
from tinyserve_llm_amd.parts.linear import linear
from tinyserve_llm_amd.parts.norm import RMSNorm


@register("token_input", "gated_token_rows")
class GatedTokenRows(TokenInput):
    graph_safe = True

    def __init__(self, hidden_size: int, dim: int, offset: int, eps: float, activation: str = "gelu_tanh") -> None:
        if dim <= 0 or offset < 0 or activation not in hip.ACTIVATIONS:
            raise ValueError(f"a positive dim, an offset into the table's rows, an activation of {sorted(hip.ACTIVATIONS)}")
        self.hidden_size, self.dim, self.offset, self.activation = hidden_size, dim, offset, activation
        self.post = RMSNorm(hidden_size, eps)
        self.gate: torch.Tensor | None = None
        self.proj: torch.Tensor | None = None
        self.table: torch.Tensor | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"gate": ParamSpec((self.dim, self.hidden_size)), "proj": ParamSpec((self.hidden_size, self.dim)),
                "norm": ParamSpec((self.hidden_size,), init=(0.2, 0.05))}

    def bind(self, params) -> None:
        super().bind({n: t for n, t in params.items() if n != "norm"})
        self.post.bind({"weight": params["norm"]})

    def attach(self, table: torch.Tensor | None) -> None:
        if table is None or table.dim() != 2 or table.shape[1] < self.offset + self.dim:
            raise ValueError(f"the embedding has no second table whose rows reach {self.offset + self.dim}")
        self.table = table

    @property
    def operand_dtype(self) -> torch.dtype:
        return self.gate.dtype

    def forward(self, rows: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        sums = linear(rows, self.gate, out_dtype=torch.float32)
        gated = hip.gather_gate(sums, self.table, self.offset, ctx.token_ids, self.activation, rows.dtype)
        return linear(gated, self.proj, out_dtype=torch.float32)
