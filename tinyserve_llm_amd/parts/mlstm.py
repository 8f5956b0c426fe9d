"""mLSTM: a recurrent mixer with a matrix memory per head. One fused projection gives, per token,
q | k | v | a_i | a_f | g (heads x dim, heads x dim, heads x value_dim, a number per head for each gate, and an output
gate as wide as the values), 32-bit on its way out. With q times dim^(-1/2), the log input gate
i = cap tanh((a_i + b_i) / cap) and the log forget gate f = logsigmoid(cap tanh((a_f + b_f) / cap)), a head's state
moves as
    m' = max(f + m, i),  S' = exp(f + m - m') S + exp(i - m') k v^T,  n' = exp(f + m - m') n + exp(i - m') k,
and reads out o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6); each head's o is divided by its root mean square, the
heads side by side are multiplied by a weight and by sigmoid(g), and the output projection follows. S, n and m start at
zero, are kept in 32-bit floats in the request's state slot, and are carried from step to step (`hip.mlstm_scan`:
token by token where every request feeds few tokens, in chunks of 64 tokens where one feeds many);
gates, exponentials and the heads' norm are 32-bit in every storage type."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import LayerMemory, Mixer, ParamSpec, StateSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy


@register("mixer", "mlstm")
class MLSTM(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, gate_cap: float, norm_eps: float) -> None:
        if min(num_heads, head_dim, value_dim) <= 0 or head_dim > hip.MLSTM_MAX_DIM or not gate_cap > 0:
            raise ValueError(f"heads, head_dim (up to {hip.MLSTM_MAX_DIM}) and value_dim are positive, and so is the gates' cap")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.gate_cap, self.norm_eps = gate_cap, norm_eps
        self.proj: torch.Tensor | None = None
        self.gate_bias: torch.Tensor | None = None      # [2 heads]: of the input gates, then of the forget gates
        self.norm: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.proj_packed = self.o_packed = None

    @property
    def out_size(self) -> int:
        return self.num_heads * self.value_dim

    @property
    def gate_at(self) -> int:
        """Column of the fused projection where the output gate starts."""
        return 2 * self.num_heads * self.head_dim + self.out_size + 2 * self.num_heads

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"proj": ParamSpec((self.gate_at + self.out_size, self.hidden_size)),
                "gate_bias": ParamSpec((2 * self.num_heads,), "float32", init=(0.0, 1.0)),
                "norm": ParamSpec((self.out_size,), "float32", init=(1.0, 0.1)),
                "o": ParamSpec((self.hidden_size, self.out_size))}

    def state_spec(self) -> StateSpec:
        return StateSpec((hip.mlstm_state_size(self.num_heads, self.head_dim, self.value_dim),), torch.float32)

    def keep_streaming_copies(self) -> int:
        self.proj_packed, self.o_packed = streaming_copy(self.proj), streaming_copy(self.o)
        return sum(c.nbytes() for c in (self.proj_packed, self.o_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        H = self.num_heads
        proj = linear(x, self.proj, out_dtype=torch.float32, packed=self.proj_packed)
        o = hip.mlstm_scan(proj, self.gate_bias[:H], self.gate_bias[H:], mem.state, ctx.cu_seqlens, ctx.state_slots, H,
                           self.head_dim, self.value_dim, self.gate_cap, host_cu_seqlens=ctx.host_cu_seqlens, scratch=ctx.scratch)
        gated = hip.mlstm_finish(o, self.norm, proj[:, self.gate_at:], H, self.value_dim, self.norm_eps, x.dtype)
        return linear(gated, self.o, out_dtype=torch.float32, packed=self.o_packed)
