"""Recurrent mixers of the linear-attention kind: per head a matrix state S [dim, value_dim] that every token decays
channel by channel and adds k v^T to (`hip.decay_scan`). The state starts at zero, is kept in 32-bit floats in the
request's state slot and is carried from step to step; decays (their logarithms and exponentials), the state, the
read-out and the heads' norm are 32-bit in every storage type, and so are the projections' sums on their way there.

* `GatedLinearAttention` ("gated_linear_attention"): q = W_q h dim^(-1/2), k, v; a decay per key channel
  alpha = sigmoid(A_up (A_down h) + b)^(1 / tau); S <- diag(alpha) S + k v^T, o = S^T q; each head's o divided by its root
  mean square and multiplied by a weight of the head's size that all heads share, the heads side by side times
  silu(W_g h), then W_o.
* `ShiftedDecayRecurrence` ("shifted_decay_recurrence"): RWKV-style time mixing. With h' the previous token's h (zeros
  before a request's first token; the last h of a step is part of the state) each of r, k, v, g, w reads its own mix
  h + (h' - h) mu_s; r, k, v are projections of their mixes, the gate is silu(W_g x_g), the decay
  w = exp(-exp(W_up tanh(W_down x_w) + w0)); o = (S + diag(u) k v^T)^T r with a learned bonus u for the current token
  only, then S <- diag(w) S + k v^T; each head's o divided by its root mean square, the heads side by side times a
  weight and the gate, then W_o."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import LayerMemory, Mixer, ParamSpec, StateSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy


@register("mixer", "gated_linear_attention")
class GatedLinearAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay_rank: int, tau: float, norm_eps: float) -> None:
        if min(num_heads, head_dim, value_dim, decay_rank) <= 0 or head_dim > hip.DECAY_MAX_DIM or not tau > 0:
            raise ValueError(f"heads, head_dim (up to {hip.DECAY_MAX_DIM}), value_dim and the decays' rank are positive, and so is tau")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.decay_rank, self.tau, self.norm_eps = decay_rank, tau, norm_eps
        self.proj: torch.Tensor | None = None          # q | k | v | g
        self.decay_down: torch.Tensor | None = None
        self.decay_up: torch.Tensor | None = None
        self.decay_bias: torch.Tensor | None = None
        self.norm: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.proj_packed = self.o_packed = None

    @property
    def key_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def out_size(self) -> int:
        return self.num_heads * self.value_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"proj": ParamSpec((2 * self.key_size + 2 * self.out_size, self.hidden_size)),
                "decay_down": ParamSpec((self.decay_rank, self.hidden_size)),
                "decay_up": ParamSpec((self.key_size, self.decay_rank), init=(0.0, 0.2)),
                "decay_bias": ParamSpec((self.key_size,), "float32", init=(2.0, 1.0)),
                "norm": ParamSpec((self.value_dim,), "float32", init=(1.0, 0.1)),
                "o": ParamSpec((self.hidden_size, self.out_size))}

    def state_spec(self) -> StateSpec:
        return StateSpec((self.key_size * self.value_dim,), torch.float32)

    def keep_streaming_copies(self) -> int:
        self.proj_packed, self.o_packed = streaming_copy(self.proj), streaming_copy(self.o)
        return sum(c.nbytes() for c in (self.proj_packed, self.o_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        H, K, V = self.num_heads, self.key_size, self.out_size
        proj = linear(x, self.proj, out_dtype=torch.float32, packed=self.proj_packed)
        z = linear(linear(x, self.decay_down), self.decay_up, out_dtype=torch.float32)
        o = hip.decay_scan(proj[:, :K], proj[:, K:2 * K], proj[:, 2 * K:2 * K + V], z, self.decay_bias, mem.state, ctx.cu_seqlens,
                           ctx.state_slots, H, self.head_dim, self.value_dim, form="sigmoid_root", tau=self.tau,
                           q_scale=float(self.head_dim) ** -0.5, longest=ctx.max_query_len)
        gated = hip.mlstm_finish(o, self.norm, proj[:, 2 * K + V:], H, self.value_dim, self.norm_eps, x.dtype, silu_gate=True)
        return linear(gated, self.o, out_dtype=torch.float32, packed=self.o_packed)


SHIFT_MIXES = ("r", "k", "v", "g", "w")      # the order of the rows of `mu`


@register("mixer", "shifted_decay_recurrence")
class ShiftedDecayRecurrence(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, decay_rank: int, norm_eps: float) -> None:
        if min(num_heads, head_dim, decay_rank) <= 0 or head_dim > hip.DECAY_MAX_DIM:
            raise ValueError(f"heads, head_dim (up to {hip.DECAY_MAX_DIM}) and the decays' rank are positive")
        self.hidden_size, self.num_heads, self.head_dim, self.decay_rank, self.norm_eps = hidden_size, num_heads, head_dim, decay_rank, norm_eps
        self.mu: torch.Tensor | None = None            # [5, hidden]: of r, k, v, g, w
        self.r = self.k = self.v = self.g = None
        self.decay_down: torch.Tensor | None = None
        self.decay_up: torch.Tensor | None = None
        self.decay_bias: torch.Tensor | None = None
        self.bonus: torch.Tensor | None = None
        self.norm: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.packed: dict[str, hip.StreamingCopies | None] = {}

    @property
    def size(self) -> int:
        return self.num_heads * self.head_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        square = ParamSpec((self.size, self.hidden_size))
        return {"mu": ParamSpec((len(SHIFT_MIXES), self.hidden_size), "float32", init=(0.5, 0.2)),
                "r": square, "k": square, "v": square, "g": square,
                "decay_down": ParamSpec((self.decay_rank, self.hidden_size)),
                "decay_up": ParamSpec((self.size, self.decay_rank), init=(0.0, 0.2)),
                "decay_bias": ParamSpec((self.size,), "float32", init=(-1.0, 1.0)),
                "bonus": ParamSpec((self.num_heads, self.head_dim), "float32", init=(0.0, 0.5)),
                "norm": ParamSpec((self.size,), "float32", init=(1.0, 0.1)),
                "o": ParamSpec((self.hidden_size, self.size))}

    def state_spec(self) -> StateSpec:
        # S of every head, then the previous token's input row
        return StateSpec((self.size * self.head_dim + self.hidden_size,), torch.float32)

    def keep_streaming_copies(self) -> int:
        self.packed = {n: streaming_copy(getattr(self, n)) for n in ("r", "k", "v", "g", "o")}
        return sum(c.nbytes() for c in self.packed.values() if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        H, D = self.num_heads, self.head_dim
        kept = mem.state[:, self.size * D:]
        mixes = hip.token_shift(x, self.mu, kept, ctx)
        hip.token_shift_keep(kept, x, ctx)
        r, k, v, g = (linear(mixes[i], getattr(self, n), out_dtype=torch.float32, packed=self.packed.get(n))
                      for i, n in enumerate(SHIFT_MIXES[:4]))
        low = linear(mixes[4], self.decay_down, out_dtype=torch.float32)
        z = linear(hip.bias_activation(low, None, "tanh", x.dtype), self.decay_up, out_dtype=torch.float32)
        o = hip.decay_scan(r, k, v, z, self.decay_bias, mem.state, ctx.cu_seqlens, ctx.state_slots, H, D, D,
                           form="double_exponent", bonus=self.bonus, longest=ctx.max_query_len)
        gated = hip.mlstm_finish(o, self.norm, g, H, D, self.norm_eps, x.dtype, silu_gate=True)
        return linear(gated, self.o, out_dtype=torch.float32, packed=self.packed.get("o"))
