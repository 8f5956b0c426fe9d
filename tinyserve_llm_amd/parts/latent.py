"""Attention through a low-rank latent. A token's keys and values of all heads are up-projections of one latent c
(`kv_rank` numbers, divided by its root mean square and weighted), and every head's key has a further part of
`rot_dim` rotated dimensions that all heads share; queries come through a latent of their own (`q_rank`). Only
[c | rotated part] is cached, one row per token (and c once more, in the pages that hold values transposed). The up-projections move to the query's and the output's side:
    score_h(i, j) = ((W_uk,h^T q_h,plain) . c_j + q_h,rot . r_j) * scale,   out_h = W_uv,h (sum_j p_j c_j),
so attention runs as multi-query attention over the cached rows, whose first `kv_rank` numbers are also the values
(`hip.paged_attention_latent`), with a product per head before it and one after it (`hip.heads_gemm`). A sliding
window or chunks bound what a position sees; the heads' output may be multiplied by sigmoid(W_g x) before the output
projection. One fused projection gives query latent | latent and shared key part | gate, 32-bit on its way out;
norms, rotation (pairs (2i, 2i+1), a `rotary_frequencies` encoding with its amplitude), scores and weights are
32-bit in every storage type, and the queries stay 32-bit up to the scores."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import KVSpec, LayerMemory, Mixer, ParamSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy


@register("mixer", "latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int,
                 q_rank: int, position: str | None, scale: float | None = None, norm_eps: float = 1e-6, window: int = 0,
                 chunk: int = 0, gate: bool = False) -> None:
        if min(num_heads, head_dim, value_dim, kv_rank, q_rank) <= 0 or rot_dim < 0 or rot_dim % 2:
            raise ValueError("heads, head_dim, value_dim, kv_rank and q_rank are positive; rot_dim is even")
        if kv_rank > hip.LATENT_MAX_RANK or kv_rank + rot_dim > hip.LATENT_MAX_ROW:
            raise ValueError(f"a latent of up to {hip.LATENT_MAX_RANK} numbers, a cached row of up to {hip.LATENT_MAX_ROW}")
        if chunk < 0 or window < 0 or (chunk and window):
            raise ValueError("a sliding window or chunks (both >= 0), not both")
        if bool(rot_dim) != bool(position):
            raise ValueError("a rotated part needs a position encoding, and only a rotated part takes one")
        self.hidden_size, self.num_heads, self.head_dim, self.rot_dim = hidden_size, num_heads, head_dim, rot_dim
        self.value_dim, self.kv_rank, self.q_rank, self.position = value_dim, kv_rank, q_rank, position
        self.scale = scale if scale is not None else (head_dim + rot_dim) ** -0.5
        self.norm_eps, self.window, self.chunk, self.has_gate = norm_eps, window, chunk, gate
        self.down: torch.Tensor | None = None
        self.q_norm: torch.Tensor | None = None
        self.kv_norm: torch.Tensor | None = None
        self.uq: torch.Tensor | None = None
        self.uk: torch.Tensor | None = None
        self.uv: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.down_packed = self.uq_packed = self.o_packed = None
        self.uk_t: torch.Tensor | None = None      # W_uk per head with the head's dimensions along memory, for the matrix cores

    def bind(self, params) -> None:
        super().bind(params)
        if self.uk is not None and self.uk.dtype == torch.bfloat16 and self.uk.is_cuda:
            self.uk_t = self.uk.view(self.num_heads, self.head_dim, self.kv_rank).transpose(1, 2).contiguous()

    @property
    def out_size(self) -> int:
        return self.num_heads * self.value_dim

    @property
    def row_size(self) -> int:
        """Numbers a token caches: the latent and the shared rotated key part."""
        return self.kv_rank + self.rot_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        H, D, R = self.num_heads, self.head_dim, self.rot_dim
        return {"down": ParamSpec((self.q_rank + self.row_size + (self.out_size if self.has_gate else 0), self.hidden_size)),
                "q_norm": ParamSpec((self.q_rank,), "float32", init=(1.0, 0.1)),
                "kv_norm": ParamSpec((self.kv_rank,), "float32", init=(1.0, 0.1)),
                "uq": ParamSpec((H * (D + R), self.q_rank), init=(0.0, self.q_rank ** -0.5)),
                "uk": ParamSpec((H * D, self.kv_rank), init=(0.0, self.kv_rank ** -0.5)),
                "uv": ParamSpec((H * self.value_dim, self.kv_rank), init=(0.0, self.kv_rank ** -0.5)),
                "o": ParamSpec((self.hidden_size, self.out_size))}

    def widest_activation(self) -> int:
        return max(self.q_rank + self.row_size + self.out_size, 2 * self.num_heads * self.row_size)

    def kv_spec(self) -> KVSpec:
        # one row per token; its first kv_rank numbers are the values, which the cache keeps once more in the pages that
        # hold values transposed, for the matrix-core kernel
        return KVSpec(1, self.row_size, self.window or self.chunk, self.kv_rank)

    def keep_streaming_copies(self) -> int:
        self.down_packed, self.uq_packed, self.o_packed = streaming_copy(self.down), streaming_copy(self.uq), streaming_copy(self.o)
        return sum(c.nbytes() for c in (self.down_packed, self.uq_packed, self.o_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        H, D, R, V, C, T = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank, ctx.num_tokens
        enc = ctx.position_encodings[self.position] if self.position else None
        freqs, amplitude = (enc.frequencies(), getattr(enc, "amplitude", 1.0)) if enc is not None else (None, 1.0)
        if enc is not None and not getattr(enc, "interleaved", True):
            raise ValueError("the latent's rotated part pairs dimensions (2i, 2i + 1)")
        down = linear(x, self.down, out_dtype=torch.float32, packed=self.down_packed)
        slots, cache, values = (ctx.slot_mapping[mem.space], mem.k_cache, mem.v_cache) if mem.store else (None, None, None)
        cq = hip.latent_finish(down, 0, self.q_rank, self.q_rank, C, R, self.q_norm, self.kv_norm, self.norm_eps, freqs, amplitude,
                               ctx.positions, slots, cache, x.dtype, v_cache=values)
        q = linear(cq, self.uq, out_dtype=torch.float32, packed=self.uq_packed).view(T, H, D + R)
        # the keys' up-projection on the query's side: W_uk,h^T q_h beside the turned part, in the cached row's order
        absorbed = torch.empty((T, H, C + R), dtype=torch.float32, device=x.device)
        hip.heads_gemm(q[:, :, :D], self.uk.view(H, D, C) if self.uk_t is None else self.uk_t.transpose(1, 2), absorbed[:, :, :C])
        if R:
            hip.rotate_heads(absorbed[:, :, C:], q[:, :, D:], freqs, amplitude, ctx.positions, interleaved=True)
        mixed = hip.paged_attention_latent(absorbed, mem.k_cache, C, ctx, mem.space, self.scale, self.window, self.chunk, out_dtype=x.dtype,
                                           v_cache=mem.v_cache)
        # the values' up-projection on the output's side, the gate on its way out
        heads = torch.empty((T, H, V), dtype=x.dtype, device=x.device)
        hip.heads_gemm(mixed, self.uv.view(H, V, C).transpose(1, 2), heads,
                       gate=down[:, self.q_rank + self.row_size:] if self.has_gate else None)
        return linear(heads.view(T, self.out_size), self.o, out_dtype=torch.float32, packed=self.o_packed)
