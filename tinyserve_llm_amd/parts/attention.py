"""Grouped-query attention over the paged cache (tinyserve_llm/model/llama.py:189-212,
tinyserve_llm/engine/model_runner.py:100-108, tinyserve_llm/attention/torch_paged.py:15-46).

One fused projection gives q | k | v; q and k are rotated by the named position encoding; k and v
of the step's tokens are written to their cache slots; then every token attends, causally, over
the cache pages of its request (its own key included), and the output projection follows.
For steps of few tokens (`hip.qkv_rope_max_rows` says how many for the layer's width) projection,
rotation and cache write are one kernel (`hip.qkv_rope_store`), which also takes a deferred norm
where it reaches; larger steps run them one after the other.
"""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import KVSpec, LayerMemory, Mixer, ParamSpec, StateSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import DeferredNorm, linear, streaming_copy


@register("mixer", "attention")
class Attention(Mixer):
    graph_safe = True
    takes_deferred_norm = True
    finishes_into_norm = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: str | None = "rope", scale: float | None = None, window: int = 0) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not divide into {num_kv_heads} key/value heads")
        if head_dim % 16 or head_dim > 256:
            raise ValueError(f"head_dim {head_dim}: the attention kernels take multiples of 16 up to 256")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.position = position
        self.scale = scale if scale is not None else head_dim ** -0.5
        self.window = window
        self.qkv: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.qkv_packed: hip.StreamingCopies | None = None
        self.qkv_rope_packed: torch.Tensor | None = None     # for the one-kernel path: `hip.pack_weight_rope`
        self.o_packed: hip.StreamingCopies | None = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def keep_streaming_copies(self) -> int:
        self.qkv_packed, self.o_packed = streaming_copy(self.qkv), streaming_copy(self.o)
        if self.qkv_packed is not None and self.qkv_packed.by16 is not None and self.head_dim % 32 == 0:
            self.qkv_rope_packed = hip.pack_weight_rope(self.qkv, self.head_dim)
            if hip.qkv_rope_max_rows(self.hidden_size) >= hip.STREAMING_MAX_ROWS:
                self.qkv_packed = None           # every step that would stream the plain copy takes the one-kernel path
        copies = sum(c.nbytes() for c in (self.qkv_packed, self.o_packed) if c is not None)
        return copies + (0 if self.qkv_rope_packed is None else self.qkv_rope_packed.numel() * 2)

    def _project_fused(self, x, table, positions, slots, k_store, v_store) -> torch.Tensor | None:
        """Projection, rotation and cache write in one kernel where a step is small enough for the
        weight-streaming kernel (in two, with the reduction in slices, for a few dozen rows over a
        reduction that kernel does not take); None where neither serves."""
        d = x if isinstance(x, DeferredNorm) else None
        by16 = self.qkv_rope_packed
        if d is not None and d.prepared is not None:     # the norm's first half is done: its operand, then a scale per row
            rows = d.prepared.operand
            if not hip.qkv_rope_fuses(rows, self.qkv, self.head_dim, k_store, table=table):
                slices = 0 if by16 is None else hip.qkv_rope_sliced_slices(rows, self.qkv, self.head_dim, k_store, table)
                if not slices:
                    return None
                return hip.qkv_rope_store_sliced(rows, by16, slices, table, positions, slots, k_store, v_store, self.num_heads,
                                                 self.num_kv_heads, self.head_dim, eps=d.eps, squares=d.prepared.squares)
            return hip.qkv_rope_store(rows, self.qkv, table, positions, slots, k_store, v_store, self.num_heads,
                                      self.num_kv_heads, self.head_dim, eps=d.eps, packed=by16, squares=d.prepared.squares)[0]
        rows = d.x if d is not None else x
        if not (rows.is_cuda and hip.qkv_rope_fuses(rows, self.qkv, self.head_dim, k_store, table=table)):
            slices = 0 if by16 is None or not rows.is_cuda else hip.qkv_rope_sliced_slices(rows, self.qkv, self.head_dim, k_store, table)
            if not slices:
                return None
            if d is not None:
                rows = d.materialize()           # the norm by its own kernel
            return hip.qkv_rope_store_sliced(rows, by16, slices, table, positions, slots, k_store, v_store, self.num_heads,
                                             self.num_kv_heads, self.head_dim)
        if d is not None and not (hip.qkv_rope_fuses(rows, self.qkv, self.head_dim, k_store, norm=True)
                                  and d.weight.dtype == torch.bfloat16
                                  and (d.residual is None or d.residual.is_contiguous())):
            rows, d = d.materialize(), None      # the norm by its own kernel, the rest in one
        if d is None:
            return hip.qkv_rope_store(rows, self.qkv, table, positions, slots, k_store, v_store, self.num_heads,
                                      self.num_kv_heads, self.head_dim, packed=by16)[0]
        q, d.residual_out = hip.qkv_rope_store(rows, self.qkv, table, positions, slots, k_store, v_store, self.num_heads,
                                               self.num_kv_heads, self.head_dim, residual=d.residual,
                                               norm_weight=d.weight, eps=d.eps, packed=by16)
        return q

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"qkv": ParamSpec((self.q_size + 2 * self.kv_size, self.hidden_size)),
                "o": ParamSpec((self.hidden_size, self.q_size))}

    def kv_spec(self) -> KVSpec:
        return KVSpec(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory, then=None) -> torch.Tensor:
        table = ctx.position_encodings[self.position].rotary_table() if self.position else None
        slots = ctx.slot_mapping[mem.space] if mem.store else None
        k_store, v_store = (mem.k_cache, mem.v_cache) if mem.store else (None, None)
        q = self._project_fused(x, table, ctx.positions, slots, k_store, v_store)
        if q is None:
            qkv = linear(x, self.qkv, packed=self.qkv_packed)
            q = hip.rope_store(qkv, table, ctx.positions, slots, k_store, v_store, self.num_heads, self.num_kv_heads,
                               self.head_dim)
        # (a single token: the o projection adds the chunks of a split walk up itself, on its way in)
        o = hip.paged_attention(q, mem.k_cache, mem.v_cache, ctx, mem.space, self.scale, self.window,
                                leave_split=hip.split_attention_fuses(ctx.num_tokens, self.o))
        if not isinstance(o, hip.SplitAttention):
            o = o.view(ctx.num_tokens, self.q_size)
        return linear(o, self.o, packed=self.o_packed, then=then)


@register("mixer", "attention_general")
class GeneralAttention(Mixer):
    """Grouped-query attention with the options the fused rotate-half path above does not have, each
    a constructor argument: value heads of a size of their own (`value_dim`), rotary positions taken
    from frequencies (`position` names a `rotary_frequencies` encoding: interleaved or half pairs, a
    leading part of the head), q and k heads divided by their root mean square after the rotation
    (`qk_norm_eps`), value heads likewise before they are cached (`v_norm_eps`), scores capped as
    softcap * tanh(score / softcap), and a softmax with a sink (one more in the denominator).
    Separate q, k, v weights of a checkpoint land in row slices of one fused projection, whose output,
    like the output projection's, is 32-bit; rotation, norms, scores and weights are 32-bit in every
    storage type (`hip.qkv_finish`, `hip.paged_attention_general`); in bfloat16, where key and value heads
    have one of the matrix-core kernels' sizes, those kernels' general variants run instead, which cap
    in 32-bit and carry the weights into the products in two bfloat16 terms."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int | None = None,
                 position: str | None = None, scale: float | None = None, softcap: float = 0.0, sink: bool = False,
                 qk_norm_eps: float | None = None, v_norm_eps: float | None = None, window: int = 0, chunk: int = 0,
                 learned_sink: bool = False, projection_norm_eps: float | None = None, head_norm_eps: float | None = None,
                 value_position: str | None = None, head_gate: bool = False) -> None:
        """Further options. `chunk` (instead of `window`): a position sees the keys of its own chunk of that many
        positions, chunks counted from position 0. `learned_sink`: exp(sink[h]), a learned number per head, in the
        softmax's denominator (instead of `sink`'s 1). `projection_norm_eps`: the whole q projection of a token (all
        heads at once), and likewise the whole k projection, is divided by its root mean square and multiplied by a
        weight of that size (`q_norm`, `k_norm`, 32-bit) before the heads turn. `head_norm_eps` (instead): every q head and
        every k head is divided by its own root mean square and multiplied by a weight of the head's size that all heads
        share (`q_norm`, `k_norm`), before the heads turn. `value_position` names a `rotary_frequencies` encoding over
        all of `value_dim`: the value at position j is turned by j before it is cached, and each head's output at position
        i is turned back by i. `head_gate`: each head's output (turned back) is multiplied by sigmoid(W_gate h)_head, one
        number per head."""
        if projection_norm_eps is not None and head_norm_eps is not None:
            raise ValueError("a norm over the whole q and k projections or over every head, not both")
        if head_gate and value_position is None:
            raise ValueError("the gate per head rides on the kernel that turns the heads' outputs back (value_position)")
        if chunk < 0 or window < 0 or (chunk and window):
            raise ValueError("a sliding window or chunks (both >= 0), not both")
        if sink and learned_sink:
            raise ValueError("a sink of score 0 or a learned one, not both")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not divide into {num_kv_heads} key/value heads")
        value_dim = head_dim if value_dim is None else value_dim
        if not (0 < head_dim <= 256 and 0 < value_dim <= 256):
            raise ValueError(f"head sizes {head_dim} / {value_dim}: the attention kernels take up to 256")
        if softcap < 0:
            raise ValueError(f"softcap {softcap}: positive, or 0 for none")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.position = head_dim, value_dim, position
        self.scale = scale if scale is not None else head_dim ** -0.5
        self.softcap, self.sink, self.qk_norm_eps, self.v_norm_eps, self.window = softcap, sink, qk_norm_eps, v_norm_eps, window
        self.chunk, self.learned_sink, self.projection_norm_eps = chunk, learned_sink, projection_norm_eps
        self.head_norm_eps, self.value_position, self.head_gate = head_norm_eps, value_position, head_gate
        self.gate: torch.Tensor | None = None
        self.qkv: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None
        self.sinks: torch.Tensor | None = None
        self.qkv_packed: hip.StreamingCopies | None = None
        self.o_packed: hip.StreamingCopies | None = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def k_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_kv_heads * self.value_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {"qkv": ParamSpec((self.q_size + self.k_size + self.v_size, self.hidden_size)),
                 "o": ParamSpec((self.hidden_size, self.num_heads * self.value_dim))}
        if self.projection_norm_eps is not None:
            specs["q_norm"] = ParamSpec((self.q_size,), "float32", init=(1.0, 0.1))
            specs["k_norm"] = ParamSpec((self.k_size,), "float32", init=(1.0, 0.1))
        if self.head_norm_eps is not None:
            specs["q_norm"] = ParamSpec((self.head_dim,), "float32", init=(1.0, 0.1))
            specs["k_norm"] = ParamSpec((self.head_dim,), "float32", init=(1.0, 0.1))
        if self.head_gate:
            specs["gate"] = ParamSpec((self.num_heads, self.hidden_size))
        if self.learned_sink:
            specs["sinks"] = ParamSpec((self.num_heads,), "float32", init=(0.0, 1.0))
        return specs

    def kv_spec(self) -> KVSpec:
        # (a chunk's keys lie within the last `chunk` positions: the cache may give back what lies before them)
        return KVSpec(self.num_kv_heads, self.head_dim, self.window or self.chunk,
                      None if self.value_dim == self.head_dim else self.value_dim)

    def keep_streaming_copies(self) -> int:
        self.qkv_packed, self.o_packed = streaming_copy(self.qkv), streaming_copy(self.o)
        return sum(c.nbytes() for c in (self.qkv_packed, self.o_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        enc = ctx.position_encodings[self.position] if self.position else None
        slots = ctx.slot_mapping[mem.space] if mem.store else None
        k_store, v_store = (mem.k_cache, mem.v_cache) if mem.store else (None, None)
        qkv = linear(x, self.qkv, out_dtype=torch.float32, packed=self.qkv_packed)
        if self.projection_norm_eps is not None:         # in place, each over its whole stretch of the row
            hip.segment_rmsnorm_pair(qkv, (0, self.q_size, self.q_norm), (self.q_size, self.k_size, self.k_norm), self.projection_norm_eps)
        value_enc = ctx.position_encodings[self.value_position] if self.value_position else None
        if self.head_norm_eps is not None or value_enc is not None:      # in place: the heads' norms, the values' turn
            hip.qkv_prepare(qkv, ctx.positions, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                            q_weight=self.q_norm if self.head_norm_eps is not None else None,
                            k_weight=self.k_norm if self.head_norm_eps is not None else None, eps=self.head_norm_eps or 0.0,
                            value_freqs=None if value_enc is None else value_enc.frequencies(),
                            value_interleaved=getattr(value_enc, "interleaved", False))
        q = hip.qkv_finish(qkv, enc.frequencies() if enc is not None else None, ctx.positions, slots, k_store, v_store,
                           self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, x.dtype,
                           interleaved=getattr(enc, "interleaved", True), qk_norm_eps=self.qk_norm_eps,
                           v_norm_eps=self.v_norm_eps, amplitude=getattr(enc, "amplitude", 1.0))
        o = hip.paged_attention(q, mem.k_cache, mem.v_cache, ctx, mem.space, self.scale, self.window, softcap=self.softcap,
                                sink=self.sink, sinks=self.sinks, chunk_mask=self.chunk)
        if value_enc is not None:                         # each head's sum turned back by its own position, then its gate
            gate = linear(x, self.gate, out_dtype=torch.float32) if self.head_gate else None
            hip.rotate_heads(o, o, value_enc.frequencies(), 1.0, ctx.positions, interleaved=value_enc.interleaved, back=True, gate=gate)
        return linear(o.view(ctx.num_tokens, self.num_heads * self.value_dim), self.o, out_dtype=torch.float32,
                      packed=self.o_packed)


@register("mixer", "attention_conv")
class ConvAttention(Mixer):
    """Grouped-query attention without rotation whose projected q, k and v rows first pass a short causal
    convolution over time (`conv_taps` taps per channel; the last taps - 1 projected rows of a request are
    its state), every option a constructor argument: q and k heads divided by their root mean square and
    scaled by a weight shared by all heads (`qk_norm_eps`), q multiplied by
    1 + q_temp_coef ln(floor((p + 1) / q_temp_every) + 1) at position p, a penalty on distance
    2^(-slope_exponent (h + 1) / heads) * (i - j) taken off head h's scores (`slope_exponent` None: not), a
    window, a learned per-head sink in the softmax's denominator (`sink`), and the heads' output multiplied
    by sigmoid(W_g x) before the output projection (`gate`). `own_kv` False: the mixer projects queries (and
    the gate) only and reads the cache of another run of the order. `cache_window`: how long the cache keeps
    keys where other runs read it through wider windows than this one's (None: `window`). One fused
    projection gives q | k | v | gate, 32-bit on its way out; convolution, norms, scores, weights and the
    gate are 32-bit in every storage type."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int | None = None,
                 conv_taps: int = 1, own_kv: bool = True, scale: float | None = None, window: int = 0,
                 cache_window: int | None = None, qk_norm_eps: float | None = None, q_temp_coef: float = 0.0,
                 q_temp_every: int = 1, slope_exponent: float | None = None, sink: bool = False, gate: bool = False) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not divide into {num_kv_heads} key/value heads")
        value_dim = head_dim if value_dim is None else value_dim
        if not (0 < head_dim <= 256 and 0 < value_dim <= 256):
            raise ValueError(f"head sizes {head_dim} / {value_dim}: the attention kernels take up to 256")
        if not 1 <= conv_taps <= hip.CONV_MAX_TAPS:
            raise ValueError(f"conv_taps {conv_taps}: 1 to {hip.CONV_MAX_TAPS}")
        if window < 0 or q_temp_every < 1:
            raise ValueError("window >= 0 (0: none), q_temp_every >= 1")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.conv_taps, self.own_kv = head_dim, value_dim, conv_taps, own_kv
        self.scale = scale if scale is not None else head_dim ** -0.5
        self.window = window
        self.cache_window = window if cache_window is None else cache_window
        self.qk_norm_eps, self.q_temp_coef, self.q_temp_every = qk_norm_eps, q_temp_coef, q_temp_every
        self.slope_exponent, self.has_sink, self.has_gate = slope_exponent, sink, gate
        self.proj: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.conv: torch.Tensor | None = None
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None
        self.sink: torch.Tensor | None = None
        self.slopes: torch.Tensor | None = None
        self.proj_packed: hip.StreamingCopies | None = None
        self.o_packed: hip.StreamingCopies | None = None

    @property
    def channels(self) -> int:
        """Columns of the projection that pass the convolution: q, and k and v where the mixer makes its own."""
        own = self.num_kv_heads * (self.head_dim + self.value_dim) if self.own_kv else 0
        return self.num_heads * self.head_dim + own

    @property
    def out_size(self) -> int:
        return self.num_heads * self.value_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {"proj": ParamSpec((self.channels + (self.out_size if self.has_gate else 0), self.hidden_size)),
                 "o": ParamSpec((self.hidden_size, self.out_size)),
                 "conv": ParamSpec((self.channels, self.conv_taps), "float32", init=(1.0 / self.conv_taps, 0.3))}
        if self.qk_norm_eps is not None:
            specs["q_norm"] = ParamSpec((self.head_dim,), "float32", init=(1.0, 0.1))
            if self.own_kv:
                specs["k_norm"] = ParamSpec((self.head_dim,), "float32", init=(1.0, 0.1))
        if self.has_sink:
            specs["sink"] = ParamSpec((self.num_heads,), "float32", init=(0.0, 1.0))
        return specs

    def bind(self, params) -> None:
        super().bind(params)
        if self.slope_exponent is not None:
            slopes = [2.0 ** (-self.slope_exponent * (h + 1) / self.num_heads) for h in range(self.num_heads)]
            self.slopes = torch.tensor(slopes, dtype=torch.float32).to(self.proj.device)

    def kv_spec(self) -> KVSpec:
        return KVSpec(self.num_kv_heads, self.head_dim, self.cache_window,
                      None if self.value_dim == self.head_dim else self.value_dim)

    def state_spec(self) -> StateSpec | None:
        return StateSpec((self.conv_taps - 1, self.channels), torch.float32) if self.conv_taps > 1 else None

    def keep_streaming_copies(self) -> int:
        self.proj_packed, self.o_packed = streaming_copy(self.proj), streaming_copy(self.o)
        return sum(c.nbytes() for c in (self.proj_packed, self.o_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        if self.own_kv != mem.store:
            raise ValueError("a mixer with keys and values of its own writes its cache; one without reads another's")
        proj = linear(x, self.proj, out_dtype=torch.float32, packed=self.proj_packed)
        store = (ctx.slot_mapping[mem.space], mem.k_cache, mem.v_cache) if self.own_kv else (None, None, None)
        q = hip.conv_finish(proj, self.conv, mem.state, ctx, *store, self.num_heads, self.num_kv_heads if self.own_kv else 0,
                            self.head_dim, self.value_dim, x.dtype, q_norm=self.q_norm, k_norm=self.k_norm,
                            eps=self.qk_norm_eps or 0.0, temp_coef=self.q_temp_coef, temp_every=self.q_temp_every,
                            moves_state=(fused := self.conv_taps > 1 and hip.conv_moves_state(ctx)))
        if self.conv_taps > 1 and not fused:
            hip.conv_state_update(mem.state, proj, ctx)
        o = hip.paged_attention(q, mem.k_cache, mem.v_cache, ctx, mem.space, self.scale, self.window, sinks=self.sink,
                                slopes=self.slopes, gate=proj[:, self.channels:] if self.has_gate else None)
        return linear(o.view(ctx.num_tokens, self.out_size), self.o, out_dtype=torch.float32, packed=self.o_packed)
