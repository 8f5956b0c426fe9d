"""The two ends of a model: the table that turns token ids into hidden rows, and the projection
that turns the final rows into logits (tinyserve_llm/model/llama.py:262-268,293-304: an embedding
module, and a head that is the embedding's weight when the checkpoint ties them). Another
architecture that scales its embeddings or caps its logits registers parts of its own under
"embedding" and "head"."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import Embedding, Head, ParamSpec, PartSpec, StepContext, make, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy
from tinyserve_llm_amd.parts.stream import ResidualStream


@register("embedding", "table")
class TableEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, init: tuple[float, float] = (0.0, 0.02),
                 float32_stream: bool = False, scale: float = 1.0, norm: "PartSpec | None" = None, side_width: int = 0,
                 side_init: tuple[float, float] = (0.0, 1.0)) -> None:
        """`float32_stream`: the rows start a residual stream that is kept in 32-bit floats
        (`parts.stream.ResidualStream`) whatever the table's storage type; such rows may be multiplied
        by `scale` and passed through a norm that works element by element (`norm`: its PartSpec; its
        parameters are the table's, named `norm_<name>`). `side_width` > 0: a second table `side` [vocab, side_width] of
        per-token rows that the layers' token inputs read stretches of (`parts.base.TokenInput`)."""
        self.side_width, self.side_init = side_width, tuple(side_init)
        self.side: torch.Tensor | None = None
        self.vocab_size, self.hidden_size, self.init = vocab_size, hidden_size, tuple(init)
        self.float32_stream, self.scale = float32_stream, scale
        if (scale != 1.0 or norm is not None) and not float32_stream:
            raise ValueError("a scaled or normalised embedding starts a 32-bit stream (float32_stream=True)")
        self.norm = make("norm", norm) if norm is not None else None
        if self.norm is not None and not hasattr(self.norm, "elementwise"):
            raise ValueError(f"the embedding takes a norm that works element by element, not {norm.kind!r}")
        self.weight: torch.Tensor | None = None

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {"weight": ParamSpec((self.vocab_size, self.hidden_size), init=self.init)}
        if self.side_width:
            specs["side"] = ParamSpec((self.vocab_size, self.side_width), init=self.side_init)
        if self.norm is not None:
            specs.update({f"norm_{name}": ps for name, ps in self.norm.param_specs().items()})
        return specs

    def bind(self, params) -> None:
        super().bind({n: t for n, t in params.items() if not n.startswith("norm_")})
        if self.norm is not None:
            self.norm.bind({n[len("norm_"):]: t for n, t in params.items() if n.startswith("norm_")})

    def table(self) -> torch.Tensor | None:
        return self.weight

    def side_table(self) -> torch.Tensor | None:
        return self.side

    def forward(self, ctx: StepContext) -> "torch.Tensor | ResidualStream":
        if self.float32_stream and (self.scale != 1.0 or self.norm is not None):
            return ResidualStream(hip.embedding_dyt_stream(self.weight, ctx.token_ids, self.scale,
                                                           self.norm.elementwise() if self.norm is not None else None))
        if self.float32_stream:
            return ResidualStream(hip.embedding_stream(self.weight, ctx.token_ids))
        return hip.embedding(self.weight, ctx.token_ids)      # (ids are checked against the vocabulary on the host)


@register("head", "projection")
class ProjectionHead(Head):
    """float32 logits = rows · Wᵀ with W [vocab, hidden], its own or the embedding's."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, init: tuple[float, float] = (0.0, 0.02)) -> None:
        self.vocab_size, self.hidden_size, self.tied, self.init = vocab_size, hidden_size, tied, tuple(init)
        self.weight: torch.Tensor | None = None
        self.weight_packed = None                # `streaming_copy` of the weight, if the model keeps them

    def param_specs(self) -> dict[str, ParamSpec]:
        return {} if self.tied else {"weight": ParamSpec((self.vocab_size, self.hidden_size), init=self.init)}

    def tie(self, table: torch.Tensor) -> None:
        if table is None or tuple(table.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"a tied head needs the embedding's [{self.vocab_size}, {self.hidden_size}] table")
        self.weight = table

    def keep_streaming_copies(self) -> int:
        # (a step reads the whole vocabulary matrix once whatever its size: at the 1B sizes a fifth of a decode step's bytes)
        self.weight_packed = streaming_copy(self.weight)
        return 0 if self.weight_packed is None else self.weight_packed.nbytes()

    def forward(self, rows: torch.Tensor) -> torch.Tensor:
        return linear(rows, self.weight, out_dtype=torch.float32, packed=self.weight_packed)
