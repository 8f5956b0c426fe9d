"""A residual stream kept in 32-bit floats whatever the engine's storage type, with its next update
pending: what the branches of a layer have made is not added when the layer ends but when the next
consumer takes the stream, which then does the sum and its own norms in one kernel
(`hip.stream_update_norm`). A model asks for it with `ModelSpec.residual_dtype = "float32"`; blocks
that pass it on declare `keeps_stream`. What a branch has made may have to pass a norm of its own
before it is added (`post`: arrangements with a norm after every part): the consumer's kernel does
that too where both norms are of the element-by-element kind (`hip.dyt_stream`)."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip


class ResidualStream:
    """x [tokens, hidden] float32 and, pending, x += mult * (a + b + bias): `a`, `b` the outputs of a
    layer's branches (float32 or the engine's storage type; either may be None), `bias` [hidden] a
    bias that the last projection of a branch left to the sum. With `post` (a norm; then only `a` is
    pending and `mult` is 1) the pending update is x += post(a), or x += post(a) * scale with `scale`
    (float32 [hidden], a learned factor per channel; with an RMS norm as `post` only)."""

    def __init__(self, x: torch.Tensor, a: torch.Tensor | None = None, b: torch.Tensor | None = None,
                 bias: torch.Tensor | None = None, mult: float = 1.0, post=None, scale: torch.Tensor | None = None) -> None:
        if x.dtype != torch.float32:
            raise ValueError("the stream is float32")
        if post is not None and (a is None or b is not None or bias is not None or mult != 1.0):
            raise ValueError("a norm after a branch goes with that branch's rows alone")
        if scale is not None and not hasattr(post, "weight32"):
            raise ValueError("a scale per channel rides on the kernel of an RMS norm after the branch")
        self.x, self.a, self.b, self.bias, self.mult, self.post, self.scale = x, a, b, bias, mult, post, scale

    def _apply_post(self, weight: torch.Tensor | None = None, eps: float = 0.0, out_dtype: torch.dtype | None = None):
        """The branch's rows through the norm that follows them. An RMS norm's kernel (`hip.stream_post_norm`) also adds
        them to the stream, and may leave the updated rows on its way out: through a norm of their own (`weight`
        float32, `eps`) or as they are, in `out_dtype`; what it leaves comes back. Any other norm runs its own kernel,
        and the sum stays pending."""
        if self.post is None:
            return None
        if hasattr(self.post, "weight32"):
            out = hip.stream_post_norm(self.x, self.a, self.post.weight32, self.scale, self.post.eps, weight, eps, out_dtype)
            self.a = self.post = self.scale = None
            return out
        self.a, self.post = self.post(self.a)[0], None
        return None

    def rows_as(self, dtype: torch.dtype) -> "tuple[torch.Tensor, torch.Tensor]":
        """Does the pending sum and returns (x, x in `dtype`): the stream's rows as a projection's operand."""
        if dtype == torch.float32:
            return self.settle()[0], self.x
        if hasattr(self.post, "weight32"):
            return self.x, self._apply_post(out_dtype=dtype)
        raise TypeError("the stream's rows leave in another type on the way out of an RMS norm's sum")

    def take(self, norm=None, rows: torch.Tensor | None = None, out_dtype: torch.dtype = torch.float32):
        """Does the pending sum and returns (x, norm(x)) (norm(x) of the picked `rows` only if given; None
        if no norm is). Norms that work element by element (they have `elementwise()`: alpha, w, b of
        tanh(alpha x) w + b) ride in the kernel that sums; any other norm gets the settled stream."""
        fused = norm is None or hasattr(norm, "elementwise")
        if fused and (self.post is None or hasattr(self.post, "elementwise")) and self.b is None and self.bias is None \
                and self.mult == 1.0:
            post = self.post.elementwise() if self.post is not None else None
            pre = norm.elementwise() if norm is not None else None
            a, self.a, self.post = self.a, None, None
            if rows is not None:
                if a is not None:
                    hip.dyt_stream(self.x, a, post, None, out_dtype)
                return self.x, (hip.dyt(self.x, *pre, out_dtype, rows=rows)[0] if pre is not None else None)
            if a is None and pre is None:
                return self.x, None
            return self.x, hip.dyt_stream(self.x, a, post, pre, out_dtype)
        if norm is not None and not hasattr(norm, "elementwise") and hasattr(self.post, "weight32"):
            return self.x, norm(self, None, rows)[0]     # (an RMS norm after the branch: its kernel may make `norm` as well)
        self._apply_post()
        if norm is None:
            return self.settle()[0], None
        if hasattr(norm, "elementwise"):
            self.settle()
            return self.x, hip.dyt(self.x, *norm.elementwise(), out_dtype, rows=rows)[0]
        return self.x, norm(self, None, rows)[0]

    @property
    def pending(self) -> bool:
        return self.a is not None or self.b is not None

    def settle(self, weights: "tuple[torch.Tensor | None, torch.Tensor | None]" = (None, None), eps: float = 0.0,
               out_dtype: torch.dtype = torch.float32) -> "tuple[torch.Tensor, torch.Tensor | None, torch.Tensor | None]":
        """Does the pending sum; returns (x, norm(x) * weights[0], norm(x) * weights[1]) with None for a
        weight not given, the norms in `out_dtype`."""
        self._apply_post()
        a, b, bias = self.a, self.b, self.bias
        if a is None and b is not None and bias is None:
            a, b = b, None
        h1, h2 = (None, None)
        if self.pending or weights[0] is not None or weights[1] is not None:
            h1, h2 = hip.stream_update_norm(self.x, a, b, bias, self.mult, weights, eps, out_dtype=out_dtype)
        self.a = self.b = self.bias = None
        return self.x, h1, h2

    def norm_rows(self, rows: torch.Tensor | None, weight: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
        """norm(x) * weight of the rows picked (all of them if `rows` is None), after the pending sum."""
        if rows is None and hasattr(self.post, "weight32") and weight.dtype == torch.float32:
            return self._apply_post(weight, eps, out_dtype)      # the sum and this norm in the kernel of the norm before
        self._apply_post()
        if rows is None:
            return self.settle((weight, None), eps, out_dtype)[1]
        self.settle()
        return hip.stream_update_norm(self.x, weights=(weight, None), eps=eps, rows=rows, out_dtype=out_dtype)[0]
