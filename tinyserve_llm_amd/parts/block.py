"""Arrangements of a layer's parts. "pre_norm" is the Llama block with the residual add deferred
into the next norm (tinyserve_llm/model/llama.py:238-253): a layer returns (feed-forward output,
residual) without adding them; the following norm adds. It equals h += mixer(norm(h));
h += feed_forward(norm(h)).

Norms travel between parts in two directions. Forward: a norm hands its input, deferred, to the
part after it, whose first projection fuses it (`Norm.defer`, `takes_deferred_norm`). Backward: a
norm asks the part before it to finish into it (`Norm.request`, `finishes_into_norm`): that part's
last projection then leaves the residual sum and half of the norm, and what the part returns is the
norm deferred, for the part after it. Between layers the model does the asking: it tells a block
which norm the next block starts with (`following=`), and a block that `starts_with` a norm accepts
that norm, deferred, as its `hidden` (with `residual` None: the sum is inside)."""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from tinyserve_llm_amd.parts.base import FeedForward, LayerMemory, Mixer, Norm, StepContext, register


@dataclass
class Layer:
    mixer: Mixer
    feed_forward: FeedForward
    norms: dict[str, Norm]           # by the names the arrangement uses
    block: str = "pre_norm"
    block_args: dict = field(default_factory=dict)      # the arrangement's own constants (a residual multiplier, say)
    token_inputs: dict = field(default_factory=dict)    # parts that add something made from the token ids, by name

    def parts(self) -> dict[str, object]:
        """Every part by the name its parameters are known under (`layers.<i>.<name>.<parameter>`)."""
        if {"mixer", "ff"} & (set(self.norms) | set(self.token_inputs)) or set(self.norms) & set(self.token_inputs):
            raise ValueError("norms and token inputs have names of their own, other than 'mixer' and 'ff'")
        return {"mixer": self.mixer, "ff": self.feed_forward, **self.norms, **self.token_inputs}


def uses_norms(*names: str):
    """Declares the norms an arrangement looks up in `layer.norms`, so that a layer that lacks one
    is refused when the model is built, not at its first step."""
    def mark(fn):
        fn.norm_names = names
        return fn
    return mark


def starts_with(name: str):
    """Declares that an arrangement applies the norm of this name to (hidden, residual) before
    anything else, takes `following=` (the norm the next arrangement starts with, or None), and
    accepts its own first norm in deferred form as `hidden`."""
    def mark(fn):
        fn.first_norm = name
        return fn
    return mark


def first_norm_of(layer: Layer) -> Norm | None:
    """The norm a layer's arrangement starts with, if it says so (`starts_with`)."""
    from tinyserve_llm_amd.parts.base import BLOCKS
    name = getattr(BLOCKS[layer.block], "first_norm", None)
    return layer.norms[name] if name else None


def _through(part, norm: Norm, x, residual, run, following: Norm | None):
    """One branch of a pre-norm arrangement: `norm` applied to (x, residual), then `part` (`run` calls
    its forward). `x` may be `norm` itself in deferred form (then `residual` is None). The norm is
    handed to the part deferred if the part takes it so; the part is asked to finish into
    `following` if it can and that norm takes requests. Returns (the part's output or `following`
    deferred, the residual stream after `norm`'s sum)."""
    pending = x if norm.made_for(x) else None
    if pending is None and part.takes_deferred_norm:
        pending = norm.defer(x, residual)
    if pending is not None and not part.takes_deferred_norm:
        x, residual, pending = pending.materialize(), pending.residual_out, None
    elif pending is None:
        x, residual = norm(x, residual)
    # the stream after this norm's sum: known now, or once the part's first projection has run
    request = following.request(pending if pending is not None else residual) \
        if following is not None and part.finishes_into_norm else None
    out = run(pending if pending is not None else x, request) if request is not None else run(pending if pending is not None else x)
    if pending is not None:
        residual = pending.residual_out
    return out, residual


@register("block", "pre_norm")
@uses_norms("mixer_norm", "ff_norm")
@starts_with("mixer_norm")
def pre_norm_block(layer: Layer, hidden, residual: torch.Tensor | None, ctx: StepContext, mem: LayerMemory,
                   following: Norm | None = None) -> tuple[torch.Tensor, torch.Tensor | None]:
    mixer_norm, ff_norm = layer.norms["mixer_norm"], layer.norms["ff_norm"]
    x, residual = _through(layer.mixer, mixer_norm, hidden, residual,
                           lambda x, then=None: layer.mixer.forward(x, ctx, mem, **({"then": then} if then else {})), ff_norm)
    if ff_norm.made_for(x):
        residual = None                      # the sum is inside the deferred norm
    x, residual = _through(layer.feed_forward, ff_norm, x, residual,
                           lambda x, then=None: layer.feed_forward.forward(x, ctx, **({"then": then} if then else {})), following)
    if following is not None and following.made_for(x):
        residual = None
    return x, residual


def keeps_stream(fn):
    """Declares that an arrangement takes a `parts.stream.ResidualStream` as `hidden` (with `residual`
    None) and returns one: a model whose residual stream is 32-bit is made of such arrangements."""
    fn.keeps_stream = True
    return fn


@register("block", "parallel")
@uses_norms("norm1")
@keeps_stream
def parallel_block(layer: Layer, hidden, residual, ctx: StepContext, mem: LayerMemory):
    """x <- x + mult * (mixer(norm1(x)) + feed_forward(norm2(x))): both branches read the same x, each
    through a norm of its own ("norm1", "norm2"; a layer whose feed-forward is "none" needs no
    "norm2"); `mult` is the layer's `block_args["residual_mult"]` (1 if not given). The stream is 32-bit. The sum is left pending in the stream that comes back, so that the next layer's
    two norms (or the final norm) are made by the kernel that adds it; the two norms of a layer share
    one mean square."""
    from tinyserve_llm_amd.parts.stream import ResidualStream
    if not isinstance(hidden, ResidualStream) or residual is not None:
        raise TypeError("the parallel arrangement runs on a 32-bit residual stream (ModelSpec.residual_dtype = 'float32')")
    norm1, norm2 = layer.norms["norm1"], layer.norms.get("norm2")
    if norm2 is not None and norm1.eps != norm2.eps:
        raise ValueError("the two norms of a parallel layer share their mean square, so also their eps")
    x, h1, h2 = hidden.settle((norm1.weight, None if norm2 is None else norm2.weight), norm1.eps, norm1.weight.dtype)
    a = layer.mixer.forward(h1, ctx, mem)
    ff = layer.feed_forward
    if norm2 is None:
        b, bias = ff.forward(None, ctx), None          # (only a part that reads nothing can do without its norm)
    elif getattr(ff, "can_defer_bias", False):
        b, bias = ff.forward(h2, ctx, defer_bias=True)
    else:
        b, bias = ff.forward(h2, ctx), None
    return ResidualStream(x, a, b, bias, float(layer.block_args.get("residual_mult", 1.0))), None


@register("block", "sandwich")
@uses_norms("norm1", "norm1b")
@keeps_stream
def sandwich_block(layer: Layer, hidden, residual, ctx: StepContext, mem: LayerMemory):
    """x <- x + norm1b(mixer(norm1(x))), then x <- x + norm2b(feed_forward(norm2(x))): a norm before and
    one after every part ("norm2", "norm2b" only where the layer has a feed-forward). The stream is
    32-bit; each sum is left pending in it, with the norm that the branch's rows still have to pass, so
    that whoever takes the stream next does both norms and the sum in one kernel."""
    from tinyserve_llm_amd.parts.stream import ResidualStream
    if not isinstance(hidden, ResidualStream) or residual is not None:
        raise TypeError("the sandwich arrangement runs on a 32-bit residual stream (ModelSpec.residual_dtype = 'float32')")
    norms = layer.norms
    x, h = hidden.take(norms["norm1"], out_dtype=norms["norm1"].weight.dtype)
    stream = ResidualStream(x, layer.mixer.forward(h, ctx, mem), post=norms["norm1b"])
    if "norm2" not in norms:
        if layer.feed_forward.forward(None, ctx) is not None:
            raise KeyError("a sandwich layer with a feed-forward names the norms 'norm2' and 'norm2b'")
        return stream, None
    x, h = stream.take(norms["norm2"], out_dtype=norms["norm2"].weight.dtype)
    return ResidualStream(x, layer.feed_forward.forward(h, ctx), post=norms["norm2b"]), None


@register("block", "pre_norm_stream")
@uses_norms("norm1")
@keeps_stream
def pre_norm_stream_block(layer: Layer, hidden, residual, ctx: StepContext, mem: LayerMemory):
    """x <- x + mixer(norm1(x)), then x <- x + feed_forward(norm2(x)) on a 32-bit residual stream ("norm2" only where
    the layer has a feed-forward). Each sum is left pending in the stream, so that the norm that reads the stream
    next (this layer's second, the next layer's first, or the model's last) is made by the kernel that adds."""
    from tinyserve_llm_amd.parts.stream import ResidualStream
    if not isinstance(hidden, ResidualStream) or residual is not None:
        raise TypeError("this arrangement runs on a 32-bit residual stream (ModelSpec.residual_dtype = 'float32')")
    norms = layer.norms
    x, h = hidden.take(norms["norm1"])
    stream = ResidualStream(x, layer.mixer.forward(h, ctx, mem))
    if "norm2" not in norms:
        if layer.feed_forward.forward(None, ctx) is not None:
            raise KeyError("a layer with a feed-forward names the norm 'norm2'")
        return stream, None
    x, h = stream.take(norms["norm2"])
    return ResidualStream(x, layer.feed_forward.forward(h, ctx)), None


@register("block", "sandwich_scaled")
@uses_norms("norm1", "norm1b", "scale1")
@keeps_stream
def sandwich_scaled_block(layer: Layer, hidden, residual, ctx: StepContext, mem: LayerMemory):
    """x <- x + s1 * norm1b(mixer(norm1(x))), then x <- x + s2 * norm2b(feed_forward(norm2(x))) with RMS norms and learned
    scales per channel ("scale1", "scale2": `parts.norm.ChannelScale`; "norm2", "norm2b", "scale2" only where the layer
    has a feed-forward), then, for every token input of the layer in turn, x <- x + post(input(x, tokens)). The stream is
    32-bit; each sum is left pending in it with the norm and the scale that the branch's rows still have to pass, so that
    whoever takes the stream next does that norm, the sum and its own norm in one kernel."""
    from tinyserve_llm_amd.parts.stream import ResidualStream
    if not isinstance(hidden, ResidualStream) or residual is not None:
        raise TypeError("this arrangement runs on a 32-bit residual stream (ModelSpec.residual_dtype = 'float32')")
    norms = layer.norms
    x, h = hidden.take(norms["norm1"])
    stream = ResidualStream(x, layer.mixer.forward(h, ctx, mem), post=norms["norm1b"], scale=norms["scale1"].weight32)
    if "norm2" in norms:
        x, h = stream.take(norms["norm2"])
        stream = ResidualStream(x, layer.feed_forward.forward(h, ctx), post=norms["norm2b"], scale=norms["scale2"].weight32)
    elif layer.feed_forward.forward(None, ctx) is not None:
        raise KeyError("a layer with a feed-forward names the norms 'norm2', 'norm2b' and 'scale2'")
    for part in layer.token_inputs.values():
        x, rows = stream.rows_as(part.operand_dtype)
        stream = ResidualStream(x, part.forward(rows, ctx), post=part.post)
    return stream, None
