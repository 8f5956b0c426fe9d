"""The Bafarax decoder as a ModelSpec. Token rows times a scale start a 32-bit residual stream; every layer is
x <- x + mixer(n1 x), x <- x + ff(n2 x) with RMS norms whose weights are stored around zero (n(x) = rms(x) (1 + w));
the mixer is, layer by layer, grouped-query attention inside chunks of positions with a norm over the whole q and
the whole k projection, rotate-half positions and a learned sink (`parts.attention.GeneralAttention`), attention
through a low-rank latent with a sliding window and an output gate (`parts.latent.LatentAttention`), or an mLSTM's
matrix memory (`parts.mlstm.MLSTM`); the feed-forward is a silu-gated unit, a mixture of ungated experts with a
squared relu, or absent. A layer may run with an earlier layer's weights: it is then a second run of that layer in
the order, with a cache or state of its own. Checkpoint names: `embed`, `l<i>.norm{1,2}`,
`l<i>.mix.{q,k,v,o,q.norm,k.norm,sink}` or `l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,g,o}` or
`l<i>.mix.{q,k,v,i,i.b,f,f.b,g,norm,o}`, `l<i>.mlp.{gate,up,down}` or `l<i>.mlp.router`, `l<i>.mlp.e<j>.{up,down}`,
`final.norm`, `head`."""

from __future__ import annotations

from tinyserve_llm_amd.config.bafarax import (BafaraxAttention, BafaraxConfig, BafaraxDense, BafaraxExperts,
                                              BafaraxLatentAttention, BafaraxMLSTM, Rotation)
from tinyserve_llm_amd.models.registry import Architecture, register_architecture
from tinyserve_llm_amd.models.spec import Destination, LayerRun, LayerSpec, ModelSpec
from tinyserve_llm_amd.parts.base import PartSpec


def _encoding(encodings: dict[str, PartSpec], rot: Rotation, interleaved: bool) -> str | None:
    """The name of the position encoding for a rotation (one per distinct set of constants), made if new."""
    if not rot.dims:
        return None
    ramp = None if rot.ramp is None else dict(factor=rot.ramp.factor, original=rot.ramp.original, fast=rot.ramp.fast,
                                              slow=rot.ramp.slow)
    name = f"rotary_{rot.dims}_{rot.base!r}_{'pairs' if interleaved else 'halves'}" + \
        ("" if ramp is None else "_ramp_" + "_".join(repr(v) for v in ramp.values()))
    encodings.setdefault(name, PartSpec("rotary_frequencies", dict(rotary_dim=rot.dims, theta=rot.base, interleaved=interleaved,
                                                                   ramp=ramp)))
    return name


def bafarax_spec(config: BafaraxConfig) -> ModelSpec:
    c = config
    norm = PartSpec("rmsnorm", dict(hidden_size=c.width, eps=c.norm_eps, one_plus=True))
    ckpt: dict[str, Destination] = {"embed": Destination("embed.weight"), "final.norm": Destination("final_norm.weight"),
                                    "head": Destination("head.weight")}
    encodings: dict[str, PartSpec] = {}
    layers: list[LayerSpec] = []
    index_of: dict[int, int] = {}            # layer of the configuration -> its place among the layers with weights
    order: list[LayerRun] = []
    for i, layer in enumerate(c.layers):
        if layer.weights_of is not None:
            order.append(LayerRun(index_of[layer.weights_of]))
            continue
        src, dst, m = f"l{i}", f"layers.{len(layers)}", layer.mixer
        index_of[i] = len(layers)
        order.append(LayerRun(len(layers)))
        ckpt[f"{src}.norm1"] = Destination(f"{dst}.norm1.weight")
        if isinstance(m, BafaraxAttention):
            mixer = PartSpec("attention_general", dict(
                hidden_size=c.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                position=_encoding(encodings, m.rot, interleaved=False), scale=m.scale, chunk=m.chunk, learned_sink=True,
                projection_norm_eps=c.norm_eps))
            q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            ckpt[f"{src}.mix.q"] = Destination(f"{dst}.mixer.qkv", 0, q)
            ckpt[f"{src}.mix.k"] = Destination(f"{dst}.mixer.qkv", q, k)
            ckpt[f"{src}.mix.v"] = Destination(f"{dst}.mixer.qkv", q + k, v)
            ckpt[f"{src}.mix.q.norm"] = Destination(f"{dst}.mixer.q_norm")
            ckpt[f"{src}.mix.k.norm"] = Destination(f"{dst}.mixer.k_norm")
            ckpt[f"{src}.mix.sink"] = Destination(f"{dst}.mixer.sinks")
        elif isinstance(m, BafaraxLatentAttention):
            mixer = PartSpec("latent_attention", dict(
                hidden_size=c.width, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim, kv_rank=m.kv_rank,
                q_rank=m.q_rank, position=_encoding(encodings, m.rot, interleaved=True), scale=m.scale, norm_eps=c.norm_eps,
                window=m.window, gate=True))
            row = m.kv_rank + m.rot_dim
            ckpt[f"{src}.mix.dq"] = Destination(f"{dst}.mixer.down", 0, m.q_rank)
            ckpt[f"{src}.mix.dkv"] = Destination(f"{dst}.mixer.down", m.q_rank, row)
            ckpt[f"{src}.mix.g"] = Destination(f"{dst}.mixer.down", m.q_rank + row, m.heads * m.vdim)
            ckpt[f"{src}.mix.dq.norm"] = Destination(f"{dst}.mixer.q_norm")
            ckpt[f"{src}.mix.dkv.norm"] = Destination(f"{dst}.mixer.kv_norm")
            for name in ("uq", "uk", "uv"):
                ckpt[f"{src}.mix.{name}"] = Destination(f"{dst}.mixer.{name}")
        else:
            assert isinstance(m, BafaraxMLSTM)
            mixer = PartSpec("mlstm", dict(hidden_size=c.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                                           gate_cap=m.gate_cap, norm_eps=c.norm_eps))
            qk, v, at = m.heads * m.dim, m.heads * m.vdim, 0
            for name, rows in (("q", qk), ("k", qk), ("v", v), ("i", m.heads), ("f", m.heads), ("g", v)):
                ckpt[f"{src}.mix.{name}"] = Destination(f"{dst}.mixer.proj", at, rows)
                at += rows
            ckpt[f"{src}.mix.i.b"] = Destination(f"{dst}.mixer.gate_bias", 0, m.heads)
            ckpt[f"{src}.mix.f.b"] = Destination(f"{dst}.mixer.gate_bias", m.heads, m.heads)
            ckpt[f"{src}.mix.norm"] = Destination(f"{dst}.mixer.norm")
        ckpt[f"{src}.mix.o"] = Destination(f"{dst}.mixer.o")
        norms = {"norm1": norm}
        if layer.mlp is None:
            ff = PartSpec("none")
        else:
            norms["norm2"] = norm
            ckpt[f"{src}.norm2"] = Destination(f"{dst}.norm2.weight")
            if isinstance(layer.mlp, BafaraxDense):
                # silu(g) u is the capped unit g sigmoid(slope g) (u + shift) without a cap, slope 1, shift 0
                ff = PartSpec("capped_glu", dict(hidden_size=c.width, intermediate_size=layer.mlp.ff, limit=0.0, slope=1.0, up_shift=0.0))
                ckpt[f"{src}.mlp.gate"] = Destination(f"{dst}.ff.gate_up", 0, layer.mlp.ff)
                ckpt[f"{src}.mlp.up"] = Destination(f"{dst}.ff.gate_up", layer.mlp.ff, layer.mlp.ff)
                ckpt[f"{src}.mlp.down"] = Destination(f"{dst}.ff.down")
            else:
                e: BafaraxExperts = layer.mlp
                ff = PartSpec("routed_dense_experts", dict(hidden_size=c.width, num_experts=e.experts, top=e.top, intermediate_size=e.ff,
                                                           activation="relu2", scoring="softmax_chosen"))
                ckpt[f"{src}.mlp.router"] = Destination(f"{dst}.ff.router")
                for j in range(e.experts):
                    ckpt[f"{src}.mlp.e{j}.up"] = Destination(f"{dst}.ff.up", index=(j,))
                    ckpt[f"{src}.mlp.e{j}.down"] = Destination(f"{dst}.ff.down", index=(j,))
        layers.append(LayerSpec(mixer, ff, norms, "pre_norm_stream"))
    table = PartSpec("table", dict(vocab_size=c.vocab, hidden_size=c.width, float32_stream=True, scale=c.embedding_scale,
                                   init=(0.0, 1.0 / max(c.embedding_scale, 1e-6))))
    return ModelSpec(
        architecture=c.architecture, vocab_size=c.vocab, hidden_size=c.width, max_position=None, layers=layers, order=order,
        final_norm=norm, position_encodings=encodings, tie_word_embeddings=False, residual_dtype="float32", embedding=table,
        checkpoint=ckpt)


BAFARAX = register_architecture(Architecture(
    name="Bafarax", model_types=("bafarax",), config_from_dict=BafaraxConfig.from_dict, build_spec=bafarax_spec,
    config_to_dict=BafaraxConfig.to_dict))
