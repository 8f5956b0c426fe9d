"""The Tegolix decoder as a ModelSpec. Token rows start a 32-bit residual stream; every layer is
x <- x + s1 * n1b(mixer(n1 x)), x <- x + s2 * n2b(ff(n2 x)) with RMS norms whose weights are stored around zero
(n(x) = rms(x) (1 + w)) and learned scales per channel, and then takes a per-layer token input: a stretch of the token's
row of a second, narrow table, gated by gelu(W_gate x), projected to the width and added through an RMS norm with a plain
weight (`parts.token_input.GatedTokenRows`). The mixer is, layer by layer, gated linear attention
(`parts.linear_attention.GatedLinearAttention`) or two mixers side by side (`parts.side_by_side.SideBySide`): grouped-query
attention in a sliding window with capped scores, a weighted norm on every q and k head, rotate-half positions with a
frequency ramp, values that turn with their position and a gate per head (`parts.attention.GeneralAttention`), beside an
RWKV-style recurrence with token shift (`parts.linear_attention.ShiftedDecayRecurrence`). The feed-forward is a relu-gated
unit, a mixture of silu-gated experts scored by a softmax over all router outputs, of which the last ones stand for
identity experts, with a shared expert behind a sigmoid gate of its own, or absent. Checkpoint names: `embed`, `side.embed`,
`l<i>.{norm1,norm1b,norm2,norm2b,ls1,ls2}`, `l<i>.side.{gate,proj,norm}`, `l<i>.mix.{q,k,v,g,o,norm,a1,a2,a2.b}` or
`l<i>.mix.left.{q,k,v,q.norm,k.norm,g,o}` with `l<i>.mix.right.{mu.r,mu.k,mu.v,mu.g,mu.w,r,k,v,g,w1,w2,w0,u,norm,o}`,
`l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{router,correction,shared.{gate,up,down,sg}}`, `l<i>.mlp.e<j>.{gate,up,down}`,
`final.norm`, `head`."""

from __future__ import annotations

from tinyserve_llm_amd.config.tegolix import TegolixConfig, TegolixDense, TegolixExperts, TegolixGLA, TegolixParallel
from tinyserve_llm_amd.models.bafarax import _encoding
from tinyserve_llm_amd.models.fanotar import _unit_names
from tinyserve_llm_amd.models.registry import Architecture, register_architecture
from tinyserve_llm_amd.models.spec import Destination, LayerRun, LayerSpec, ModelSpec
from tinyserve_llm_amd.parts.base import PartSpec
from tinyserve_llm_amd.parts.linear_attention import SHIFT_MIXES

SILU_UNIT = dict(limit=0.0, slope=1.0, up_shift=0.0)      # g sigmoid(g) u: the capped unit without a cap, slope 1, shift 0


def tegolix_spec(config: TegolixConfig) -> ModelSpec:
    c = config
    norm = PartSpec("rmsnorm", dict(hidden_size=c.width, eps=c.norm_eps, one_plus=True))
    scale = PartSpec("channel_scale", dict(hidden_size=c.width))
    ckpt: dict[str, Destination] = {"embed": Destination("embed.weight"), "final.norm": Destination("final_norm.weight"),
                                    "head": Destination("head.weight")}
    if c.side_dim:
        ckpt["side.embed"] = Destination("embed.side")
    encodings: dict[str, PartSpec] = {}
    layers: list[LayerSpec] = []
    for i, layer in enumerate(c.layers):
        src, dst, m = f"l{i}", f"layers.{i}", layer.mixer
        if isinstance(m, TegolixGLA):
            mixer = PartSpec("gated_linear_attention", dict(hidden_size=c.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                                                            decay_rank=m.decay_rank, tau=m.tau, norm_eps=c.norm_eps))
            k, v, at = m.heads * m.dim, m.heads * m.vdim, 0
            for name, rows in (("q", k), ("k", k), ("v", v), ("g", v)):
                ckpt[f"{src}.mix.{name}"] = Destination(f"{dst}.mixer.proj", at, rows)
                at += rows
            for name, param in (("a1", "decay_down"), ("a2", "decay_up"), ("a2.b", "decay_bias"), ("norm", "norm"), ("o", "o")):
                ckpt[f"{src}.mix.{name}"] = Destination(f"{dst}.mixer.{param}")
        else:
            assert isinstance(m, TegolixParallel)
            a, r = m.left, m.right
            from tinyserve_llm_amd.config.bafarax import Rotation
            left = PartSpec("attention_general", dict(
                hidden_size=c.width, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, value_dim=a.vdim,
                position=_encoding(encodings, a.rot, interleaved=False), scale=a.scale, softcap=a.softcap, window=a.window,
                head_norm_eps=c.norm_eps, value_position=_encoding(encodings, Rotation(a.vdim, a.rot.base), interleaved=False),
                head_gate=True))
            right = PartSpec("shifted_decay_recurrence", dict(hidden_size=c.width, num_heads=r.heads, head_dim=r.dim,
                                                              decay_rank=r.decay_rank, norm_eps=c.norm_eps))
            mixer = PartSpec("side_by_side", dict(left=left, right=right, left_scale=m.left_scale, right_scale=m.right_scale))
            q, k, v = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
            ckpt[f"{src}.mix.left.q"] = Destination(f"{dst}.mixer.left_qkv", 0, q)
            ckpt[f"{src}.mix.left.k"] = Destination(f"{dst}.mixer.left_qkv", q, k)
            ckpt[f"{src}.mix.left.v"] = Destination(f"{dst}.mixer.left_qkv", q + k, v)
            for name, param in (("q.norm", "q_norm"), ("k.norm", "k_norm"), ("g", "gate"), ("o", "o")):
                ckpt[f"{src}.mix.left.{name}"] = Destination(f"{dst}.mixer.left_{param}")
            for j, s in enumerate(SHIFT_MIXES):
                ckpt[f"{src}.mix.right.mu.{s}"] = Destination(f"{dst}.mixer.right_mu", index=(j,))
            for name, param in (("r", "r"), ("k", "k"), ("v", "v"), ("g", "g"), ("w1", "decay_down"), ("w2", "decay_up"),
                                ("w0", "decay_bias"), ("u", "bonus"), ("norm", "norm"), ("o", "o")):
                ckpt[f"{src}.mix.right.{name}"] = Destination(f"{dst}.mixer.right_{param}")
        norms = {"norm1": norm, "norm1b": norm, "scale1": scale}
        for name, param in (("norm1", "norm1"), ("norm1b", "norm1b"), ("ls1", "scale1")):
            ckpt[f"{src}.{name}"] = Destination(f"{dst}.{param}.weight")
        if layer.mlp is None:
            ff = PartSpec("none")
        else:
            norms.update(norm2=norm, norm2b=norm, scale2=scale)
            for name, param in (("norm2", "norm2"), ("norm2b", "norm2b"), ("ls2", "scale2")):
                ckpt[f"{src}.{name}"] = Destination(f"{dst}.{param}.weight")
            if isinstance(layer.mlp, TegolixDense):
                ff = PartSpec("capped_glu", dict(hidden_size=c.width, intermediate_size=layer.mlp.ff, limit=0.0, up_shift=0.0, activation="relu"))
                _unit_names(ckpt, f"{src}.mlp", f"{dst}.ff.", layer.mlp.ff)
            else:
                e: TegolixExperts = layer.mlp
                shared = dict(intermediate_size=e.shared_ff, **SILU_UNIT) if e.shared_ff else None
                ff = PartSpec("routed_experts", dict(
                    hidden_size=c.width, num_experts=e.experts, top=e.top, intermediate_size=e.ff, router_scale=1.0, normalize=False,
                    correction=True, shared=shared, scoring="softmax_all", identity=e.identity, shared_gate=shared is not None, **SILU_UNIT))
                ckpt[f"{src}.mlp.router"] = Destination(f"{dst}.ff.router", 0, e.experts + e.identity)
                ckpt[f"{src}.mlp.correction"] = Destination(f"{dst}.ff.correction")
                for j in range(e.experts):
                    _unit_names(ckpt, f"{src}.mlp.e{j}", f"{dst}.ff.", e.ff, index=(j,))
                if shared is not None:
                    _unit_names(ckpt, f"{src}.mlp.shared", f"{dst}.ff.shared_", e.shared_ff)
                    ckpt[f"{src}.mlp.shared.sg"] = Destination(f"{dst}.ff.router", e.experts + e.identity, 1)
        inputs = {}
        if c.side_dim:
            inputs["side"] = PartSpec("gated_token_rows", dict(hidden_size=c.width, dim=c.side_dim, offset=i * c.side_dim, eps=c.norm_eps))
            for name in ("gate", "proj", "norm"):
                ckpt[f"{src}.side.{name}"] = Destination(f"{dst}.side.{name}")
        layers.append(LayerSpec(mixer, ff, norms, "sandwich_scaled", token_inputs=inputs))
    table = PartSpec("table", dict(vocab_size=c.vocab, hidden_size=c.width, float32_stream=True, init=(0.0, 1.0),
                                   side_width=len(c.layers) * c.side_dim))
    return ModelSpec(
        architecture=c.architecture, vocab_size=c.vocab, hidden_size=c.width, max_position=None, layers=layers,
        order=[LayerRun(i) for i in range(len(layers))], final_norm=norm, position_encodings=encodings, tie_word_embeddings=False,
        residual_dtype="float32", embedding=table, checkpoint=ckpt)


TEGOLIX = register_architecture(Architecture(
    name="Tegolix", model_types=("tegolix",), config_from_dict=TegolixConfig.from_dict, build_spec=tegolix_spec,
    config_to_dict=TegolixConfig.to_dict, sizes_from_checkpoint=TegolixConfig.ranks_from))
