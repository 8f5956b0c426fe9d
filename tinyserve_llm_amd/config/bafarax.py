"""Typed configuration of the Bafarax decoder, read from the keys of its config.json: a scale on the
embedding, one eps for every norm, and a list of layers. A layer names its mixer's kind ("attention":
grouped-query attention inside chunks of positions with a learned sink; "latent_attention": attention
through a low-rank latent with a sliding window and an output gate; "mlstm": a matrix memory) with the
mixer's sizes and constants, an optional feed-forward (dense, or a mixture of experts), and optionally
an earlier layer whose weights it runs with (`weights_of`), keeping a cache or state of its own. Every
size and constant of a model stands here and nowhere else."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from tinyserve_llm_amd.config.llama import ConfigError


def _need(raw: Mapping[str, Any], key: str, where: str) -> Any:
    if not isinstance(raw, Mapping) or key not in raw or raw[key] is None:
        raise ConfigError(f"config.json lacks the required key {key!r} in {where}")
    return raw[key]


@dataclass(frozen=True)
class FrequencyRamp:
    """Slows the rotation's frequencies down by `factor` along a ramp between the pairs that make `fast`
    and `slow` turns over `original` positions."""
    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FrequencyRamp":
        c = cls(*(float(_need(raw, k, where)) for k in ("factor", "original", "fast", "slow")))
        if min(c.factor, c.original, c.fast, c.slow) <= 0:
            raise ConfigError(f"{where}: factor, original, fast and slow are positive")
        return c

    def to_dict(self) -> dict[str, Any]:
        original = int(self.original) if self.original == int(self.original) else self.original
        return {"factor": self.factor, "fast": self.fast, "original": original, "slow": self.slow}


@dataclass(frozen=True)
class Rotation:
    dims: int                    # leading dimensions of a head (or of its rotated part) that turn; 0: none
    base: float
    ramp: FrequencyRamp | None = None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any] | None, where: str) -> "Rotation":
        if not raw:
            return cls(0, 1.0)
        scaling = raw.get("scaling")
        c = cls(dims=int(_need(raw, "dims", where)), base=float(_need(raw, "base", where)),
                ramp=FrequencyRamp.from_dict(scaling, where + ".scaling") if scaling else None)
        if c.dims < 0 or c.dims % 2 or (c.dims and c.base <= 0) or (c.ramp is not None and c.base <= 1):
            raise ConfigError(f"{where}: an even number of dims, a positive base (above 1 with scaling)")
        return c

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.ramp is not None:
            out["scaling"] = self.ramp.to_dict()
        return out


def _mask_size(raw: Mapping[str, Any], where: str) -> int:
    mask = raw.get("mask")
    if not mask:
        return 0
    size = int(_need(mask, "size", where + ".mask"))
    if size < 1:
        raise ConfigError(f"{where}.mask.size {size}: a positive number of positions")
    return size


@dataclass(frozen=True)
class BafaraxAttention:
    heads: int
    kv_heads: int
    dim: int                     # size of a query / key head
    vdim: int                    # size of a value head
    scale: float
    rot: Rotation                # pairs (i, i + dims/2)
    chunk: int                   # a position sees the keys of its own chunk of this many positions (0: all before it)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "BafaraxAttention":
        c = cls(heads=int(_need(raw, "heads", where)), kv_heads=int(_need(raw, "kv_heads", where)),
                dim=int(_need(raw, "dim", where)), vdim=int(_need(raw, "vdim", where)), scale=float(_need(raw, "scale", where)),
                rot=Rotation.from_dict(raw.get("rot"), where + ".rot"), chunk=_mask_size(raw, where))
        if c.heads <= 0 or c.kv_heads <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"{where}.kv_heads: {c.heads} heads do not divide into {c.kv_heads} key/value heads")
        if c.dim <= 0 or c.vdim <= 0 or c.rot.dims > c.dim:
            raise ConfigError(f"{where}: dim and vdim are positive, rot.dims at most dim")
        return c

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.chunk:
            out["mask"] = {"size": self.chunk}
        if self.rot.dims:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class BafaraxLatentAttention:
    heads: int
    dim: int                     # unrotated query / key dimensions of a head
    rot_dim: int                 # rotated ones; the key's are shared by all heads
    vdim: int
    kv_rank: int                 # size of the latent that keys and values are made from
    q_rank: int                  # size of the queries' latent
    scale: float
    rot: Rotation                # pairs (2i, 2i + 1) of the rotated part
    window: int                  # a position sees itself and the window - 1 before it (0: all before it)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "BafaraxLatentAttention":
        c = cls(heads=int(_need(raw, "heads", where)), dim=int(_need(raw, "dim", where)), rot_dim=int(_need(raw, "rot_dim", where)),
                vdim=int(_need(raw, "vdim", where)), kv_rank=int(_need(raw, "kv_rank", where)), q_rank=int(_need(raw, "q_rank", where)),
                scale=float(_need(raw, "scale", where)), rot=Rotation.from_dict(raw.get("rot"), where + ".rot"),
                window=_mask_size(raw, where))
        if min(c.heads, c.dim, c.vdim, c.kv_rank, c.q_rank) <= 0 or c.rot_dim < 0:
            raise ConfigError(f"{where}: heads, dim, vdim, kv_rank and q_rank are positive")
        if c.rot.dims != c.rot_dim:
            raise ConfigError(f"{where}.rot.dims {c.rot.dims}: the whole rotated part of {c.rot_dim} turns")
        return c

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
                               "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.rot.dims:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class BafaraxMLSTM:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "BafaraxMLSTM":
        c = cls(heads=int(_need(raw, "heads", where)), dim=int(_need(raw, "dim", where)), vdim=int(_need(raw, "vdim", where)),
                gate_cap=float(_need(raw, "gate_cap", where)))
        if min(c.heads, c.dim, c.vdim) <= 0 or c.gate_cap <= 0:
            raise ConfigError(f"{where}: heads, dim, vdim and gate_cap are positive")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"dim": self.dim, "gate_cap": self.gate_cap, "heads": self.heads, "vdim": self.vdim}


MIXERS = {"attention": BafaraxAttention, "latent_attention": BafaraxLatentAttention, "mlstm": BafaraxMLSTM}


@dataclass(frozen=True)
class BafaraxDense:
    ff: int

    def to_dict(self) -> dict[str, Any]:
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class BafaraxExperts:
    experts: int
    top: int
    ff: int                      # width of one expert

    def to_dict(self) -> dict[str, Any]:
        return {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}


def _mlp(raw: Mapping[str, Any] | None, where: str) -> "BafaraxDense | BafaraxExperts | None":
    if raw is None:
        return None
    kind = _need(raw, "kind", where)
    if kind == "dense":
        c = BafaraxDense(ff=int(_need(raw, "ff", where)))
        if c.ff <= 0:
            raise ConfigError(f"{where}.ff: positive")
        return c
    if kind == "moe":
        router = _need(raw, "router", where)
        e = BafaraxExperts(experts=int(_need(router, "experts", where + ".router")), top=int(_need(router, "top", where + ".router")),
                           ff=int(_need(_need(raw, "expert", where), "ff", where + ".expert")))
        if e.ff <= 0 or not 1 <= e.top <= e.experts:
            raise ConfigError(f"{where}: a positive expert.ff, and router.top between 1 and the {e.experts} experts")
        return e
    raise ConfigError(f"{where}.kind {kind!r}: 'dense' or 'moe'")


@dataclass(frozen=True)
class BafaraxLayer:
    type: str
    mixer: "BafaraxAttention | BafaraxLatentAttention | BafaraxMLSTM"
    mlp: "BafaraxDense | BafaraxExperts | None"
    weights_of: int | None = None        # the earlier layer whose weights this one runs with (None: its own)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "BafaraxLayer":
        kind = _need(raw, "type", where)
        if kind not in MIXERS:
            raise ConfigError(f"{where}.type {kind!r}: one of {sorted(MIXERS)}")
        shared = raw.get("weights_of")
        return cls(kind, MIXERS[kind].from_dict(_need(raw, "mixer", where), where + ".mixer"), _mlp(raw.get("mlp"), where + ".mlp"),
                   None if shared is None else int(shared))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


@dataclass(frozen=True)
class BafaraxConfig:
    vocab: int
    width: int
    layers: tuple[BafaraxLayer, ...]
    norm_eps: float
    embedding_scale: float = 1.0
    architecture: str = "Bafarax"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "BafaraxConfig":
        layers = tuple(BafaraxLayer.from_dict(l, f"layers[{i}]") for i, l in enumerate(_need(raw, "layers", "config.json")))
        if not layers:
            raise ConfigError("layers: the model has at least one")
        for i, layer in enumerate(layers):
            j = layer.weights_of
            if j is None:
                continue
            if not 0 <= j < i or layers[j].weights_of is not None:
                raise ConfigError(f"layers[{i}].weights_of {j}: an earlier layer with weights of its own")
            if (layers[j].type, layers[j].mixer, layers[j].mlp) != (layer.type, layer.mixer, layer.mlp):
                raise ConfigError(f"layers[{i}].weights_of {j}: the two layers' entries differ")
        embedding = raw.get("embedding") or {}
        c = cls(vocab=int(_need(raw, "vocab", "config.json")), width=int(_need(raw, "width", "config.json")), layers=layers,
                norm_eps=float(_need(_need(raw, "norm", "config.json"), "eps", "norm")),
                embedding_scale=float(embedding.get("scale", 1.0)))
        if c.vocab <= 0 or c.width <= 0 or c.norm_eps < 0:
            raise ConfigError("vocab and width are positive, norm.eps is not negative")
        return c

    def to_dict(self) -> dict[str, Any]:
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
                "width": self.width}
